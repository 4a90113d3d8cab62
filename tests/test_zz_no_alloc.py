"""The decode attention's entry point that allocates nothing (krm_attention_state_noalloc):
through the C ABI, against krm_attention_state on the same inputs, bit for bit, on two calls
in a row of which the second is smaller (the built-in scratch keeps the first call's partials
and counters); then a call beyond the built-in scratch, which must be rejected with a clear
error and leave the entry point usable."""
import numpy as np
import pytest

import karume_amd as ka
from helpers import StateCase, oracle
from test_gpu_attention import random_state_inputs, run_attention

pytestmark = pytest.mark.gpu


def run_noalloc(ctx, case, x, io, kv):
    bufs = {k: ctx.upload(np.ascontiguousarray(v, dtype=io if k in ("q", "ins_k", "ins_v") else kv))
            for k, v in x.items()}
    out_elems = case.batch * case.heads * case.chunk_rows * case.depth
    out = ctx.upload(np.full(out_elems, 123.0, dtype=io))  # every element must be overwritten
    ctx.attention_state_noalloc(
        bufs["q"], bufs["ins_k"], bufs["ins_v"], bufs["slot_k"], bufs["slot_v"], out,
        half_scale=oracle.half_scale(case.depth), io_dtype=ka.dtype_code(io),
        kv_dtype=ka.dtype_code(kv), **case.kwargs())
    got = out.download(io, (case.batch, case.heads, case.chunk_rows, case.depth))
    for b in list(bufs.values()) + [out]:
        b.free()
    return got


CASES = [
    # many splits (32 x 128 columns), GQA 4:1, fp16: config 2's shape
    (StateCase("config 2", 1, 32, 8, 1, 128, 4096, 0, 4095, 1), np.float16, np.float16),
    # smaller: 6 splits, batch 2, f32 in / fp16 slots
    (StateCase("B2 P700", 2, 8, 2, 1, 128, 1024, 0, 700, 1), np.float32, np.float16),
    # one split (no partials at all) and a prefill chunk through the generic kernel
    (StateCase("one split", 1, 4, 4, 1, 64, 512, 0, 300, 1), np.float32, np.float32),
    (StateCase("prefill chunk", 1, 4, 2, 6, 32, 64, 0, 5, 4), np.float32, np.float32),
    # many splits again after the small ones
    (StateCase("sliding W3000", 1, 8, 8, 1, 128, 3000, 3000, 9000, 1), np.float16, np.float16),
]


def test_noalloc_equals_attention_state_bitwise_on_calls_in_a_row(gpu_ctx):
    for case, io, kv in CASES:
        x = random_state_inputs(case, seed=case.past + case.depth, f16_values=True)
        want = run_attention(gpu_ctx, case, x, io=io, kv=kv)
        got = run_noalloc(gpu_ctx, case, x, io, kv)
        assert np.all(np.isfinite(got.astype(np.float32))), case.name
        assert got.tobytes() == want.tobytes(), case.name


def test_noalloc_rejects_what_its_scratch_cannot_hold(gpu_ctx):
    # 128 heads over 16384 columns: 128 splits x 128 heads x 130 floats = 8.5 MB > 4 MiB
    case = StateCase("too large", 1, 128, 32, 1, 128, 16384, 0, 16383, 1)
    tiny = gpu_ctx.alloc(64)
    with pytest.raises(ka.GpuValidationError, match="built-in scratch"):
        gpu_ctx.attention_state_noalloc(tiny, tiny, tiny, tiny, tiny, tiny,
                                        half_scale=0.3, io_dtype=ka.F16, kv_dtype=ka.F16,
                                        **case.kwargs())
    tiny.free()
    # still usable afterwards
    case, io, kv = CASES[1]
    x = random_state_inputs(case, seed=5, f16_values=True)
    assert run_noalloc(gpu_ctx, case, x, io, kv).tobytes() == \
        run_attention(gpu_ctx, case, x, io=io, kv=kv).tobytes()


def test_noalloc_without_scratch_needs_runs_whatever_the_size(gpu_ctx):
    """Calls that need no scratch are never measured against it: a prefill chunk with many
    heads (the chunk kernels keep everything in the workgroup), and a decode step with more
    (batch, head) pairs than the built-in array has arrival counters, which takes the generic
    kernel; both against the CPU oracle at the reference's gate (atol 5e-6)."""
    from helpers import oracle_state_attention
    for case in (StateCase("chunk, 96 x 8 heads", 96, 8, 2, 4, 64, 64, 0, 7, 3),
                 StateCase("decode, 640 (batch, head) pairs", 40, 16, 4, 1, 64, 256, 0, 200, 1)):
        x = random_state_inputs(case, seed=3, f16_values=True)
        got = run_noalloc(gpu_ctx, case, x, np.float32, np.float32)
        want = oracle_state_attention(case, x)
        ok, fails, max_abs, worst = oracle.allclose(got, want, atol=5e-6, rtol=0)
        assert ok, (case.name, fails, max_abs, worst)


def test_noalloc_recorded_in_a_graph_replays_to_the_eager_result(gpu_ctx):
    """The entry may sit inside a recorded sequence (its scratch address is resolved when the
    context is created, its counters are cleared by a fill kernel): three replays with eager
    work and synchronisations between them, each equal to the eager call bit for bit."""
    case, io, kv = CASES[0]
    x = random_state_inputs(case, seed=21, f16_values=True)
    want = run_attention(gpu_ctx, case, x, io=io, kv=kv)
    bufs = {k: gpu_ctx.upload(np.ascontiguousarray(v, dtype=io if k in ("q", "ins_k", "ins_v") else kv))
            for k, v in x.items()}
    out = gpu_ctx.alloc(want.nbytes)
    with gpu_ctx.record() as rec:
        gpu_ctx.attention_state_noalloc(
            bufs["q"], bufs["ins_k"], bufs["ins_v"], bufs["slot_k"], bufs["slot_v"], out,
            half_scale=oracle.half_scale(case.depth), io_dtype=ka.dtype_code(io),
            kv_dtype=ka.dtype_code(kv), **case.kwargs())
    for replay in range(3):
        out.zero()
        # eager use of the same scratch between replays (a smaller call)
        small, sio, skv = CASES[1]
        run_noalloc(gpu_ctx, small, random_state_inputs(small, seed=replay, f16_values=True),
                    sio, skv)
        rec.graph.launch()
        gpu_ctx.sync()
        assert out.download(io, want.shape).tobytes() == want.tobytes(), replay
    rec.graph.destroy()
    for b in list(bufs.values()) + [out]:
        b.free()
