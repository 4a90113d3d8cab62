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
    # 64 x 32 heads over 16384 columns: 129 splits x 2048 heads x 130 floats >> 4 MiB
    case = StateCase("too large", 64, 32, 8, 1, 128, 16384, 0, 16383, 1)
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
