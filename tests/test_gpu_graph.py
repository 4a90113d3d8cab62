"""Recorded launch sequences with parallel branches (krm_graph_begin / krm_graph_branch /
krm_graph_end): independent ops recorded on different branches give, on every replay, the bits
of the same ops run one after the other; ops that use the context's own scratch (which assumes
launch order) are rejected while a side branch is selected and leave the recording usable."""
import numpy as np
import pytest

import helpers
import karume_amd as ka
from helpers import StateCase, oracle
from test_gpu_attention import random_state_inputs, run_attention

pytestmark = pytest.mark.gpu


def test_ops_on_two_side_branches_equal_the_serial_result_bitwise(gpu_ctx):
    ctx = gpu_ctx
    rng = np.random.default_rng(77)
    n, k, g = 1536, 2048, 128
    problems = []
    for _ in range(3):  # main branch, side branch 1, side branch 2
        packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
        x = rng.normal(size=(1, k)).astype(np.float16)
        problems.append(dict(x=ctx.upload(x), w=ctx.upload(packed), s=ctx.upload(scale),
                             out=ctx.alloc(n * 2), serial=None))

    def gemv(p):
        ctx.linear_i4(p["x"], p["w"], p["s"], None, p["out"], 1, n, k, g, ka.F16, ka.F16)

    for p in problems:
        gemv(p)
        p["serial"] = p["out"].download(np.float16, (n,)).tobytes()
        p["out"].zero()
    with ctx.record() as rec:
        gemv(problems[0])
        rec.branch(1)
        gemv(problems[1])
        rec.branch(2)
        gemv(problems[2])
        rec.branch(0)
    graph = rec.graph
    for replay in range(3):
        for p in problems:
            p["out"].zero()
        ctx.sync()  # the program's own eager work and a synchronisation between replays
        graph.launch()
        ctx.sync()
        for index, p in enumerate(problems):
            assert p["out"].download(np.float16, (n,)).tobytes() == p["serial"], (replay, index)
    graph.destroy()
    for p in problems:
        for name in ("x", "w", "s", "out"):
            p[name].free()


def test_scratch_users_are_rejected_on_a_side_branch(gpu_ctx):
    """The split decode attention merges through the context's arrival counters: on a side
    branch it fails with a validation error and records nothing; the same call on the main
    branch of the same recording is accepted and replays to the eager result."""
    ctx = gpu_ctx
    case = StateCase("config 2", 1, 32, 8, 1, 128, 4096, 0, 4095, 1)
    x = random_state_inputs(case, seed=11, f16_values=True)
    want = run_attention(ctx, case, x, io=np.float16, kv=np.float16)
    bufs = {name: ctx.upload(np.ascontiguousarray(v, dtype=np.float16)) for name, v in x.items()}
    out = ctx.alloc(want.nbytes)
    ws = ctx.alloc(ctx.attention_state_workspace(1, 32, 8, 1, 128, 0, 4095))

    def attention():
        ctx.attention_state(bufs["q"], bufs["ins_k"], bufs["ins_v"], bufs["slot_k"],
                            bufs["slot_v"], out, half_scale=oracle.half_scale(128),
                            io_dtype=ka.F16, kv_dtype=ka.F16, workspace=ws, **case.kwargs())

    # an f32-class MFMA product (row scales in the context's scratch)
    rng = np.random.default_rng(5)
    m, n, k, g = 64, 256, 512, 128
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    dx = ctx.upload(rng.normal(size=(m, k)).astype(np.float32))
    dw, ds, dout = ctx.upload(packed), ctx.upload(scale), ctx.alloc(m * n * 4)

    with ctx.record() as rec:
        rec.branch(1)
        with pytest.raises(ka.GpuValidationError, match="main branch"):
            attention()
        with pytest.raises(ka.GpuValidationError, match="main branch"):
            ctx.linear_i4(dx, dw, ds, None, dout, m, n, k, g, ka.F32, ka.F16, ka.COMPUTE_F32)
        rec.branch(0)
        attention()
    out.zero()
    rec.graph.launch()
    ctx.sync()
    assert out.download(np.float16, want.shape).tobytes() == want.tobytes()
    rec.graph.destroy()
    for b in list(bufs.values()) + [out, ws, dx, dw, ds, dout]:
        b.free()
