"""GPU parity of states-form attention, state_append and the ragged decode batch (through the
C ABI) against the CPU oracle."""
import numpy as np
import pytest

import helpers
import karume_amd as ka
from helpers import PARITY_CASES, StateCase, make_state_inputs, oracle, oracle_state_attention

pytestmark = pytest.mark.gpu

# The reference's own gate for this op: atol 5e-6, rtol 0, outputs O(1)
# (packages/runtime/tests/gpu_state_attention_test.ts:41-54; its measured worst is 6.6e-7).
STATE_ATOL = 5e-6


def run_attention(ctx, case: StateCase, x: dict, io=np.float32, kv=np.float32, scale=None,
                  workspace_bytes=None):
    bufs = {k: ctx.upload(np.ascontiguousarray(v, dtype=io if k in ("q", "ins_k", "ins_v") else kv))
            for k, v in x.items()}
    out_elems = case.batch * case.heads * case.chunk_rows * case.depth
    out = ctx.upload(np.full(out_elems, 123.0, dtype=io))  # every element must be overwritten
    ws_bytes = ctx.attention_state_workspace(case.batch, case.heads, case.kv_heads,
                                             case.chunk_rows, case.depth, case.window,
                                             min(case.past, 1 << 20), case.query)
    if workspace_bytes is not None:
        ws_bytes = workspace_bytes
    ws = ctx.alloc(max(ws_bytes, 16))
    ctx.attention_state(
        bufs["q"], bufs["ins_k"], bufs["ins_v"], bufs["slot_k"], bufs["slot_v"], out,
        half_scale=oracle.half_scale(case.depth) if scale is None else scale,
        io_dtype=ka.dtype_code(io), kv_dtype=ka.dtype_code(kv), workspace=ws,
        workspace_bytes=ws_bytes, **case.kwargs())
    got = out.download(io, (case.batch, case.heads, case.chunk_rows, case.depth))
    for b in list(bufs.values()) + [out, ws]:
        b.free()
    return got


@pytest.mark.parametrize("case", PARITY_CASES, ids=lambda c: c.name)
def test_parity_grid(gpu_ctx, case):
    """The reference's 17-case grid with poison in every place that must not be read
    (gpu_state_attention_test.ts:119-347): atol 5e-6 rtol 0, pad rows exact +0."""
    x = make_state_inputs(case)
    want = oracle_state_attention(case, x)
    got = run_attention(gpu_ctx, case, x)
    ok, fails, max_abs, worst = oracle.allclose(got, want, atol=STATE_ATOL, rtol=0)
    assert ok, (fails, max_abs, worst)
    pad = got[:, :, case.query:, :]
    assert np.all(pad == 0.0) and not np.any(np.signbit(pad))


DECODE_CASES = [
    StateCase("decode r4 D128 P300", 1, 8, 2, 1, 128, 512, 0, 300, 1),
    StateCase("decode r4 D128 P127 one split", 2, 8, 2, 1, 128, 128, 0, 127, 1),
    StateCase("decode r4 D128 P128 boundary", 1, 8, 2, 1, 128, 256, 0, 128, 1),
    StateCase("decode r8 D64 P383", 1, 32, 4, 1, 64, 512, 0, 383, 1),
    StateCase("decode r1 D64 P0", 1, 4, 4, 1, 64, 16, 0, 0, 1),
    StateCase("decode r1 D128 P700 six splits", 1, 4, 4, 1, 128, 1024, 0, 700, 1),
    StateCase("decode r1 D64 P300 chunks together", 1, 4, 4, 1, 64, 512, 0, 300, 1),
    StateCase("decode r2 D32 B3 P77", 3, 4, 2, 1, 32, 96, 0, 77, 1),
    StateCase("decode sliding W100 P1000 C128", 1, 8, 2, 1, 128, 128, 100, 1000, 1),
    StateCase("decode sliding W300 P299", 1, 8, 2, 1, 64, 300, 300, 299, 1),
    StateCase("decode sliding W256 P5000", 2, 8, 8, 1, 64, 256, 256, 5000, 1),
]


def random_state_inputs(case: StateCase, seed: int, f16_values: bool):
    rng = np.random.default_rng(seed)
    b, h, hkv, m, d, c = (case.batch, case.heads, case.kv_heads, case.chunk_rows, case.depth,
                          case.capacity)
    x = dict(q=rng.normal(size=(b, h, m, d)), ins_k=rng.normal(size=(b, hkv, m, d)),
             ins_v=rng.normal(size=(b, hkv, m, d)), slot_k=rng.normal(size=(b, hkv, c, d)),
             slot_v=rng.normal(size=(b, hkv, c, d)))
    cast = (lambda a: a.astype(np.float16).astype(np.float32)) if f16_values else \
        (lambda a: a.astype(np.float32))
    x = {k: cast(v) for k, v in x.items()}
    # poison what must not be read: non-resident slot rows
    base = oracle.state_column_base(case.window, case.past)
    resident = {col % case.window if case.window else col for col in range(base, case.past)}
    for row in range(c):
        if row not in resident:
            x["slot_k"][:, :, row] = 9.0
            x["slot_v"][:, :, row] = 400.0
    return x


@pytest.mark.parametrize("case", DECODE_CASES, ids=lambda c: c.name)
@pytest.mark.parametrize("io,kv", [(np.float32, np.float32), (np.float16, np.float16),
                                   (np.float32, np.float16)])
def test_decode_split_k(gpu_ctx, case, io, kv):
    """The split-K decode path (Q = 1, M = 1) over one or several splits, full and sliding.
    f32 output: atol 5e-6 rtol 0 (the reference's gate).  fp16 output: the oracle's value
    rounded to fp16, +-1 fp16 ulp."""
    x = random_state_inputs(case, seed=case.past + case.depth, f16_values=True)
    want = oracle_state_attention(case, x)
    got = run_attention(gpu_ctx, case, x, io=io, kv=kv)
    if io == np.float32:
        ok, fails, max_abs, worst = oracle.allclose(got, want, atol=STATE_ATOL, rtol=0)
        assert ok, (fails, max_abs, worst)
    else:
        want16 = want.astype(np.float16)
        ulp = np.abs(np.nextafter(want16, np.float16(np.inf)).astype(np.float32)
                     - want16.astype(np.float32))
        err = np.abs(got.astype(np.float32) - want16.astype(np.float32))
        assert np.all(err <= ulp), float(np.max(err))


ROWS_CASES = [
    # chunks of rows with D = 64 / 128: the matrix-core form (16 query rows a workgroup, key
    # blocks of 32 dealt to the waves: eight for D = 64, four for D = 128)
    StateCase("rows D64 M128 P0 r8 (decoder prefill)", 1, 32, 4, 128, 64, 256, 0, 0, 128),
    StateCase("rows D64 M40 Q33 P100 pad + slot/ins straddle", 2, 8, 2, 40, 64, 192, 0, 100, 33),
    StateCase("rows D128 M64 P31 r1", 1, 4, 4, 64, 128, 128, 0, 31, 64),
    StateCase("rows D128 M33 Q2 P0", 1, 2, 1, 33, 128, 64, 0, 0, 2),
    StateCase("rows D64 sliding W48 P200 wrap", 2, 4, 2, 70, 64, 48, 48, 200, 70),
    StateCase("rows D64 sliding W16 M64 Q50 gt W", 1, 4, 4, 64, 64, 16, 16, 7, 50),
    StateCase("rows D128 sliding W100 C128 P1000", 1, 8, 2, 35, 128, 128, 100, 1000, 20),
    StateCase("rows D64 M2 Q1 P5", 1, 4, 2, 2, 64, 16, 0, 5, 1),
    # more key blocks than waves, D = 64
    StateCase("rows D64 M64 P300, 12 blocks", 1, 8, 2, 64, 64, 512, 0, 300, 64),
    StateCase("rows D64 M40 Q37 P1000, 33 blocks", 2, 4, 1, 40, 64, 1100, 0, 1000, 37),
    StateCase("rows D64 sliding W300 P900", 1, 4, 2, 48, 64, 300, 300, 900, 48),
]


@pytest.mark.parametrize("case", ROWS_CASES, ids=lambda c: c.name)
@pytest.mark.parametrize("io,kv", [(np.float32, np.float32), (np.float16, np.float16),
                                   (np.float32, np.float16)])
def test_chunks_of_rows_on_the_matrix_cores(gpu_ctx, case, io, kv):
    """M > 1 with D = 64 / 128 (f32 MFMA, online softmax per lane): the reference's gate for
    f32 output (atol 5e-6, rtol 0); for fp16 output the same gate plus one fp16 ulp of the
    oracle's value (the rounding of the stored result); pad rows exact +0; poison in every slot
    row that must not be read and in the ins pad rows."""
    x = random_state_inputs(case, seed=case.past + case.depth + case.chunk_rows, f16_values=True)
    x["ins_k"][:, :, case.query:] = 9.0
    x["ins_v"][:, :, case.query:] = 400.0
    want = oracle_state_attention(case, x)
    got = run_attention(gpu_ctx, case, x, io=io, kv=kv)
    pad = got[:, :, case.query:, :]
    assert np.all(pad == 0.0) and not np.any(np.signbit(pad))
    if io == np.float32:
        ok, fails, max_abs, worst = oracle.allclose(got, want, atol=STATE_ATOL, rtol=0)
        assert ok, (fails, max_abs, worst)
    else:
        want16 = want.astype(np.float16)
        ulp = np.abs(np.nextafter(want16, np.float16(np.inf)).astype(np.float32)
                     - want16.astype(np.float32))
        err = np.abs(got.astype(np.float32) - want16.astype(np.float32))
        assert np.all(err <= ulp + STATE_ATOL), float(np.max(err - ulp))


def test_chunk_rows_do_not_depend_on_the_batch(gpu_ctx):
    """A large grid puts two blocks of 16 query rows into one workgroup (the parked K / V blocks
    serve both); a row's arithmetic is the same, so one sequence alone and the same sequence as
    the first of eight give the same bits."""
    big = StateCase("rows D64 M64 P70 B8", 8, 32, 32, 64, 64, 160, 0, 70, 61)
    x = random_state_inputs(big, seed=3, f16_values=False)
    whole = run_attention(gpu_ctx, big, x)
    one = StateCase("rows D64 M64 P70 B1", 1, 32, 32, 64, 64, 160, 0, 70, 61)
    first = {k: np.ascontiguousarray(v[:1]) for k, v in x.items()}
    alone = run_attention(gpu_ctx, one, first)
    assert np.array_equal(alone.view(np.uint32), whole[:1].view(np.uint32))
    ok, fails, max_abs, worst = oracle.allclose(alone, oracle_state_attention(one, first),
                                                atol=STATE_ATOL, rtol=0)
    assert ok, (fails, max_abs, worst)


def test_chunks_of_rows_with_device_lengths_and_mutation_witness(gpu_ctx):
    """The device-lengths form of a chunk equals the scalar form bit for bit, and a dropped
    window bound, a ring taken modulo the capacity, or an ignored kv repeat (the oracle's
    mutations) would each be seen at this gate."""
    case = StateCase("rows D64 sliding W40 C48 P200 Q33", 2, 8, 2, 40, 64, 48, 40, 200, 33)
    x = random_state_inputs(case, seed=5, f16_values=False)
    got = run_attention(gpu_ctx, case, x)
    want = oracle_state_attention(case, x)
    ok, fails, max_abs, worst = oracle.allclose(got, want, atol=STATE_ATOL, rtol=0)
    assert ok, (fails, max_abs, worst)
    for mutation in (oracle.MUT_DROP_LOWER_BOUND, oracle.MUT_RING_MOD_CAPACITY,
                     oracle.MUT_IGNORE_KV_REPEAT):
        wrong = oracle_state_attention(case, x, mutation=mutation)
        assert not oracle.allclose(got, wrong, atol=STATE_ATOL, rtol=0)[0], mutation
    bufs = {k: gpu_ctx.upload(np.ascontiguousarray(v, dtype=np.float32)) for k, v in x.items()}
    out = gpu_ctx.upload(np.full(got.size, 7.0, dtype=np.float32))
    lengths = gpu_ctx.zeros(16)
    gpu_ctx.lengths_set(lengths, case.past, case.query)
    spec = {k: v for k, v in case.kwargs().items() if k not in ("past", "query")}
    gpu_ctx.attention_state_lengths(bufs["q"], bufs["ins_k"], bufs["ins_v"], bufs["slot_k"],
                                    bufs["slot_v"], out, half_scale=oracle.half_scale(case.depth),
                                    lengths=lengths, max_past=case.capacity - 1, **spec)
    again = out.download(np.float32, got.shape)
    assert np.array_equal(again.view(np.uint32), got.view(np.uint32))
    assert lengths.download(np.uint32, (4,))[2] == 0


@pytest.mark.parametrize("case", DECODE_CASES, ids=lambda c: c.name)
@pytest.mark.parametrize("io,kv", [(np.float32, np.float32), (np.float16, np.float16)])
def test_decode_with_device_lengths_equals_scalar_form(gpu_ctx, case, io, kv):
    """pastLength read on the device (a recorded decode step) gives the bits of the call that
    carries it as an argument.  Without a window the device form asks for the first chunk's
    rows before the lengths arrive, bounded by the capacity only: every slot row the step must
    not see (columns >= pastLength) holds NaN here and must not reach the result."""
    x = random_state_inputs(case, seed=case.past * 3 + case.depth, f16_values=True)
    if case.window == 0:
        x["slot_k"][:, :, case.past:] = np.nan
        x["slot_v"][:, :, case.past:] = np.nan
    want = run_attention(gpu_ctx, case, x, io=io, kv=kv)
    assert np.all(np.isfinite(want.astype(np.float32)))
    bufs = {k: gpu_ctx.upload(np.ascontiguousarray(
        v, dtype=io if k in ("q", "ins_k", "ins_v") else kv)) for k, v in x.items()}
    out = gpu_ctx.upload(np.full(want.size, 123.0, dtype=io))
    max_past = case.past if case.window else case.capacity - 1
    ws = gpu_ctx.alloc(max(16, gpu_ctx.attention_state_workspace(
        case.batch, case.heads, case.kv_heads, 1, case.depth, case.window, max_past, 1)))
    lengths = gpu_ctx.zeros(16)
    gpu_ctx.lengths_set(lengths, case.past, 1)
    gpu_ctx.attention_state_lengths(
        bufs["q"], bufs["ins_k"], bufs["ins_v"], bufs["slot_k"], bufs["slot_v"], out,
        batch=case.batch, heads=case.heads, kv_heads=case.kv_heads, chunk_rows=1,
        depth=case.depth, capacity=case.capacity, window=case.window,
        half_scale=oracle.half_scale(case.depth), lengths=lengths, max_past=max_past,
        io_dtype=ka.dtype_code(io), kv_dtype=ka.dtype_code(kv), workspace=ws)
    got = out.download(io, want.shape)
    assert lengths.download(np.uint32, (4,))[2] == 0
    assert got.tobytes() == want.tobytes()
    for b in list(bufs.values()) + [out, ws, lengths]:
        b.free()


@pytest.mark.parametrize("max_past,device_past", [(600, 900), (100, 700)])
def test_replay_beyond_the_sized_past_raises_the_fault_word(gpu_ctx, max_past, device_past):
    """A launch sized for `max_past` (5 splits, or a single split without a workspace) meets a
    device-side pastLength that needs more splits: the fault word is raised, `out` keeps its
    bytes, and the arrival counters stay clean — the same launch with a legal pastLength
    afterwards still equals the scalar form bitwise.  Every workgroup exits normally."""
    case = StateCase("guard", 1, 8, 2, 1, 128, 1024, 0, device_past, 1)
    x = random_state_inputs(case, seed=11, f16_values=True)
    io = kv = np.float16
    bufs = {k: gpu_ctx.upload(np.ascontiguousarray(v, dtype=np.float16)) for k, v in x.items()}
    sentinel = np.full(case.heads * case.depth, 123.0, dtype=io)
    out = gpu_ctx.upload(sentinel)
    ws = gpu_ctx.alloc(max(16, gpu_ctx.attention_state_workspace(
        1, case.heads, case.kv_heads, 1, case.depth, 0, max_past, 1)))
    lengths = gpu_ctx.zeros(16)

    def launch():
        gpu_ctx.attention_state_lengths(
            bufs["q"], bufs["ins_k"], bufs["ins_v"], bufs["slot_k"], bufs["slot_v"], out,
            batch=1, heads=case.heads, kv_heads=case.kv_heads, chunk_rows=1, depth=case.depth,
            capacity=case.capacity, window=0, half_scale=oracle.half_scale(case.depth),
            lengths=lengths, max_past=max_past, io_dtype=ka.F16, kv_dtype=ka.F16,
            workspace=ws if max_past > 512 else None)

    gpu_ctx.lengths_set(lengths, device_past, 1)
    launch()
    state = lengths.download(np.uint32, (4,))
    assert state[2] == 1 and state[0] == device_past
    assert out.download(io, sentinel.shape).tobytes() == sentinel.tobytes()
    # a legal pastLength through the same launch shape afterwards
    legal = StateCase("legal", 1, 8, 2, 1, 128, 1024, 0, max_past, 1)
    want = run_attention(gpu_ctx, legal, x, io=io, kv=kv)
    gpu_ctx.lengths_set(lengths, max_past, 1)
    launch()
    assert lengths.download(np.uint32, (4,))[2] == 0
    assert out.download(io, want.shape).tobytes() == want.tobytes()
    for b in list(bufs.values()) + [out, ws, lengths]:
        b.free()


def test_config2_decode_attention(gpu_ctx):
    """benchmark config 2: B=1, H=32, Hkv=8, D=128, 4095 slot rows + this step's row, fp16."""
    case = StateCase("config 2", 1, 32, 8, 1, 128, 4096, 0, 4095, 1)
    x = random_state_inputs(case, seed=2, f16_values=True)
    want = oracle_state_attention(case, x)
    got32 = run_attention(gpu_ctx, case, x, io=np.float32, kv=np.float16)
    ok, fails, max_abs, worst = oracle.allclose(got32, want, atol=STATE_ATOL, rtol=0)
    assert ok, (fails, max_abs, worst)
    got16 = run_attention(gpu_ctx, case, x, io=np.float16, kv=np.float16)
    want16 = want.astype(np.float16).astype(np.float32)
    assert np.max(np.abs(got16.astype(np.float32) - want16)) <= 2.5e-4  # 1 ulp at |out| < 0.25
    # identical bits for a larger capacity: the work never depends on C
    big = StateCase("config 2 C8192", 1, 32, 8, 1, 128, 8192, 0, 4095, 1)
    xb = {k: v.copy() for k, v in x.items()}
    for name in ("slot_k", "slot_v"):
        grown = np.full((1, 8, 8192, 128), 9.0 if name == "slot_k" else 400.0, dtype=np.float32)
        grown[:, :, :4096] = x[name]
        xb[name] = grown
    got_big = run_attention(gpu_ctx, big, xb, io=np.float32, kv=np.float16)
    assert np.array_equal(got_big.view(np.uint32), got32.view(np.uint32))


def test_mutations_would_be_caught(gpu_ctx):
    """The GPU result sits within tolerance of the faithful oracle and far from every mutated
    oracle on that mutation's witness case."""
    witnesses = {
        oracle.MUT_DROP_LOWER_BOUND: "sliding W4 P10 wrap",
        oracle.MUT_RING_MOD_CAPACITY: "sliding W4 C8 wrap",
        oracle.MUT_PAD_ROWS_COMPUTED: "full r2 pad B2 D6",
        oracle.MUT_IGNORE_KV_REPEAT: "full r2 pad B2 D6",
        oracle.MUT_SCALE_ONE_SIDE: "full r1 prefill B2",
        oracle.MUT_OVERFLOW_FORM: "sliding W2 P near u32 max",
    }
    for mutation, name in witnesses.items():
        case = next(c for c in PARITY_CASES if c.name == name)
        x = make_state_inputs(case)
        got = run_attention(gpu_ctx, case, x)
        bad = oracle_state_attention(case, x, mutation=mutation)
        assert np.max(np.abs(got - bad)) > 1e-3, name


def test_attention_rejections(gpu_ctx):
    buf = gpu_ctx.zeros(1 << 16)
    base = dict(batch=1, heads=4, kv_heads=2, chunk_rows=2, depth=8, capacity=8, window=0,
                half_scale=0.5, past=0, query=1)
    call = lambda **kw: gpu_ctx.attention_state(buf, buf, buf, buf, buf, buf,  # noqa: E731
                                                **{**base, **kw})
    with pytest.raises(ka.GpuValidationError):
        call(heads=3)
    with pytest.raises(ka.GpuValidationError):
        call(window=9)
    with pytest.raises(ka.ExecutionError):  # capacity overflow is rejected before launch
        call(past=7, query=2)
    with pytest.raises(ka.ExecutionError):
        call(query=3)
    with pytest.raises(ka.ExecutionError):
        call(query=0)
    with pytest.raises(ka.GpuValidationError):
        call(half_scale=float("nan"))
    # split-K needs a workspace when there is more than one split
    big = dict(batch=1, heads=8, kv_heads=2, chunk_rows=1, depth=128, capacity=4096, window=0,
               half_scale=0.3, past=4000, query=1, io_dtype=ka.F16, kv_dtype=ka.F16)
    huge = gpu_ctx.zeros(2 * 4096 * 128 * 2)
    with pytest.raises(ka.GpuValidationError):
        gpu_ctx.attention_state(buf, buf, buf, huge, huge, buf, **big)
    huge.free()
    buf.free()


# ---------------------------------------------------------------------------- state_append

def run_append(ctx, x, slot, xd=np.float32, sd=np.float32, **spec):
    dx = ctx.upload(np.ascontiguousarray(x, dtype=xd))
    ds = ctx.upload(np.ascontiguousarray(slot, dtype=sd))
    ctx.state_append(dx, ds, x_dtype=ka.dtype_code(xd), slot_dtype=ka.dtype_code(sd), **spec)
    got = ds.download(sd, np.shape(slot))
    dx.free()
    ds.free()
    return got


def test_append_reference_vectors(gpu_ctx):
    # packages/runtime/tests/kernel_state_attention_test.ts:481-503
    spec = dict(kv_planes=1, chunk_rows=4, depth=1, capacity=4, window=4)
    slot = np.array([-1, -2, -3, -4], dtype=np.float32)
    x = np.array([100, 200, 300, 400], dtype=np.float32)
    assert run_append(gpu_ctx, x, slot, past=2, query=2, **spec).tolist() == [-1, -2, 100, 200]
    assert run_append(gpu_ctx, x, slot, past=3, query=3, **spec).tolist() == [200, 300, -3, 100]
    collide = run_append(gpu_ctx, x, np.array([-1, -2], dtype=np.float32), kv_planes=1,
                         chunk_rows=4, depth=1, capacity=2, window=2, past=0, query=4)
    assert collide.tolist() == [300, 400]


@pytest.mark.parametrize("window,capacity,past,query,m", [(0, 64, 5, 7, 9), (6, 6, 13, 3, 5),
                                                          (4, 8, 9, 2, 3), (2, 2, 5, 4, 4),
                                                          (0, 40, 39, 1, 1)])
def test_append_matches_oracle_bytes(gpu_ctx, window, capacity, past, query, m):
    rng = np.random.default_rng(past)
    planes, d = 6, 16
    x = rng.normal(size=(planes, m, d)).astype(np.float32)
    x[:, query:] = 9.0  # pad rows must never reach the slot
    slot = rng.normal(size=(planes, capacity, d)).astype(np.float32)
    spec = dict(kv_planes=planes, chunk_rows=m, depth=d, capacity=capacity, window=window,
                past=past, query=query)
    want = oracle.state_append(x, slot, **spec)
    got = run_append(gpu_ctx, x, slot, **spec)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # f32 -> f16 slot: round to nearest even of the same values
    got16 = run_append(gpu_ctx, x, slot.astype(np.float16), sd=np.float16, **spec)
    want16 = oracle.state_append(x.astype(np.float16).astype(np.float32),
                                 slot.astype(np.float16).astype(np.float32), **spec)
    assert np.array_equal(got16, want16.astype(np.float16))


def test_append_rejections(gpu_ctx):
    buf = gpu_ctx.zeros(4096)
    spec = dict(kv_planes=1, chunk_rows=2, depth=4, capacity=4, window=0, past=0, query=1)
    with pytest.raises(ka.ExecutionError):
        gpu_ctx.state_append(buf, buf, **{**spec, "past": 3, "query": 2})
    with pytest.raises(ka.ExecutionError):
        gpu_ctx.state_append(buf, buf, **{**spec, "query": 3})
    with pytest.raises(ka.GpuValidationError):
        gpu_ctx.state_append(buf, buf, **{**spec, "window": 5})
    buf.free()


def test_chain_prefill_then_decode_on_device(gpu_ctx):
    """Prefill -> decode chain with slots that live on the device and start as zeros
    (packages/runtime/tests/gpu_state_execution_test.ts:152-212,268-350): readers first, then
    append; equals ONE full-history causal attention in float64."""
    heads, kv_heads, depth, capacity = 8, 2, 64, 64
    r = heads // kv_heads
    rng = np.random.default_rng(77)
    slot_k = gpu_ctx.zeros(kv_heads * capacity * depth * 4)
    slot_v = gpu_ctx.zeros(kv_heads * capacity * depth * 4)
    ws = gpu_ctx.alloc(gpu_ctx.attention_state_workspace(1, heads, kv_heads, 8, depth, 0, capacity))
    past = 0
    outs, qs, ks, vs = [], [], [], []
    for m, query in [(8, 8), (8, 3)] + [(1, 1)] * 20:
        q = rng.normal(size=(1, heads, m, depth)).astype(np.float32)
        k = rng.normal(size=(1, kv_heads, m, depth)).astype(np.float32)
        v = rng.normal(size=(1, kv_heads, m, depth)).astype(np.float32)
        k[:, :, query:] = 9.0
        v[:, :, query:] = 400.0
        dq, dk, dv = gpu_ctx.upload(q), gpu_ctx.upload(k), gpu_ctx.upload(v)
        out = gpu_ctx.alloc(q.nbytes)
        gpu_ctx.attention_state(dq, dk, dv, slot_k, slot_v, out, batch=1, heads=heads,
                                kv_heads=kv_heads, chunk_rows=m, depth=depth, capacity=capacity,
                                window=0, half_scale=oracle.half_scale(depth), past=past,
                                query=query, workspace=ws)
        spec = dict(kv_planes=kv_heads, chunk_rows=m, depth=depth, capacity=capacity, window=0,
                    past=past, query=query)
        gpu_ctx.state_append(dk, slot_k, **spec)
        gpu_ctx.state_append(dv, slot_v, **spec)
        outs.append(out.download(np.float32, q.shape)[:, :, :query])
        qs.append(q[:, :, :query])
        ks.append(k[:, :, :query])
        vs.append(v[:, :, :query])
        past += query
        for b in (dq, dk, dv, out):
            b.free()
    cat = lambda parts: np.concatenate(parts, axis=2)  # noqa: E731
    total = past
    i = np.arange(total)
    s = float(oracle.half_scale(depth))
    want = helpers.dense_attention_f64(cat(qs), np.repeat(cat(ks), r, axis=1),
                                       np.repeat(cat(vs), r, axis=1), i[None, :] <= i[:, None],
                                       s * s)
    assert np.max(np.abs(cat(outs) - want)) <= STATE_ATOL
    # the slot holds exactly the valid rows; rows past `total` are still the initial zeros
    got_k = slot_k.download(np.float32, (kv_heads, capacity, depth))
    assert np.array_equal(got_k[:, :total], cat(ks)[0])
    assert np.all(got_k[:, total:] == 0.0)
    for b in (slot_k, slot_v, ws):
        b.free()


# ---------------------------------------------------------------------------- ragged batch

def test_config3_ragged_batch_equals_one_at_a_time(gpu_ctx):
    """benchmark config 3: 16 sequences, KV lengths ~ U{128..4096} (seeded), packed with
    prefix-sum offsets, H=32, Hkv=8, D=128, fp16 KV.  One launch; every sequence is then run
    alone through krm_attention_state and the bits must agree; a few are checked against the
    oracle (atol 5e-6 on f32 output)."""
    rng = np.random.default_rng(3)
    nseq, heads, kv_heads, depth = 16, 32, 8, 128
    lengths = rng.integers(128, 4097, size=nseq)
    cu = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    total = int(cu[-1])
    f16 = lambda a: a.astype(np.float16)  # noqa: E731
    slot_k = f16(rng.normal(size=(kv_heads, total, depth)))
    slot_v = f16(rng.normal(size=(kv_heads, total, depth)))
    q = f16(rng.normal(size=(nseq, heads, depth))).astype(np.float32)
    ins_k = f16(rng.normal(size=(nseq, kv_heads, depth))).astype(np.float32)
    ins_v = f16(rng.normal(size=(nseq, kv_heads, depth))).astype(np.float32)
    half = oracle.half_scale(depth)

    d = {name: gpu_ctx.upload(arr) for name, arr in
         dict(q=q, ins_k=ins_k, ins_v=ins_v, slot_k=slot_k, slot_v=slot_v).items()}
    out = gpu_ctx.alloc(q.nbytes)
    ws = gpu_ctx.alloc(gpu_ctx.attention_varlen_workspace(nseq, heads, kv_heads, depth, total))
    gpu_ctx.attention_varlen(d["q"], d["ins_k"], d["ins_v"], d["slot_k"], d["slot_v"], out, cu,
                             heads=heads, kv_heads=kv_heads, depth=depth, total_rows=total,
                             half_scale=half, io_dtype=ka.F32, kv_dtype=ka.F16, workspace=ws)
    batched = out.download(np.float32, q.shape)
    for b in list(d.values()) + [out, ws]:
        b.free()

    for i in range(nseq):
        past = int(lengths[i])
        case = StateCase(f"seq {i}", 1, heads, kv_heads, 1, depth, past + 1, 0, past, 1)
        sk = np.zeros((1, kv_heads, past + 1, depth), dtype=np.float32)
        sv = np.zeros_like(sk)
        sk[0, :, :past] = slot_k[:, cu[i]:cu[i + 1]]
        sv[0, :, :past] = slot_v[:, cu[i]:cu[i + 1]]
        x = dict(q=q[i].reshape(1, heads, 1, depth), ins_k=ins_k[i].reshape(1, kv_heads, 1, depth),
                 ins_v=ins_v[i].reshape(1, kv_heads, 1, depth), slot_k=sk, slot_v=sv)
        alone = run_attention(gpu_ctx, case, x, io=np.float32, kv=np.float16)
        assert np.array_equal(alone.reshape(heads, depth).view(np.uint32),
                              batched[i].view(np.uint32)), i
        if i % 5 == 0:
            want = oracle_state_attention(case, x)
            ok, fails, max_abs, worst = oracle.allclose(alone, want, atol=STATE_ATOL, rtol=0)
            assert ok, (i, fails, max_abs, worst)


def test_varlen_edges(gpu_ctx):
    """Empty past (a sequence whose only column is its own) and single-split sequences."""
    heads, kv_heads, depth = 8, 2, 64
    lengths = np.array([0, 5, 256, 257, 0, 1])
    cu = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    total = int(cu[-1])
    rng = np.random.default_rng(9)
    nseq = len(lengths)
    slot_k = rng.normal(size=(kv_heads, total, depth)).astype(np.float32)
    slot_v = rng.normal(size=(kv_heads, total, depth)).astype(np.float32)
    q = rng.normal(size=(nseq, heads, depth)).astype(np.float32)
    ins_k = rng.normal(size=(nseq, kv_heads, depth)).astype(np.float32)
    ins_v = rng.normal(size=(nseq, kv_heads, depth)).astype(np.float32)
    d = {name: gpu_ctx.upload(arr) for name, arr in
         dict(q=q, ins_k=ins_k, ins_v=ins_v, slot_k=slot_k, slot_v=slot_v).items()}
    out = gpu_ctx.alloc(q.nbytes)
    ws = gpu_ctx.alloc(gpu_ctx.attention_varlen_workspace(nseq, heads, kv_heads, depth, total))
    gpu_ctx.attention_varlen(d["q"], d["ins_k"], d["ins_v"], d["slot_k"], d["slot_v"], out, cu,
                             heads=heads, kv_heads=kv_heads, depth=depth, total_rows=total,
                             half_scale=oracle.half_scale(depth), workspace=ws)
    got = out.download(np.float32, q.shape)
    for i in range(nseq):
        past = int(lengths[i])
        case = StateCase(f"seq {i}", 1, heads, kv_heads, 1, depth, past + 1, 0, past, 1)
        sk = np.zeros((1, kv_heads, past + 1, depth), dtype=np.float32)
        sv = np.zeros_like(sk)
        sk[0, :, :past] = slot_k[:, cu[i]:cu[i + 1]]
        sv[0, :, :past] = slot_v[:, cu[i]:cu[i + 1]]
        x = dict(q=q[i].reshape(1, heads, 1, depth), ins_k=ins_k[i].reshape(1, kv_heads, 1, depth),
                 ins_v=ins_v[i].reshape(1, kv_heads, 1, depth), slot_k=sk, slot_v=sv)
        want = oracle_state_attention(case, x)
        assert np.max(np.abs(got[i].reshape(want.shape) - want)) <= STATE_ATOL, i
    with pytest.raises(ka.GpuValidationError):  # not ascending
        gpu_ctx.attention_varlen(d["q"], d["ins_k"], d["ins_v"], d["slot_k"], d["slot_v"], out,
                                 [0, 5, 3], heads=heads, kv_heads=kv_heads, depth=depth,
                                 total_rows=total, half_scale=0.3, workspace=ws)
    for b in list(d.values()) + [out, ws]:
        b.free()


def test_varlen_planned_on_the_device_is_recordable(gpu_ctx):
    """The ragged step with its tables built on the device: equals the host-table form bitwise;
    recorded once and replayed while the sequences grow (the offsets are rewritten between the
    replays, with eager work and synchronisations in between) every replay equals the eager
    host-table result of the same lengths; offsets that are not ascending raise the plan's
    fault word and leave `out` untouched."""
    heads, kv_heads, depth, nseq = 8, 2, 128, 5
    capacity_rows = [700, 300, 900, 140, 20]           # rows each sequence owns in the slot
    starts = np.concatenate([[0], np.cumsum(capacity_rows)]).astype(np.int64)
    total = int(starts[-1])
    rng = np.random.default_rng(17)
    f16 = lambda a: a.astype(np.float16)  # noqa: E731
    slot_k, slot_v = (f16(rng.normal(size=(kv_heads, total, depth))) for _ in range(2))
    q, ins_k, ins_v = (f16(rng.normal(size=(nseq, h, depth))) for h in (heads, kv_heads, kv_heads))
    d = {name: gpu_ctx.upload(arr) for name, arr in
         dict(q=q, ins_k=ins_k, ins_v=ins_v, slot_k=slot_k, slot_v=slot_v).items()}
    half = oracle.half_scale(depth)
    out, out_host = gpu_ctx.alloc(q.nbytes), gpu_ctx.alloc(q.nbytes)
    ws = gpu_ctx.alloc(gpu_ctx.attention_varlen_workspace(nseq, heads, kv_heads, depth, total))
    ws_host = gpu_ctx.alloc(gpu_ctx.attention_varlen_workspace(nseq, heads, kv_heads, depth, total))
    plan = gpu_ctx.alloc(gpu_ctx.attention_varlen_plan_bytes(nseq))
    max_splits = gpu_ctx.attention_varlen_max_splits(nseq, depth, ka.F16, total)
    assert max_splits == total // 128 + nseq
    cu_dev = gpu_ctx.alloc(4 * (nseq + 1))
    common = dict(heads=heads, kv_heads=kv_heads, depth=depth, total_rows=total, half_scale=half,
                  io_dtype=ka.F16, kv_dtype=ka.F16)

    # each replay sees other (ascending) offsets: sequence i holds fill * capacity_rows[i] rows
    def offsets(fill):
        cu = np.zeros(nseq + 1, dtype=np.int32)
        for i in range(nseq):
            cu[i + 1] = cu[i] + int(capacity_rows[i] * fill)
        return cu

    with gpu_ctx.record() as rec:
        gpu_ctx.attention_varlen_plan(cu_dev, plan, nseq=nseq, depth=depth, kv_dtype=ka.F16,
                                      total_rows=total, max_splits=max_splits)
        gpu_ctx.attention_varlen_planned(d["q"], d["ins_k"], d["ins_v"], d["slot_k"], d["slot_v"],
                                         out, plan, nseq=nseq, max_splits=max_splits,
                                         workspace=ws, **common)
    for fill in (0.25, 0.6, 1.0, 0.4):
        cu = offsets(fill)
        cu_dev.upload(cu)
        out.upload(np.full(q.size, 77.0, dtype=np.float16))
        rec.graph.launch()
        got = out.download(np.float16, q.shape)
        assert plan.download(np.int32, (2 * (nseq + 1) + 1,))[-1] == 0
        gpu_ctx.attention_varlen(d["q"], d["ins_k"], d["ins_v"], d["slot_k"], d["slot_v"],
                                 out_host, cu, workspace=ws_host, **common)
        want = out_host.download(np.float16, q.shape)
        assert got.tobytes() == want.tobytes(), fill
    rec.graph.destroy()

    # offsets that break the contract: fault word, no store
    for bad in ([0, 50, 40, 60, 70, 80], [0, 10, 20, 30, 40, total + 1], [-1, 10, 20, 30, 40, 50]):
        cu_dev.upload(np.array(bad, dtype=np.int32))
        sentinel = np.full(q.size, 55.0, dtype=np.float16)
        out.upload(sentinel)
        gpu_ctx.attention_varlen_plan(cu_dev, plan, nseq=nseq, depth=depth, kv_dtype=ka.F16,
                                      total_rows=total, max_splits=max_splits)
        gpu_ctx.attention_varlen_planned(d["q"], d["ins_k"], d["ins_v"], d["slot_k"], d["slot_v"],
                                         out, plan, nseq=nseq, max_splits=max_splits,
                                         workspace=ws, **common)
        assert plan.download(np.int32, (2 * (nseq + 1) + 1,))[-1] == 1, bad
        assert out.download(np.float16, (q.size,)).tobytes() == sentinel.tobytes(), bad
    # a legal plan afterwards still works (the counters were left clean)
    cu = offsets(1.0)
    cu_dev.upload(cu)
    gpu_ctx.attention_varlen_plan(cu_dev, plan, nseq=nseq, depth=depth, kv_dtype=ka.F16,
                                  total_rows=total, max_splits=max_splits)
    gpu_ctx.attention_varlen_planned(d["q"], d["ins_k"], d["ins_v"], d["slot_k"], d["slot_v"],
                                     out, plan, nseq=nseq, max_splits=max_splits, workspace=ws,
                                     **common)
    gpu_ctx.attention_varlen(d["q"], d["ins_k"], d["ins_v"], d["slot_k"], d["slot_v"], out_host,
                             cu, workspace=ws_host, **common)
    assert out.download(np.float16, q.shape).tobytes() == out_host.download(np.float16, q.shape).tobytes()
    for b in list(d.values()) + [out, out_host, ws, ws_host, plan, cu_dev]:
        b.free()


@pytest.mark.parametrize("io,kv", [(np.float32, np.float32), (np.float16, np.float16),
                                   (np.float32, np.float16)])
@pytest.mark.parametrize("dyn", [False, True])
def test_attention_chunk_equals_attention_transpose_and_appends(gpu_ctx, io, kv, dyn):
    """krm_attention_chunk with the row-major output and the fused append writes the bits of
    krm_attention_state + krm_transpose_01 + two krm_state_append (pad rows: zeros in the output,
    nothing appended; every other slot row untouched); with a window the append is refused and
    the row-major output alone still matches."""
    case = StateCase("chunk D64 M40 Q33 P100", 2, 8, 2, 40, 64, 192, 0, 100, 33)
    x = random_state_inputs(case, seed=77, f16_values=True)
    b, h, hkv, m, d, c = (case.batch, case.heads, case.kv_heads, case.chunk_rows, case.depth,
                          case.capacity)
    io_code, kv_code = ka.dtype_code(io), ka.dtype_code(kv)

    def upload():
        return {k: gpu_ctx.upload(np.ascontiguousarray(v, dtype=io if k in ("q", "ins_k", "ins_v")
                                                       else kv)) for k, v in x.items()}
    ref = upload()
    want_hm = gpu_ctx.upload(np.full(b * h * m * d, 5.0, dtype=io))
    gpu_ctx.attention_state(ref["q"], ref["ins_k"], ref["ins_v"], ref["slot_k"], ref["slot_v"],
                            want_hm, half_scale=oracle.half_scale(d), io_dtype=io_code,
                            kv_dtype=kv_code, **case.kwargs())
    spec = dict(kv_planes=b * hkv, chunk_rows=m, depth=d, capacity=c, window=0, x_dtype=io_code,
                slot_dtype=kv_code)
    gpu_ctx.state_append(ref["ins_k"], ref["slot_k"], past=case.past, query=case.query, **spec)
    gpu_ctx.state_append(ref["ins_v"], ref["slot_v"], past=case.past, query=case.query, **spec)
    want = want_hm.download(io, (b, h, m, d)).transpose(0, 2, 1, 3)

    got = upload()
    out = gpu_ctx.upload(np.full(b * h * m * d, 7.0, dtype=io))
    lengths = None
    if dyn:
        lengths = gpu_ctx.zeros(16)
        gpu_ctx.lengths_set(lengths, case.past, case.query)
    geometry = {k: v for k, v in case.kwargs().items() if k not in ("past", "query")}
    gpu_ctx.attention_chunk(got["q"], got["ins_k"], got["ins_v"], got["slot_k"], got["slot_v"],
                            out, half_scale=oracle.half_scale(d), past=0 if dyn else case.past,
                            query=0 if dyn else case.query, lengths=lengths, io_dtype=io_code,
                            kv_dtype=kv_code, row_major=True, append=True, **geometry)
    bits = np.uint32 if io == np.float32 else np.uint16
    kbits = np.uint32 if kv == np.float32 else np.uint16
    assert np.array_equal(out.download(io, (b, m, h, d)).view(bits), np.ascontiguousarray(want).view(bits))
    for name in ("slot_k", "slot_v"):
        assert np.array_equal(got[name].download(kv, (b, hkv, c, d)).view(kbits),
                              ref[name].download(kv, (b, hkv, c, d)).view(kbits)), name
    if dyn:
        assert lengths.download(np.uint32, (4,))[2] == 0
    with pytest.raises(ka.GpuValidationError, match="window == 0"):
        gpu_ctx.attention_chunk(got["q"], got["ins_k"], got["ins_v"], got["slot_k"], got["slot_v"],
                                out, half_scale=oracle.half_scale(d), past=case.past,
                                query=case.query, io_dtype=io_code, kv_dtype=kv_code, append=True,
                                **{**geometry, "window": 64})
    with pytest.raises(ka.GpuValidationError, match="D = 64, 128 or 256"):
        gpu_ctx.attention_chunk(got["q"], got["ins_k"], got["ins_v"], got["slot_k"], got["slot_v"],
                                out, half_scale=0.5, past=0, query=1, io_dtype=io_code,
                                kv_dtype=kv_code, **{**geometry, "depth": 32})


# ---- KV-sharing layers: two readers, one append -------------------------------------------------

SHARED_SERIES = [
    # packages/runtime/tests/gpu_state_acceptance_test.ts:846-864
    dict(name="full", heads=2, kv_heads=2, depth=4, capacity=16, window=0, chunk=3,
         steps=[(3, 3), (3, 3), (3, 3), (1, 1)], order_probe=None),
    # a ring of W = C = 4: the append of step 1 (past 3, Q 3) writes physical rows 3, 0, 1, two of
    # which the readers of the same step still have to read — the one place where the order of
    # readers and append shows in the values
    dict(name="sliding W=4", heads=2, kv_heads=2, depth=4, capacity=4, window=4, chunk=3,
         steps=[(3, 3), (3, 3), (3, 3), (1, 1)], order_probe=1),
]


@pytest.mark.parametrize("series", SHARED_SERIES, ids=lambda s: s["name"])
def test_two_readers_one_append(gpu_ctx, series):
    """Two attention calls with different queries read the same K / V rows and the same state
    slots, then ONE pair of appends follows (packages/runtime/tests/
    gpu_state_acceptance_test.ts:866-977): both outputs equal the oracle on the slots as they
    were BEFORE the append (atol 5e-6), differ from each other, and — where the ring wraps into
    rows of the same step — differ from an oracle that appended first; the slot bytes after
    every step equal the oracle's chained slots."""
    ctx = gpu_ctx
    H, Hkv, D, C, W, M = (series[k] for k in ("heads", "kv_heads", "depth", "capacity", "window",
                                              "chunk"))
    scale = oracle.half_scale(D)
    slot_k = np.zeros((1, Hkv, C, D), dtype=np.float32)
    slot_v = np.zeros((1, Hkv, C, D), dtype=np.float32)
    dk, dv = ctx.upload(slot_k), ctx.upload(slot_v)
    past = 0
    for index, (rows, query) in enumerate(series["steps"]):
        salt = 17 + index * 23
        count = Hkv * rows * D
        qs = [helpers.seeded(H * rows * D, lambda i, s=salt + 101 * r: helpers.QUERY(i + s))
              .reshape(1, H, rows, D) for r in range(2)]
        k = helpers.seeded(count, lambda i: helpers.KEY(i + salt)).reshape(1, Hkv, rows, D)
        v = helpers.seeded(count, lambda i: helpers.VALUE(i + salt)).reshape(1, Hkv, rows, D)
        common = dict(chunk_rows=rows, depth=D, capacity=C, window=W, past=past, query=query)

        def read(q, sk, sv):
            return oracle.state_attention(q, k, v, sk, sv, batch=1, heads=H, kv_heads=Hkv,
                                          scale=scale, **common)

        bk, bv = ctx.upload(k), ctx.upload(v)
        outs = []
        for q in qs:   # both readers first ...
            bq, out = ctx.upload(q), ctx.alloc(q.nbytes)
            ws = ctx.alloc(ctx.attention_state_workspace(1, H, Hkv, rows, D, W, past, query))
            ctx.attention_state(bq, bk, bv, dk, dv, out, batch=1, heads=H, kv_heads=Hkv,
                                half_scale=scale, workspace=ws, **common)
            outs.append(out.download(np.float32, q.shape))
            for b in (bq, out, ws):
                b.free()
        for src, slot in ((bk, dk), (bv, dv)):   # ... then the one pair of appends
            ctx.state_append(src, slot, kv_planes=Hkv, **common)
        for q, got in zip(qs, outs):
            want = read(q, slot_k, slot_v)
            assert np.any(np.abs(want) > 1e-3), "the expected output is trivial"
            ok, fails, max_abs, worst = oracle.allclose(got, want, atol=STATE_ATOL, rtol=0)
            assert ok, (series["name"], index, fails, max_abs, worst)
        assert outs[0].tobytes() != outs[1].tobytes()
        new_k = oracle.state_append(k, slot_k, kv_planes=Hkv, **common)
        new_v = oracle.state_append(v, slot_v, kv_planes=Hkv, **common)
        if series["order_probe"] == index:
            for q, got in zip(qs, outs):
                wrong = read(q, new_k, new_v)
                ok, *_ = oracle.allclose(got, wrong, atol=STATE_ATOL, rtol=0)
                assert not ok, "the probe step does not tell reader-first from append-first"
        slot_k, slot_v = new_k, new_v
        past += query
        assert dk.download(np.float32, slot_k.shape).tobytes() == slot_k.tobytes()
        assert dv.download(np.float32, slot_v.shape).tobytes() == slot_v.tobytes()
        bk.free()
        bv.free()
    dk.free()
    dv.free()


# ---- head dims of 256 (a sliding layer of a Gemma-4-style decoder) -------------------------------

@pytest.mark.parametrize("case,io,kv", [
    (StateCase("chunk 40 rows, past 70, D 256", 1, 4, 2, 40, 256, 128, 0, 70, 37), np.float32, np.float32),
    (StateCase("chunk 33 rows, window 48, D 256", 2, 2, 1, 33, 256, 64, 48, 90, 33), np.float32, np.float32),
    (StateCase("chunk 16 rows, D 256, fp16 state", 1, 8, 1, 16, 256, 64, 0, 20, 16), np.float32, np.float16),
    (StateCase("decode, past 300, D 256", 1, 8, 2, 1, 256, 512, 0, 300, 1), np.float32, np.float32),
    (StateCase("decode, 8:1, past 700, D 256", 1, 8, 1, 1, 256, 1024, 0, 700, 1), np.float32, np.float32),
    (StateCase("decode, window 128, D 256", 2, 4, 4, 1, 256, 128, 128, 1000, 1), np.float32, np.float32),
    (StateCase("decode, past 900, D 512 fp16", 1, 8, 1, 1, 512, 1024, 0, 900, 1), np.float16, np.float16),
], ids=lambda v: v.name if isinstance(v, StateCase) else None)
def test_head_dim_256_forms(gpu_ctx, case, io, kv):
    """The chunk kernel's D = 256 form (two waves a workgroup) and the decode kernel with rows
    that span a whole wave (f32 D = 256, fp16 D = 512) against the oracle: atol 5e-6 for f32
    output (the reference's gate), one fp16 ulp for fp16 output; pad rows exact +0."""
    x = random_state_inputs(case, seed=case.past + case.depth, f16_values=True)
    want = oracle_state_attention(case, x)
    got = run_attention(gpu_ctx, case, x, io=io, kv=kv)
    if io == np.float32:
        ok, fails, max_abs, worst = oracle.allclose(got, want, atol=STATE_ATOL, rtol=0)
        assert ok, (case.name, fails, max_abs, worst)
    else:
        ref = want.astype(np.float16).astype(np.float32)
        assert np.all(np.abs(got.astype(np.float32) - ref) <= np.abs(ref) * 2.0 ** -10 + 1e-6)
    pad = got[:, :, case.query:, :]
    assert not pad.size or (np.all(pad == 0) and not np.any(np.signbit(pad)))
