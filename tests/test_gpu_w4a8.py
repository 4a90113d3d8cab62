"""GPU parity of the w4a8 path (activation quantiser + integer-dot `linear`, through the C ABI)
against the CPU oracle.  The contract is atol = 0: group sums are exact integers and every
floating-point step is one correctly rounded operation in a fixed order
(docs/decisions/0076-w4a8-linear-execution.md:40-60), so every comparison here is bitwise
(NaN where the oracle has NaN)."""
import numpy as np
import pytest

import helpers
import karume_amd as ka
from helpers import oracle

pytestmark = pytest.mark.gpu


def assert_exact(got, want, what):
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, what
    nan = np.isnan(want) if want.dtype.kind == "f" else np.zeros(want.shape, bool)
    assert np.array_equal(np.isnan(got) if got.dtype.kind == "f" else nan, nan), what
    assert np.array_equal(got[~nan], want[~nan]), (what, np.argwhere(got != want)[:5])


def run_quantize(ctx, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, dim = x.shape
    dx = ctx.upload(x)
    dq, ds = ctx.alloc(max(rows * dim, 16)), ctx.alloc(max(rows * 4, 16))
    ctx.quantize_rows(dx, dq, ds, rows, dim)
    q = dq.download(np.int8, (rows, dim))
    s = ds.download(np.float32, (rows,))
    for b in (dx, dq, ds):
        b.free()
    return q, s


def run_w4a8(ctx, x, packed, scale, bias, n, k, group):
    """quantize_rows + linear_w4a8 with node-local temporaries, as the reference's builder
    issues them (packages/runtime/src/runtime/recipe-builder.ts:1428-1488)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    scale = np.ascontiguousarray(scale)
    m = x.shape[0]
    dx, dw, dsc = ctx.upload(x), ctx.upload(packed), ctx.upload(scale)
    db = ctx.upload(np.ascontiguousarray(bias, dtype=np.float32)) if bias is not None else None
    dq, dxs = ctx.alloc(max(m * k, 16)), ctx.alloc(max(m * 4, 16))
    out = ctx.alloc(max(m * n * 4, 16))
    ctx.quantize_rows(dx, dq, dxs, m, k)
    ctx.linear_w4a8(dq, dxs, dw, dsc, db, out, m, n, k, group, ka.dtype_code(scale.dtype))
    got = out.download(np.float32, (m, n))
    for b in (dx, dw, dsc, dq, dxs, out) + ((db,) if db is not None else ()):
        b.free()
    return got


# ---- quantize_rows: packages/runtime/tests/gpu_i8a8_test.ts:216-330 ---------------------------

def test_quantize_ties_round_to_even(gpu_ctx):
    values = np.array([[127, 0.5, 1.5, -0.5, -1.5, 2.5, 3.5, -3.5]], dtype=np.float32)
    q, s = run_quantize(gpu_ctx, values)
    assert float(s[0]) == 1.0
    assert q.tolist() == [[127, 0, 2, 0, -2, 2, 4, -4]]


def test_quantize_matches_oracle_rows_of_different_size(gpu_ctx):
    rows, dim = 7, 20  # a multiple of 4 that is no multiple of 16
    x = np.array([[0 if r == 3 else helpers.SIGNED_A8(r * dim + i) * (1 + r * 3)
                   for i in range(dim)] for r in range(rows)], dtype=np.float32)
    q, s = run_quantize(gpu_ctx, x)
    want_q, want_s = oracle.quantize_rows(x, dim)
    assert_exact(s, want_s, "scale")
    assert_exact(q, want_q, "codes")
    assert float(s[3]) == 1.1754943508222875e-38 and not q[3].any()


def test_quantize_propagates_nan_and_inf_to_the_row_scale(gpu_ctx):
    rows, dim = 4, 8
    x = helpers.seeded(rows * dim, helpers.SIGNED_A8).reshape(rows, dim)
    x[1, dim - 1] = np.nan
    x[2, 3] = np.inf
    x[3, 3] = -np.inf
    q, s = run_quantize(gpu_ctx, x)
    want_q, want_s = oracle.quantize_rows(x, dim)
    assert_exact(s, want_s, "scale")
    assert np.isfinite(s[0]) and np.isnan(s[1]) and s[2] == np.inf and s[3] == np.inf
    assert_exact(q, want_q, "codes")  # also the non-finite rows: a NaN quotient stores 0


@pytest.mark.parametrize("rows, dim", [(1, 4096), (3, 11008), (300, 260), (2, 4)])
def test_quantize_random_rows_bit_exact_without_a_tie_margin(gpu_ctx, rows, dim):
    """Random data, no margin gate: the device division is correctly rounded, so the codes
    equal the oracle's even where x / s sits next to a half-integer."""
    rng = np.random.default_rng(rows * 131 + dim)
    x = (rng.normal(size=(rows, dim)) * rng.uniform(0.01, 30, size=(rows, 1))).astype(np.float32)
    x[0, : min(dim, 8)] = [0.5, 1.5, 2.5, -0.5, 127, -127, 63.5, 0][: min(dim, 8)]
    q, s = run_quantize(gpu_ctx, x)
    want_q, want_s = oracle.quantize_rows(x, dim)
    assert_exact(s, want_s, "scale")
    assert_exact(q, want_q, "codes")


def test_quantize_quotients_on_and_next_to_every_tie(gpu_ctx):
    """Rows built so that x / s lands on, one ulp below and one ulp above each half-integer of
    the code range (scales that are no power of two), plus rows in the subnormal range: the
    quantiser takes a reciprocal product where that provably rounds like the quotient and the
    division elsewhere — the codes must equal the oracle's everywhere."""
    rng = np.random.default_rng(5)
    rows = []
    for top in (1.0, 3.0, 0.7310585975646973, 1234.5677490234375, 6.103515625e-05, 2.9e37,
                1.3e-36):
        s = np.float32(np.float32(top) * np.float32(1.0 / 127.0))
        halves = (np.arange(-127, 127, dtype=np.float64) + 0.5)
        centre = (halves * np.float64(s)).astype(np.float32)
        row = np.concatenate([[np.float32(top)], centre, np.nextafter(centre, np.float32(np.inf)),
                              np.nextafter(centre, np.float32(-np.inf)),
                              np.nextafter(np.nextafter(centre, np.float32(np.inf)),
                                           np.float32(np.inf))]).astype(np.float32)
        row = row[np.abs(row) <= np.float32(top)]
        rows.append(np.resize(row, 1024))
    sub = rng.integers(-(1 << 22), 1 << 22, size=1024).astype(np.int32)   # subnormal bit patterns
    rows.append((np.abs(sub).astype(np.uint32) | np.where(sub < 0, 1 << 31, 0).astype(np.uint32))
                .view(np.float32))
    rows.append(rows[-1] * np.float32(0.01))
    x = np.stack(rows).astype(np.float32)
    q, s = run_quantize(gpu_ctx, x)
    want_q, want_s = oracle.quantize_rows(x, x.shape[1])
    assert_exact(s, want_s, "scale")
    assert_exact(q, want_q, "codes")
    assert len(np.unique(want_q[0])) > 200  # the rows do walk the code range


def test_quantize_rejections(gpu_ctx):
    buf = gpu_ctx.alloc(256)
    with pytest.raises(ka.GpuValidationError, match="multiple of 4"):
        gpu_ctx.quantize_rows(buf, buf, buf, 1, 6)
    with pytest.raises(ka.GpuValidationError, match="positive"):
        gpu_ctx.quantize_rows(buf, buf, buf, 1, 0)
    gpu_ctx.quantize_rows(buf, buf, buf, 0, 8)  # no rows: nothing to do
    buf.free()


# ---- linear: packages/runtime/tests/gpu_i8a8_test.ts:758-912 ----------------------------------

@pytest.mark.parametrize("case", helpers.W4A8_CASES, ids=lambda c: c.name)
def test_w4a8_reference_cases_bit_exact(gpu_ctx, case):
    x, packed, q, scale, bias = helpers.make_w4a8(case)
    want = oracle.linear_w4a8(x, packed, scale, bias, case.n, case.k, case.group)
    got = run_w4a8(gpu_ctx, x, packed, scale, bias, case.n, case.k, case.group)
    assert_exact(got, want, case.name)
    assert len(set(got.reshape(-1).tolist())) > 1


def test_w4a8_nan_row_zero_row(gpu_ctx):
    case = helpers.W4A8_CASES[0]
    nan_row, zero_row = 2, 5

    def x_value(i, m, k):
        row = i // k
        if row == zero_row:
            return 0.0
        if row == nan_row and i % k == k - 3:
            return float("nan")
        return helpers.SIGNED_A8(i)

    x, packed, q, scale, bias = helpers.make_w4a8(case, x_value)
    want = oracle.linear_w4a8(x, packed, scale, bias, case.n, case.k, case.group)
    got = run_w4a8(gpu_ctx, x, packed, scale, bias, case.n, case.k, case.group)
    assert_exact(got, want, "nan / zero rows")
    assert np.isnan(got[nan_row]).all() and np.isfinite(got[nan_row + 1]).all()
    assert np.array_equal(got[zero_row], bias)


def test_w4a8_differs_from_the_f32_activation_path(gpu_ctx):
    case = helpers.W4A8_CASES[3]
    x, packed, q, scale, bias = helpers.make_w4a8(case)
    got = run_w4a8(gpu_ctx, x, packed, scale, bias, case.n, case.k, case.group)
    f32_path = oracle.linear_i4(x, packed, scale, bias, case.n, case.k, case.group)
    assert not np.array_equal(got, f32_path)
    assert np.allclose(got, f32_path, rtol=0.05, atol=0.5)  # same op, coarser activations


SHAPES = [  # (m, n, k, group, fp16 scales, bias)
    (1, 4096, 4096, 128, True, False),    # the decode GEMV shape
    (1, 130, 2048, 32, False, True),      # one group per lane
    (1, 64, 6144, 2048, True, True),      # one group per step
    (2, 70, 4096, 64, True, True),
    (4, 100, 1024, 128, False, True),     # K shorter than a step
    (7, 33, 5632, 128, True, True),       # K with a partial last step
    (8, 16, 11008, 64, True, False),
    (1, 9, 8192, 4096, True, True),       # a group longer than a step (fallback form)
    (3, 21, 64, 16, False, True),         # two groups per lane (fallback form)
    (16, 4096, 4096, 128, True, True),    # the ragged batch's GEMV shape
    (40, 300, 1024, 128, True, True),
    # the matrix-core form (M > 8, group >= 64)
    (70, 260, 5696, 64, True, True),      # K ends inside an LDS stage; N one past a block
    (9, 31, 512, 512, False, True),       # a group over two stages
    (33, 64, 4096, 2048, True, False),
    (100, 257, 1024, 256, False, True),
    (512, 1000, 4096, 128, True, True),   # the prefill row count
    (130, 96, 11008, 128, True, True),    # the down-projection's K
]


@pytest.mark.parametrize("m, n, k, group, scale_f16, with_bias", SHAPES)
def test_w4a8_random_shapes_bit_exact(gpu_ctx, m, n, k, group, scale_f16, with_bias):
    rng = np.random.default_rng(m * 7919 + n * 31 + k + group)
    packed, q, scale = helpers.synthetic_int4(rng, n, k, group, scale_f16)
    x = rng.normal(size=(m, k)).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32) if with_bias else None
    want = oracle.linear_w4a8(x, packed, np.asarray(scale, dtype=np.float32), bias, n, k, group)
    got = run_w4a8(gpu_ctx, x, packed, scale, bias, n, k, group)
    assert_exact(got, want, (m, n, k, group))


def test_w4a8_rows_do_not_depend_on_the_batch(gpu_ctx):
    rng = np.random.default_rng(3)
    n, k, group = 512, 4096, 128
    packed, q, scale = helpers.synthetic_int4(rng, n, k, group)
    x = rng.normal(size=(16, k)).astype(np.float32)
    whole = run_w4a8(gpu_ctx, x, packed, scale, None, n, k, group)
    for rows in (1, 3, 8):
        part = run_w4a8(gpu_ctx, x[:rows], packed, scale, None, n, k, group)
        assert np.array_equal(part, whole[:rows])


def test_w4a8_rejections(gpu_ctx):
    buf = gpu_ctx.alloc(4096)
    args = (buf, buf, buf, buf, None, buf)
    with pytest.raises(ka.GpuValidationError, match="multiple of 4"):
        gpu_ctx.linear_w4a8(*args, 1, 4, 0, 16)
    with pytest.raises(ka.GpuValidationError, match="power of two"):
        gpu_ctx.linear_w4a8(*args, 1, 4, 48, 24)
    with pytest.raises(ka.GpuValidationError, match="power of two"):
        gpu_ctx.linear_w4a8(*args, 1, 4, 32, 8)
    with pytest.raises(ka.GpuValidationError, match="not a multiple of group_size"):
        gpu_ctx.linear_w4a8(*args, 1, 4, 48, 32)
    with pytest.raises(ka.GpuValidationError, match="int32 reduction limit"):
        gpu_ctx.linear_w4a8(*args, 1, 1, 1 << 22, 1 << 22)
    buf.free()


# ---- the pair behind one call: the same bits from one launch ---------------------------------

def run_w4a8_fused(ctx, x, packed, scale, bias, n, k, group, work=True):
    x = np.ascontiguousarray(x, dtype=np.float32)
    scale = np.ascontiguousarray(scale)
    m = x.shape[0]
    dx, dw, dsc = ctx.upload(x), ctx.upload(packed), ctx.upload(scale)
    db = ctx.upload(np.ascontiguousarray(bias, dtype=np.float32)) if bias is not None else None
    dq = ctx.alloc(max(m * k, 16)) if work else None
    dxs = ctx.alloc(max(m * 4, 16)) if work else None
    out = ctx.alloc(max(m * n * 4, 16))
    try:
        ctx.linear_w4a8_fused(dx, dw, dsc, db, out, m, n, k, group, ka.dtype_code(scale.dtype),
                              xq_i8=dq, xs_f32=dxs)
        return out.download(np.float32, (m, n))
    finally:
        for b in (dx, dw, dsc, out, dq, dxs, db):
            if b is not None:
                b.free()


FUSED_SHAPES = [  # (m, n, k, group, fp16 scales, bias, one launch)
    (1, 4096, 4096, 128, True, False, True),     # the decode GEMV shape
    (1, 130, 2048, 32, False, True, True),
    (1, 64, 6144, 2048, True, True, True),
    (1, 40, 11008, 64, True, True, True),        # partial last step, 11 quads a thread
    (1, 24, 16384, 128, True, True, True),       # the longest single row of the one-launch form
    (1, 24, 16512, 128, True, True, False),      # one group past it: two launches
    (2, 70, 4096, 64, True, True, True),
    (2, 70, 8192, 64, False, True, True),
    (3, 50, 4096, 128, True, True, True),        # a block of four rows with one row unused
    (4, 100, 1024, 128, False, True, True),      # K shorter than a step
    (7, 33, 2048, 128, True, True, True),        # two blocks, the second ragged
    (8, 16, 4096, 64, True, False, True),
    (7, 33, 5632, 128, True, True, False),       # four rows of 5632 do not fit: two launches
    (3, 21, 64, 16, False, True, False),         # groups of 16: two launches
    (40, 300, 1024, 128, True, True, False),     # the matrix-core form
]


@pytest.mark.parametrize("m, n, k, group, scale_f16, with_bias, one_launch", FUSED_SHAPES)
def test_w4a8_fused_call_equals_the_two_steps(gpu_ctx, m, n, k, group, scale_f16, with_bias,
                                              one_launch):
    rng = np.random.default_rng(m * 104729 + n * 31 + k + group)
    packed, q, scale = helpers.synthetic_int4(rng, n, k, group, scale_f16)
    x = (rng.normal(size=(m, k)) * rng.choice([1e-3, 1.0, 300.0], size=(m, 1))).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32) if with_bias else None
    want = oracle.linear_w4a8(x, packed, np.asarray(scale, dtype=np.float32), bias, n, k, group)
    assert_exact(run_w4a8_fused(gpu_ctx, x, packed, scale, bias, n, k, group), want,
                 (m, n, k, group))
    assert_exact(run_w4a8(gpu_ctx, x, packed, scale, bias, n, k, group), want, "two steps")
    if one_launch:  # needs no work buffers
        assert_exact(run_w4a8_fused(gpu_ctx, x, packed, scale, bias, n, k, group, work=False),
                     want, "no work buffers")
    else:
        with pytest.raises(ka.GpuValidationError, match="work buffers"):
            run_w4a8_fused(gpu_ctx, x, packed, scale, bias, n, k, group, work=False)


def test_w4a8_fused_call_special_rows_and_ties(gpu_ctx):
    """A NaN row, a row of zeros, a row with an infinity and quotients on rounding ties."""
    rng = np.random.default_rng(11)
    n, k, group = 48, 1024, 128
    packed, q, scale = helpers.synthetic_int4(rng, n, k, group)
    x = rng.normal(size=(4, k)).astype(np.float32)
    x[0, 17] = np.nan
    x[1] = 0.0
    x[2, 5] = np.inf
    x[3] = rng.integers(-254, 255, size=k).astype(np.float32) * 0.5   # halves: ties everywhere
    x[3, 0] = 127.0                                                   # scale exactly 1
    want = oracle.linear_w4a8(x, packed, np.asarray(scale, dtype=np.float32), None, n, k, group)
    got = run_w4a8_fused(gpu_ctx, x, packed, scale, None, n, k, group, work=False)
    assert_exact(got, want, "special rows")
    assert np.isnan(got[0]).all() and (got[1] == 0).all()
    for row in range(4):  # each row alone (block of one) gives the same bits
        alone = run_w4a8_fused(gpu_ctx, x[row:row + 1], packed, scale, None, n, k, group,
                               work=False)
        assert_exact(alone[0], want[row], ("alone", row))
