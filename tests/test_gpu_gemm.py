"""GPU parity of the MFMA GEMM paths of `linear` (M > 16) against the CPU oracle.

Two numerics classes (stated in the kernels):
* exact-operand kernel (large shapes; KRM_COMPUTE_F16, and KRM_COMPUTE_F32 with the f32
  activations split into fp16 hi + lo): weights enter as exact integers, the group scale
  multiplies f32 group sums — gated at the GEMV's tolerance (`row_gate`: atol 3e-5 times the
  row's largest |x|, rtol 1e-5).
* fp16-weight kernels (smaller shapes under KRM_COMPUTE_F16): x rounded to fp16, each weight
  dequantised to fp16 as fp16((u-8) * scale) — one fp16 rounding, relative error <= 2^-11 — and
  products accumulated in f32.  With K terms of typical size t the error of an output behaves
  like sqrt(K) * t * 2^-11 / sqrt(3); those tests scale their tolerance with the RMS of the
  oracle's output:  |got - want| <= 2e-3 * rms(want) + 1e-3 * |want|  (measured worst case about
  a third of that).  When every scale is a power of two the dequantised weights are exact and
  the gate tightens to f32-accumulation level (atol 3e-5 * rms, measured ~5e-6).
"""
import numpy as np
import pytest

import helpers
import karume_amd as ka
from helpers import oracle
from test_gpu_linear import run_linear

pytestmark = pytest.mark.gpu


def sampled_oracle(x, packed, scale, bias, n, k, g, cols):
    """Oracle output restricted to a sample of output columns (weight rows)."""
    rows = packed.reshape(n, k // 2)[cols]
    return oracle.linear_i4(x, rows.reshape(-1), scale[cols], bias[cols], len(cols), k, g)


def check(got, want, exact_weights=False):
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    err = np.abs(got.astype(np.float64) - want)
    if exact_weights:
        bound = 3e-5 * rms + 1e-6 * np.abs(want)
    else:
        bound = 2e-3 * rms + 1e-3 * np.abs(want)
    worst = float(np.max(err / bound))
    assert worst <= 1.0, (worst, float(err.max()), rms)
    return worst


@pytest.mark.parametrize("m,n,k,g", [(512, 11008, 4096, 128), (512, 4096, 11008, 128)])
@pytest.mark.parametrize("io", [np.float16, np.float32])
def test_config1_prefill_gemm(gpu_ctx, m, n, k, g, io):
    """benchmark config 1 at full size (up- and down-projection); 192 sampled output columns
    are checked against the f64 oracle, all rows."""
    rng = np.random.default_rng(n + k)
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(m, k)).astype(np.float16)
    bias = rng.normal(size=n).astype(np.float16)
    got = run_linear(gpu_ctx, x.astype(io), packed, scale, bias, n, k, g, compute=ka.COMPUTE_F16)
    cols = np.sort(rng.choice(n, size=192, replace=False))
    cols[:3] = [0, 1, 63]
    cols[-3:] = [n - 65, n - 2, n - 1]
    cols = np.unique(cols)
    want = sampled_oracle(x.astype(np.float32), packed, scale.astype(np.float32),
                          bias.astype(np.float32), n, k, g, cols)
    got_cols = got[:, cols].astype(np.float32)
    if io == np.float16:  # add the output rounding to the budget: half an fp16 ulp of |want|
        rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
        err = np.abs(got_cols - want)
        bound = 2e-3 * rms + 1.5e-3 * np.abs(want) + 1e-3
        assert np.all(err <= bound), float(np.max(err / bound))
    else:
        check(got_cols, want)


@pytest.mark.parametrize("shape", [(17, 64, 64, 16), (65, 68, 48, 16), (130, 200, 96, 32),
                                   (100, 129, 320, 64), (300, 1000, 2048, 128),
                                   (64, 256, 512, 128), (33, 8, 128, 128),
                                   # enough 128 x 256 tiles for the packed-weights form, with
                                   # ragged edges in M, N and K (K ends inside a 128-code stage)
                                   (300, 13349, 320, 64),
                                   # the same with a K long enough for the (tile, stage) units to
                                   # be dealt over the CUs: tiles shared by 2-3 workgroups
                                   (300, 13349, 2624, 64)])
def test_gemm_edges_exact_weights(gpu_ctx, shape):
    """Tile edges in M, N and K (K not a multiple of the 64-code stage, N not a multiple of
    the tile) with power-of-two scales: dequantised weights are exact in fp16, x is fp16, so
    only the f32 accumulation order differs from the oracle."""
    m, n, k, g = shape
    rng = np.random.default_rng(m * 1000 + n)
    q = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    scale = (2.0 ** rng.integers(-8, -3, size=(n, k // g))).astype(np.float32)
    packed = oracle.pack_i4(q)
    x = rng.normal(size=(m, k)).astype(np.float16).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32)
    want = oracle.linear_i4(x, packed, scale, bias, n, k, g)
    got = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g, compute=ka.COMPUTE_F16)
    check(got, want, exact_weights=True)
    got_h = run_linear(gpu_ctx, x.astype(np.float16), packed, scale.astype(np.float16),
                       bias.astype(np.float16), n, k, g, compute=ka.COMPUTE_F16)
    want_h = oracle.linear_i4(x, packed, scale, bias.astype(np.float16).astype(np.float32), n, k,
                              g)
    assert np.max(np.abs(got_h.astype(np.float32) - want_h)
                  - 1e-3 * np.abs(want_h)) <= 2e-3  # fp16 output rounding


def test_gemm_with_tiles_shared_between_workgroups_is_reproducible(gpu_ctx):
    """86 tiles of 32 stages on 256 CUs: the (tile, stage) units are dealt 10 or 11 to a
    workgroup, so every tile is the sum of 3-4 partials added by whichever workgroup arrives
    last.  The sum is taken in K order whoever that is: repeated runs give the same bits, and
    the result meets the exact-weights gate."""
    m, n, k, g = 256, 11008, 4096, 128
    rng = np.random.default_rng(77)
    q = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    scale = (2.0 ** rng.integers(-8, -3, size=(n, k // g))).astype(np.float32)
    packed = oracle.pack_i4(q)
    x = rng.normal(size=(m, k)).astype(np.float16).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32)
    first = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g, compute=ka.COMPUTE_F16)
    for _ in range(4):
        again = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g, compute=ka.COMPUTE_F16)
        assert np.array_equal(first.view(np.uint32), again.view(np.uint32))
    check(first, oracle.linear_i4(x, packed, scale, bias, n, k, g), exact_weights=True)


def test_gemm_reference_cases(gpu_ctx):
    """The reference's tile-edge shapes with its own generators (M = 65 and 17 take the MFMA
    path with KRM_COMPUTE_F16); arbitrary f32 scales, f32 x that is not fp16-representable."""
    for case in helpers.I4_LINEAR_CASES[:2]:
        x, packed, _q, scale, bias = helpers.make_i4_linear(case)
        want = oracle.linear_i4(x, packed, scale, bias, case.n, case.k, case.group)
        got = run_linear(gpu_ctx, x, packed, scale, bias, case.n, case.k, case.group,
                         compute=ka.COMPUTE_F16)
        check(got, want)


def test_gemm_f32_mode_stays_on_f32_arithmetic(gpu_ctx):
    """KRM_COMPUTE_F32 with M > 16 keeps f32 products and accumulation (the GEMV over row
    blocks): same gate as the GEMV tests (atol 3e-5, rtol 1e-5), far tighter than fp16."""
    rng = np.random.default_rng(5)
    m, n, k, g = 40, 512, 1024, 128
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(m, k)).astype(np.float32)  # not fp16-representable
    bias = rng.normal(size=n).astype(np.float32)
    want = oracle.linear_i4(x, packed, scale.astype(np.float32), bias, n, k, g)
    got = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g, compute=ka.COMPUTE_F32)
    ok, fails, max_abs, worst = oracle.allclose(got, want, atol=3e-5, rtol=1e-5)
    assert ok, (fails, max_abs, worst)


def row_gate(x):
    """Absolute tolerance per output row of the exact-operand forms: the GEMV's gate
    (atol 3e-5 for activations of unit size, rtol 1e-5) scaled with the row's largest |x|."""
    top = np.max(np.abs(np.where(np.isfinite(x), x, 0.0)), axis=1, keepdims=True)
    return 3e-5 * np.maximum(top, 1e-30)


@pytest.mark.parametrize("m,n,k,g", [(512, 11008, 4096, 128), (512, 4096, 11008, 128)])
def test_config1_f32_class_runs_on_the_matrix_cores_within_the_gemv_gate(gpu_ctx, m, n, k, g):
    """KRM_COMPUTE_F32 with f32 activations at benchmark config 1's shapes: the activations are
    split into fp16 hi + lo (22 bits, scaled per row), the weights enter as exact integers, the
    group scale multiplies f32 group sums.  Rows of very different magnitude (1e5, 1e-6, beyond
    the fp16 range in both directions), a row of zeros and values that are not
    fp16-representable; 160 sampled columns against the f64 oracle at the GEMV's gate."""
    rng = np.random.default_rng(n * 3 + k)
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[3] *= 1e5
    x[4] *= 3e7
    x[5] *= 1e-6
    x[6] *= 1e-30
    x[7] = 0.0
    x[8, ::2] *= 1e-4          # wide dynamic range inside one row
    bias = rng.normal(size=n).astype(np.float32)
    got = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g, compute=ka.COMPUTE_F32)
    cols = np.unique(np.concatenate([[0, 1, 63, 64, 511, 512, n - 513, n - 65, n - 2, n - 1],
                                     rng.choice(n, size=150, replace=False)]))
    want = sampled_oracle(x, packed, scale.astype(np.float32), bias, n, k, g, cols)
    err = np.abs(got[:, cols].astype(np.float64) - want)
    bound = row_gate(x) + 1e-5 * np.abs(want)
    assert np.all(err <= bound), float(np.max(err / bound))
    assert np.all(got[7] == bias)      # the row of zeros: exactly the bias


@pytest.mark.parametrize("io", [np.float16, np.float32])
def test_config1_f16_operands_are_exact_integers_times_fp16_x(gpu_ctx, io):
    """KRM_COMPUTE_F16 at config 1's up-projection: with fp16-representable activations every
    product is exact and the group scale multiplies f32 sums, so the result meets the GEMV's
    gate (the per-weight fp16 rounding of the small-shape kernels is gone here)."""
    m, n, k, g = 512, 11008, 4096, 128
    rng = np.random.default_rng(91)
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(m, k)).astype(np.float16)
    bias = rng.normal(size=n).astype(np.float16)
    got = run_linear(gpu_ctx, x.astype(io), packed, scale, bias.astype(io), n, k, g,
                     compute=ka.COMPUTE_F16)
    cols = np.unique(rng.choice(n, size=128, replace=False))
    want = sampled_oracle(x.astype(np.float32), packed, scale.astype(np.float32),
                          bias.astype(np.float32), n, k, g, cols)
    err = np.abs(got[:, cols].astype(np.float64) - want)
    bound = row_gate(x.astype(np.float32)) + 1e-5 * np.abs(want)
    if io == np.float16:                # the output rounding: half an fp16 ulp of |want|
        bound = bound + 2.0 ** -11 * np.abs(want) + 1e-7
    assert np.all(err <= bound), float(np.max(err / bound))


def test_f32_class_gemm_edges_and_non_finite_rows(gpu_ctx):
    """Ragged M, N and K (K ends inside a 128-code stage, two scale groups a stage), f32 scales,
    and rows holding Inf / NaN: those rows come out non-finite where the oracle's do, every
    other row meets the gate."""
    m, n, k, g = 300, 13349, 2624, 64
    rng = np.random.default_rng(12)
    q = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    scale = np.abs(rng.normal(0, 0.02, size=(n, k // g))).astype(np.float32) + 1e-4
    packed = oracle.pack_i4(q)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[11, 5] = np.inf
    x[12, 2000] = np.nan
    bias = rng.normal(size=n).astype(np.float32)
    got = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g, compute=ka.COMPUTE_F32)
    cols = np.unique(np.concatenate([[0, 511, 512, n - 1], rng.choice(n, size=60, replace=False)]))
    want = sampled_oracle(x, packed, scale, bias, n, k, g, cols)
    finite = np.ones(m, dtype=bool)
    finite[[11, 12]] = False
    err = np.abs(got[finite][:, cols].astype(np.float64) - want[finite])
    bound = row_gate(x[finite]) + 1e-5 * np.abs(want[finite])
    assert np.all(err <= bound), float(np.max(err / bound))
    assert not np.any(np.isfinite(got[[11, 12]][:, cols]))
    assert not np.any(np.isfinite(want[[11, 12]]))


# ---------------------------------------------------------------- few rows (a prefill chunk)

def run_rows(ctx, x, packed, scale, bias, n, k, group, compute, residual=None,
             epilogue=ka.EPILOGUE_NONE):
    x = np.ascontiguousarray(x)
    m = x.shape[0]
    n_out = n // 2 if epilogue == ka.EPILOGUE_SILU_PAIRS else n
    dx, dw, ds = ctx.upload(x), ctx.upload(packed), ctx.upload(np.ascontiguousarray(scale))
    db = ctx.upload(np.ascontiguousarray(bias, dtype=x.dtype)) if bias is not None else None
    dr = ctx.upload(np.ascontiguousarray(residual, dtype=x.dtype)) if residual is not None else None
    out = ctx.alloc(max(m * n_out * x.itemsize, 16))
    ctx.linear_i4_rows(dx, dw, ds, out, m, n, k, group, bias=db, residual=dr,
                       io_dtype=ka.dtype_code(x.dtype), scale_dtype=ka.dtype_code(scale.dtype),
                       compute=compute, epilogue=epilogue)
    got = out.download(x.dtype, (m, n_out))
    for b in (dx, dw, ds, out, db, dr):
        if b is not None:
            b.free()
    return got


ROWS_SHAPES = [(128, 2560, 2048, 128),   # a 128-row chunk of the benchmark decoder: [q; k; v]
               (128, 2048, 5632, 128),   # its down-projection: 44 groups over 8 waves
               (40, 512, 1024, 128), (100, 129, 320, 64), (257, 96, 4096, 256),
               (100, 2700, 1088, 64),    # 64-column tiles; K ends inside a chunk's second half
               (17, 33, 192, 64),        # fewer 64-code chunks than waves
               (1, 64, 2048, 128)]


@pytest.mark.parametrize("m,n,k,g", ROWS_SHAPES)
@pytest.mark.parametrize("mode", ["f32", "f16 on f32", "f16"])
def test_few_row_products_meet_the_gemv_gate(gpu_ctx, m, n, k, g, mode):
    """Shapes too small for the 64 x 512 deal run on the few-row kernel (eight waves split K):
    exact integer weights and f32 group sums, so the f32 class (x split hi + lo) and the fp16
    class (x rounded to fp16 once: the oracle is given the rounded x) both meet the GEMV's
    gate.  Ragged M, N, K, a single row and a K shorter than eight chunks included."""
    rng = np.random.default_rng(m * 7 + n + k)
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[0] *= 300.0
    if m > 2:
        x[2] *= 1e-3
    bias = rng.normal(size=n).astype(np.float32)
    if mode == "f32":
        got = run_rows(gpu_ctx, x, packed, scale, bias, n, k, g, ka.COMPUTE_F32)
        seen = x
    elif mode == "f16 on f32":
        got = run_rows(gpu_ctx, x, packed, scale, bias, n, k, g, ka.COMPUTE_F16)
        seen = x.astype(np.float16).astype(np.float32)
    else:
        got = run_rows(gpu_ctx, x.astype(np.float16), packed, scale, bias, n, k, g,
                       ka.COMPUTE_F16)
        seen = x.astype(np.float16).astype(np.float32)
        bias = bias.astype(np.float16).astype(np.float32)
    if m > 16 and mode != "f16":   # krm_linear_i4 takes the same kernel for these shapes
        compute = ka.COMPUTE_F32 if mode == "f32" else ka.COMPUTE_F16
        same = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g, compute=compute)
        assert np.array_equal(got.view(np.uint32), same.view(np.uint32))
    want = oracle.linear_i4(seen, packed, scale.astype(np.float32), bias, n, k, g)
    err = np.abs(got.astype(np.float64) - want)
    bound = row_gate(seen) + 1e-5 * np.abs(want)
    if mode == "f16":
        bound = bound + 2.0 ** -11 * np.abs(want) + 1e-7
    assert np.all(err <= bound), float(np.max(err / bound))


def test_few_row_epilogues_against_the_oracle_and_the_separate_ops(gpu_ctx):
    """residual add and the gate/up pairs folded into the few-row kernel: equal to the plain
    call followed by the oracle's add / silu-mul within one rounding of the stored type, and
    the oracle's own chain within the gate."""
    rng = np.random.default_rng(404)
    m, n, k, g = 96, 1408, 2048, 128
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(m, k)).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32)
    residual = rng.normal(size=(m, n)).astype(np.float32)
    plain = run_rows(gpu_ctx, x, packed, scale, bias, n, k, g, ka.COMPUTE_F32)
    via_linear = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g, compute=ka.COMPUTE_F32)
    assert np.array_equal(plain.view(np.uint32), via_linear.view(np.uint32))
    with_res = run_rows(gpu_ctx, x, packed, scale, bias, n, k, g, ka.COMPUTE_F32, residual=residual)
    assert np.array_equal(with_res.view(np.uint32), (plain + residual).view(np.uint32))
    # pairs: rows (2i, 2i+1) of w are (gate_i, up_i)
    paired = run_rows(gpu_ctx, x, packed, scale, bias, n, k, g, ka.COMPUTE_F32,
                      epilogue=ka.EPILOGUE_SILU_PAIRS)
    want = oracle.linear_i4(x, packed, scale.astype(np.float32), bias, n, k, g)
    chain = oracle.silu_mul(want[:, 0::2].astype(np.float32), want[:, 1::2].astype(np.float32))
    scale_of = np.abs(want[:, 0::2]) * np.abs(want[:, 1::2]) + np.abs(want[:, 1::2]) + 1.0
    assert np.all(np.abs(paired.astype(np.float64) - chain) <= 1e-4 * scale_of)
    separate = oracle.silu_mul(plain[:, 0::2].copy(), plain[:, 1::2].copy())
    assert np.all(np.abs(paired - separate) <= 4e-6 * scale_of)
    # fp16 storage, the wide (64-column) tiles: n / 32 x m / 64 workgroups beyond two a CU
    m, n, k, g = 128, 11264, 2048, 128
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(m, k)).astype(np.float16)
    paired = run_rows(gpu_ctx, x, packed, scale, None, n, k, g, ka.COMPUTE_F16,
                      epilogue=ka.EPILOGUE_SILU_PAIRS)
    cols = np.unique(rng.choice(n // 2, size=96, replace=False))
    rows = np.stack([2 * cols, 2 * cols + 1], axis=1).reshape(-1)
    want = sampled_oracle(x.astype(np.float32), packed, scale.astype(np.float32),
                          np.zeros(n, dtype=np.float32), n, k, g, rows)
    chain = oracle.silu_mul(want[:, 0::2].astype(np.float32), want[:, 1::2].astype(np.float32))
    err = np.abs(paired[:, cols].astype(np.float64) - chain)
    assert np.all(err <= 1e-3 * np.abs(chain) + 1e-3), float(err.max())


def test_few_row_kernel_rejects_what_it_does_not_cover(gpu_ctx):
    rng = np.random.default_rng(1)
    packed, _q, scale = helpers.synthetic_int4(rng, 64, 64, 16)
    x = rng.normal(size=(20, 64)).astype(np.float32)
    with pytest.raises(ka.GpuValidationError, match="group_size >= 64"):
        run_rows(gpu_ctx, x, packed, scale, None, 64, 64, 16, ka.COMPUTE_F32)
    with pytest.raises(ka.GpuValidationError, match="even n"):
        packed, _q, scale = helpers.synthetic_int4(rng, 33, 128, 64)
        run_rows(gpu_ctx, rng.normal(size=(20, 128)).astype(np.float32), packed, scale, None, 33,
                 128, 64, ka.COMPUTE_F32, epilogue=ka.EPILOGUE_SILU_PAIRS)


@pytest.mark.parametrize("compute", [ka.COMPUTE_F32, ka.COMPUTE_F16])
def test_few_row_results_do_not_depend_on_the_batch(gpu_ctx, compute):
    """In the reference an output row has the same bits whatever M is
    (packages/runtime/tests/gpu_gemm_skinny_test.ts:11-15,156-198).  The few-row kernel keeps
    that: a row's products, its split over the eight waves (a function of K) and the order of the
    final sum do not depend on the other rows, on the row's place in the chunk, or on the tile
    width chosen for the chunk (32 or 64 columns)."""
    rng = np.random.default_rng(808)
    n, k, g = 4224, 1024, 128      # 128 rows: 4 x 132 tiles > 256 CUs -> 64-column tiles
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(128, k)).astype(np.float32)
    x[5] *= 1e4
    bias = rng.normal(size=n).astype(np.float32)
    whole = run_rows(gpu_ctx, x, packed, scale, bias, n, k, g, compute)
    for rows in ([5], [0, 5, 77], list(range(40, 73))):   # 1, 3 and 33 rows: 32-column tiles
        part = run_rows(gpu_ctx, x[rows], packed, scale, bias, n, k, g, compute)
        assert np.array_equal(part.view(np.uint32), whole[rows].view(np.uint32)), rows
