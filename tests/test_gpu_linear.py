"""GPU parity of the int4 dequant kernel and the `linear` op (through the C ABI) against the
CPU oracle.  Tolerances are written where they are used and follow the reference's rule for
kernels whose reduction order differs from the oracle's: measure, then add margin
(docs/decisions/0022-gemm-register-blocking.md:22-24)."""
import numpy as np
import pytest

import helpers
import karume_amd as ka
from helpers import oracle

pytestmark = pytest.mark.gpu


def run_dequant(ctx, packed, scale, rows, width, group):
    scale = np.ascontiguousarray(scale)
    w = ctx.upload(packed)
    s = ctx.upload(scale)
    out = ctx.alloc(rows * width * 4)
    ctx.dequant_i4(w, s, out, rows, width, group, ka.dtype_code(scale.dtype))
    got = out.download(np.float32, (rows, width))
    for b in (w, s, out):
        b.free()
    return got


def run_linear(ctx, x, packed, scale, bias, n, k, group, compute=ka.COMPUTE_F32):
    """x: [m, k] float32 or float16 array (its dtype selects the io dtype)."""
    x = np.ascontiguousarray(x)
    scale = np.ascontiguousarray(scale)
    m = x.shape[0]
    dx, dw, ds = ctx.upload(x), ctx.upload(packed), ctx.upload(scale)
    db = ctx.upload(np.ascontiguousarray(bias, dtype=x.dtype)) if bias is not None else None
    out = ctx.alloc(max(m * n * x.itemsize, 16))
    ctx.linear_i4(dx, dw, ds, db, out, m, n, k, group, ka.dtype_code(x.dtype),
                  ka.dtype_code(scale.dtype), compute)
    got = out.download(x.dtype, (m, n))
    for b in (dx, dw, ds, out) + ((db,) if db is not None else ()):
        b.free()
    return got


def test_dequant_bit_exact_all_codes_all_positions(gpu_ctx):
    """All 16 codes x 8 in-word positions with row x group varying scales: GPU bits == decodeI4
    bits (packages/runtime/tests/gpu_i4_weights_test.ts:404-459, extended to u = 0)."""
    rows, width, g = 16, 32, 16
    q = np.array([(r + c) % 16 - 8 for r in range(rows) for c in range(width)], dtype=np.int8)
    scale = np.array([[0.1 + 0.017 * r + 0.31 * gi for gi in range(width // g)]
                      for r in range(rows)], dtype=np.float32)
    packed = oracle.pack_i4(q)
    want = oracle.decode_i4(packed, [rows, width], scale, [rows, width // g], g)
    got = run_dequant(gpu_ctx, packed, scale, rows, width, g)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("scale_dtype", [np.float32, np.float16])
def test_dequant_bit_exact_random(gpu_ctx, scale_dtype):
    rng = np.random.default_rng(21)
    rows, width, g = 67, 384, 128
    packed, _q, scale = helpers.synthetic_int4(rng, rows, width, g, scale_f16=True)
    scale = scale.astype(scale_dtype)
    if scale_dtype == np.float32:  # arbitrary f32 scales: the product rounds, once
        scale = (scale.astype(np.float32) * np.float32(1.2345678)).astype(np.float32)
    want = oracle.decode_i4(packed, [rows, width], scale.astype(np.float32),
                            [rows, width // g], g)
    got = run_dequant(gpu_ctx, packed, scale, rows, width, g)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("case", helpers.I4_LINEAR_CASES, ids=lambda c: c.name)
def test_linear_reference_cases_f32(gpu_ctx, case):
    """The reference's tile-edge shapes (gpu_i4_weights_test.ts:116-145), f32 in/out, f32
    scales.  |out| reaches ~1e3 here; gate: the reference's default allclose (atol 1e-5,
    rtol 1e-3) AND a tighter atol 2e-3 / rtol 2e-6 derived from f32 accumulation of ~1e3-sized
    partial sums (measured worst 2.4e-4)."""
    x, packed, _q, scale, bias = helpers.make_i4_linear(case)
    want = oracle.linear_i4(x, packed, scale, bias, case.n, case.k, case.group)
    got = run_linear(gpu_ctx, x, packed, scale, bias, case.n, case.k, case.group)
    ok, fails, max_abs, worst = oracle.allclose(got, want, atol=1e-5, rtol=1e-3)
    assert ok, (fails, max_abs, worst)
    ok, fails, max_abs, worst = oracle.allclose(got, want, atol=2e-3, rtol=2e-6)
    assert ok, (fails, max_abs, worst)


def test_linear_packed_equals_preexpanded_through_same_kernel(gpu_ctx):
    """Invariant of gpu_i4_weights_test.ts:262-298 restated for this backend: weights with
    scale 1 and the same codes must give exactly sum(q * x) — integer arithmetic, bit-exact —
    and scaling every group by a power of two must scale the output exactly."""
    rng = np.random.default_rng(2)
    n, k, g = 40, 256, 32
    q = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    x = rng.integers(-4, 5, size=(3, k)).astype(np.float32)
    packed = oracle.pack_i4(q)
    ones = np.ones((n, k // g), dtype=np.float32)
    got = run_linear(gpu_ctx, x, packed, ones, None, n, k, g)
    want = (x.astype(np.int64) @ q.astype(np.int64).T).astype(np.float32)
    assert np.array_equal(got, want)
    got4 = run_linear(gpu_ctx, x, packed, ones * 0.25, None, n, k, g)
    assert np.array_equal(got4, want * 0.25)


@pytest.mark.parametrize("io", [np.float16, np.float32])
def test_linear_config0_gemv(gpu_ctx, io):
    """benchmark config 0: M=1, K=N=4096, int4 g128, fp16 scales |N(0,0.02)|, x ~ N(0,1) in fp16.
    f32 output: atol 2e-5 (|out| ~ 5, f32 accumulation; measured worst 4e-6), rtol 0.
    fp16 output: the oracle's f32 result rounded to fp16, within 1 fp16 ulp."""
    rng = np.random.default_rng(40960)
    n = k = 4096
    g = 128
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(1, k)).astype(np.float16)
    want = oracle.linear_i4(x.astype(np.float32), packed, scale.astype(np.float32),
                            np.zeros(n, dtype=np.float32), n, k, g)
    got = run_linear(gpu_ctx, x.astype(io), packed, scale, None, n, k, g)
    if io == np.float32:
        ok, fails, max_abs, worst = oracle.allclose(got, want, atol=2e-5, rtol=0)
        assert ok, (fails, max_abs, worst)
    else:
        want16 = want.astype(np.float16)
        ulp = np.abs(np.nextafter(want16, np.float16(np.inf)).astype(np.float32)
                     - want16.astype(np.float32))
        assert np.all(np.abs(got.astype(np.float32) - want16.astype(np.float32)) <= ulp)


@pytest.mark.parametrize("io", [np.float16, np.float32])
def test_linear_batched_rows_equal_single_rows_bitwise(gpu_ctx, io):
    """benchmark config 3 (GEMV part): M = 16 in one launch vs the rows in smaller launches.
    f32 activations: the per-row reduction order does not depend on M, so the bits agree with
    single-row launches.  fp16 activations: batches of 2..16 rows run on the matrix cores,
    where a row's bits do not depend on the batch it sits in; a single row takes the
    dot-product kernel and agrees to the output's rounding."""
    rng = np.random.default_rng(16)
    n = k = 4096
    g = 128
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(16, k)).astype(np.float16).astype(io)
    batched = run_linear(gpu_ctx, x, packed, scale, None, n, k, g)
    for m_sub in (2, 5):
        part = run_linear(gpu_ctx, x[:m_sub], packed, scale, None, n, k, g)
        assert np.array_equal(part.view(np.uint8), batched[:m_sub].view(np.uint8)), m_sub
    pair = run_linear(gpu_ctx, x[10:12], packed, scale, None, n, k, g)
    assert np.array_equal(pair.view(np.uint8), batched[10:12].view(np.uint8))
    single = run_linear(gpu_ctx, x[11:12], packed, scale, None, n, k, g)
    if io == np.float32:
        assert np.array_equal(single.view(np.uint8), batched[11:12].view(np.uint8))
    else:
        a, b = single.astype(np.float32), batched[11:12].astype(np.float32)
        # both round an f32-accurate sum (each within 2e-5 of the exact one): at most one fp16
        # ulp apart, plus that noise where the output is tiny
        assert np.all(np.abs(a - b) <= 2.0 ** -10 * np.maximum(np.abs(a), np.abs(b)) + 4e-5)
    want = oracle.linear_i4(x.astype(np.float32), packed, scale.astype(np.float32),
                            np.zeros(n, dtype=np.float32), n, k, g)
    tol = 2e-5 if io == np.float32 else 8e-3  # fp16 output: half an ulp at |out| < 16
    assert np.max(np.abs(batched.astype(np.float32) - want)) <= tol


@pytest.mark.parametrize("m,n,k,g,scale_f16,with_bias", [
    (2, 16, 1024, 128, True, False), (16, 4096, 4096, 128, True, True),
    (7, 100, 2048, 128, False, True), (16, 33, 8192, 256, True, False),
    (3, 250, 3072, 128, True, True), (16, 64, 5120, 1024, False, False),
    # K a multiple of 256 only: the chunks are dealt unevenly to the waves (some get none)
    (16, 2048, 5632, 128, True, True), (5, 100, 11008, 128, True, False),
    (3, 40, 256, 128, False, True), (16, 64, 768, 256, True, False)])
def test_batched_fp16_rows_on_matrix_cores_match_oracle(gpu_ctx, m, n, k, g, scale_f16, with_bias):
    """2..16 fp16 rows take the MFMA kernel (K a multiple of 256, group >= 128): ragged N,
    every compile-time chunk count and the loop form (K = 3072, 5120), group sizes up to
    1024, f32 and fp16 scales, bias.  Gate: the oracle's f32 result rounded to fp16, one ulp."""
    rng = np.random.default_rng(m * 1000 + n)
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g, scale_f16=scale_f16)
    x = rng.normal(size=(m, k)).astype(np.float16)
    bias = rng.normal(size=n).astype(np.float16) if with_bias else None
    got = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g)
    want = oracle.linear_i4(x.astype(np.float32), packed, scale.astype(np.float32),
                            (bias if with_bias else np.zeros(n)).astype(np.float32), n, k, g)
    err = np.abs(got.astype(np.float32) - want)
    assert np.all(err <= 2.0 ** -10 * np.abs(want) + 4e-5), float(err.max())


@pytest.mark.parametrize("shape", [(1, 256, 2048, 128), (3, 2048, 5632, 128), (1, 100, 11008, 128),
                                   (7, 33, 96, 32), (2, 5, 64, 16), (16, 32000, 2048, 128)])
def test_linear_shapes_of_the_decoder(gpu_ctx, shape):
    """The GEMV over the layer shapes of the 1.1B decoder (N x K) and ragged edges; f32 io,
    gate atol 3e-5 rtol 1e-5 against the f64 oracle (measured worst 6e-6)."""
    m, n, k, g = shape
    rng = np.random.default_rng(n * 7 + k)
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(m, k)).astype(np.float16).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32)
    want = oracle.linear_i4(x, packed, scale.astype(np.float32), bias, n, k, g)
    got = run_linear(gpu_ctx, x, packed, scale, bias, n, k, g)
    ok, fails, max_abs, worst = oracle.allclose(got, want, atol=3e-5, rtol=1e-5)
    assert ok, (fails, max_abs, worst)


@pytest.mark.parametrize("k,io,many", [(2048, np.float32, 8256), (5632, np.float32, 8256),
                                       (4096, np.float16, 8256), (4096, np.float16, 16512)])
def test_row_bits_do_not_depend_on_rows_per_wave(gpu_ctx, k, io, many):
    """A narrow output gives a wave one row, a wide one two (K = 5632, or fp16) or four
    (K = 2048 with f32 activations, fp16 activations from 16384 rows) that are reduced together:
    the same weight row and x give the same bits either way (one fixed order of additions for
    every form of the wave reduction)."""
    g, few = 128, 64
    rng = np.random.default_rng(k)
    packed, _q, scale = helpers.synthetic_int4(rng, many, k, g)
    x = rng.normal(size=(1, k)).astype(io)
    wide = run_linear(gpu_ctx, x, packed, scale, None, many, k, g)
    narrow = run_linear(gpu_ctx, x, packed.reshape(-1)[:few * k // 2], scale[:few], None, few, k, g)
    assert wide[:, :few].tobytes() == narrow.tobytes()


def test_linear_rejections(gpu_ctx):
    """Unsupported combinations fail before launch (never approximated)."""
    buf = gpu_ctx.zeros(4096)
    with pytest.raises(ka.GpuValidationError):  # group does not divide k
        gpu_ctx.linear_i4(buf, buf, buf, None, buf, 1, 4, 48, 32)
    with pytest.raises(ka.GpuValidationError):  # group not a power of two >= 16
        gpu_ctx.linear_i4(buf, buf, buf, None, buf, 1, 4, 48, 24)
    with pytest.raises(ka.GpuValidationError):
        gpu_ctx.linear_i4(buf, buf, buf, None, buf, 1, 4, 64, 8)
    with pytest.raises(ka.GpuValidationError):  # NULL weights
        gpu_ctx.linear_i4(buf, None, buf, None, buf, 1, 4, 64, 32)
    with pytest.raises(ka.GpuValidationError):
        gpu_ctx.dequant_i4(buf, buf, buf, 2, 8, 3)
    buf.free()


def test_linear_fused_decode_forms(gpu_ctx):
    """krm_linear_i4_fused: rms_norm folded in front, residual and silu(gate)*up folded behind,
    against the oracle's op chain rms_norm -> linear -> (+ residual | silu*mul).  f32 io: atol
    3e-5 rtol 2e-5 (the normalised row is not rounded between the ops here, so the result sits
    slightly closer to the f64 chain than the unfused launches do)."""
    rng = np.random.default_rng(8)
    # (1, 72, 8192, 128): K too long for registers, the prefetching loop with the norm in front
    for m, n, k, g in [(1, 2560, 2048, 128), (3, 512, 1024, 128), (1, 64, 256, 32), (2, 40, 96, 16),
                       (1, 72, 8192, 128)]:
        packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
        x = (rng.normal(size=(m, k)) * 5).astype(np.float32)
        gamma = rng.normal(size=k).astype(np.float32)
        res = rng.normal(size=(m, n)).astype(np.float32)
        sf = scale.astype(np.float32)
        zeros = np.zeros(n, dtype=np.float32)
        xn = oracle.rms_norm(x, gamma, 1e-5)
        lin = oracle.linear_i4(xn, packed, sf, zeros, n, k, g)
        bufs = [gpu_ctx.upload(a) for a in (x, packed, scale, gamma, res)]
        dx, dw, ds, dg, dr = bufs
        out = gpu_ctx.alloc(m * n * 4)
        # norm + linear + residual
        gpu_ctx.linear_i4_fused(dx, dw, ds, out, m, n, k, g, norm_weight=dg, norm_eps=1e-5,
                                residual=dr, scale_dtype=ka.F16)
        got = out.download(np.float32, (m, n))
        ok, fails, max_abs, worst = oracle.allclose(got, lin + res, atol=3e-5, rtol=2e-5)
        assert ok, (m, n, k, fails, max_abs, worst)
        # in place on the residual buffer
        gpu_ctx.linear_i4_fused(dx, dw, ds, dr, m, n, k, g, residual=dr, scale_dtype=ka.F16)
        plain = oracle.linear_i4(x, packed, sf, zeros, n, k, g)
        ok, fails, max_abs, worst = oracle.allclose(dr.download(np.float32, (m, n)), plain + res,
                                                    atol=2e-4, rtol=2e-5)
        assert ok, (fails, max_abs, worst)
        # norm + interleaved gate/up + silu*mul
        gpu_ctx.linear_i4_fused(dx, dw, ds, out, m, n, k, g, norm_weight=dg, norm_eps=1e-5,
                                scale_dtype=ka.F16, epilogue=ka.EPILOGUE_SILU_PAIRS)
        got = out.download(np.float32, (m, n // 2))
        want = oracle.silu_mul(lin[:, 0::2], lin[:, 1::2])
        ok, fails, max_abs, worst = oracle.allclose(got, want, atol=3e-5, rtol=5e-5)
        assert ok, (fails, max_abs, worst)
        for b in bufs + [out]:
            b.free()
    buf = gpu_ctx.zeros(1 << 16)
    with pytest.raises(ka.GpuValidationError):  # prefill chunks use the separate ops
        gpu_ctx.linear_i4_fused(buf, buf, buf, buf, 17, 64, 128, 128)
    with pytest.raises(ka.GpuValidationError):
        gpu_ctx.linear_i4_fused(buf, buf, buf, buf, 1, 63, 128, 128,
                                epilogue=ka.EPILOGUE_SILU_PAIRS)
    buf.free()


def test_linear_from_a_model_file(gpu_ctx):
    """File -> reader -> device: an int4 `linear` weight written as an I4 tensor with its F32
    group scale is handed to the kernel as the reader's views of the file (no re-packing) and
    must match the oracle run on the same bytes.  Gate as in the reference cases above."""
    import json
    from karume_amd.format_model import (build_safetensors, i4_resident_initializers, open_model,
                                         packed_int4)
    rng = np.random.default_rng(11)
    n, k, g, m = 96, 512, 64, 3
    q = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    scale = rng.uniform(0.005, 0.05, size=(n, k // g)).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32)
    graph = {
        "format": "karume-ir", "version": 1, "requires": {"ops": ["linear"]}, "symbols": [],
        "inputs": [{"name": "x", "dtype": "f32", "shape": [m, k]}], "outputs": ["y"],
        "initializers": {
            "w": {"tensor": "proj.weight",
                  "storage": {"dtype": "i4", "scale": "karume.scale.proj.weight", "group_size": g}},
            "b": {"tensor": "proj.bias", "storage": {"dtype": "f32"}}},
        "values": {"w": {"dtype": "f32", "shape": [n, k]}, "b": {"dtype": "f32", "shape": [n]},
                   "y": {"dtype": "f32", "shape": [m, n]}},
        "nodes": [{"op": "linear", "ins": ["x", "w", "b"], "outs": ["y"], "attrs": {}}]}
    blob = build_safetensors(
        [("karume.scale.proj.weight", "F32", [n, k // g], scale.tobytes()),
         ("proj.bias", "F32", [n], bias.tobytes()),
         ("proj.weight", "I4", [n, k], oracle.pack_i4(q).tobytes())],
        {"karume_ir": json.dumps(graph)})
    model = open_model(blob)
    assert i4_resident_initializers(model) == {"w"}
    weight = packed_int4(model, "w")
    x = rng.normal(size=(m, k)).astype(np.float32)
    want = oracle.linear_i4(x, weight.packed, weight.scales, bias, n, k, g)
    got = run_linear(gpu_ctx, x, weight.packed, weight.scales, bias, n, k, g)
    ok, fails, max_abs, worst = oracle.allclose(got, want, atol=1e-5, rtol=1e-3)
    assert ok, (fails, max_abs, worst)


def test_probe_linear_series_is_a_loop_of_linear_calls(gpu_ctx):
    """krm_probe_linear_series queues `count` plain linear_i4 launches over rotating weights:
    the output is that of the last launch's weights, bit for bit; it refuses to be recorded."""
    n, k, g = 256, 512, 128
    rng = np.random.default_rng(77)
    sets = [helpers.synthetic_int4(rng, n, k, g) for _ in range(3)]
    x = rng.normal(size=(1, k)).astype(np.float16)
    dx = gpu_ctx.upload(x)
    dws = [gpu_ctx.upload(p) for p, _q, _s in sets]
    dss = [gpu_ctx.upload(s) for _p, _q, s in sets]
    out, ref = gpu_ctx.alloc(n * 2), gpu_ctx.alloc(n * 2)
    gpu_ctx.probe_linear_series(dx, dws, dss, out, 5, 1, n, k, g, ka.F16, ka.F16)
    last = (5 - 1) % 3
    gpu_ctx.linear_i4(dx, dws[last], dss[last], None, ref, 1, n, k, g, ka.F16, ka.F16)
    assert out.download(np.uint16, (n,)).tobytes() == ref.download(np.uint16, (n,)).tobytes()
    with gpu_ctx.record() as rec:
        with pytest.raises(ka.GpuValidationError):
            gpu_ctx.probe_linear_series(dx, dws, dss, out, 2, 1, n, k, g, ka.F16, ka.F16)
        gpu_ctx.linear_i4(dx, dws[0], dss[0], None, ref, 1, n, k, g, ka.F16, ka.F16)
    rec.graph.destroy()
    for b in [dx, out, ref] + dws + dss:
        b.free()


def test_probe_exchange_is_bounded_and_clean(gpu_ctx):
    """The in-kernel hand-over probe: every wait in it is bounded, so the launch ends whatever
    the spin limit is and the fault word is 0 (every poll succeeded) or 1 (some poll gave up).
    A generous limit gives 0 only while all 256 workgroups are resident together, which the
    probe cannot guarantee on a GPU it shares with another process: the value is reported, the
    assertion is on termination and on the word being one of the two."""
    entries = 2048
    work = gpu_ctx.alloc(2 * entries * 4 + 1040)
    fault_at = 2 * entries * 4 + 1024
    for phases, limit in ((200, None), (200, 1), (50, None)):  # clean again after a faulted run
        if limit is None:
            gpu_ctx.probe_exchange(work, entries, phases)
        else:
            gpu_ctx.probe_exchange(work, entries, phases, spin_limit=limit)
        gpu_ctx.sync()
        fault = int(work.download(np.uint32, (1,), byte_offset=fault_at)[0])
        print(f"[probe exchange] phases {phases}, spin limit {limit}: fault word {fault}")
        assert fault in (0, 1)
    with pytest.raises(ka.GpuValidationError):
        gpu_ctx.probe_exchange(work, 1000, 10)
    work.free()
