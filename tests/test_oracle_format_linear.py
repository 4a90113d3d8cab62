"""Pins the CPU oracle's int4 / f16 decoding and `linear` against vectors the reference's own
tests hold and against checks the mathematics fixes.  CPU only."""
import numpy as np
import pytest
from safetensors.numpy import load_file

import helpers
from helpers import oracle


# ---- packages/runtime/tests/format_i4_test.ts -------------------------------------------------

def test_pack_order_low_nibble_first():
    # format_i4_test.ts:10-15 / tools/exporter/tests/test_emit.py:588-593: q=[1,2] -> 0xA9
    assert oracle.decode_i4(bytes([0xA9]), [1, 2], [1.0], [1, 1], 2).tolist() == [[1.0, 2.0]]
    assert oracle.pack_i4([1, 2]).tolist() == [0xA9]
    # test_emit.py:595-600: [-7, 7, 0, -7] -> [0xF1, 0x18]
    assert oracle.pack_i4([-7, 7, 0, -7]).tolist() == [0xF1, 0x18]


def test_asymmetric_pattern_positions():
    # format_i4_test.ts:17-28
    q = [((i % 7) + 1) * (1 if i % 2 == 0 else -1) for i in range(16)]
    raw = bytearray(8)
    for i, value in enumerate(q):
        u = value + 8
        raw[i >> 1] |= (u << 4) if i & 1 else u
    out = oracle.decode_i4(bytes(raw), [1, 16], [0.5], [1, 1], 16)
    assert out.reshape(-1).tolist() == [v * 0.5 for v in q]
    assert bytes(oracle.pack_i4(q)) == bytes(raw)


def test_scale_is_indexed_row_then_group():
    # format_i4_test.ts:30-37
    out = oracle.decode_i4(bytes([0x99] * 8), [2, 8], [1, 2, 4, 8], [2, 2], 4)
    assert out.reshape(-1).tolist() == [1] * 4 + [2] * 4 + [4] * 4 + [8] * 4


def test_vocab_table_group32_and_rank3():
    # format_i4_test.ts:39-67
    vocab, hidden, g = 3, 64, 32
    q = [((i // hidden + i) % 15) - 7 for i in range(vocab * hidden)]
    scale = np.array([0.5, 0.25, 1, 2, 4, 8], dtype=np.float32)
    out = oracle.decode_i4(oracle.pack_i4(q), [vocab, hidden], scale, [vocab, 2], g).reshape(-1)
    want = [np.float32(v * float(scale[(i // hidden) * 2 + (i % hidden) // g]))
            for i, v in enumerate(q)]
    assert out.tolist() == want
    # format_i4_test.ts:69-96: rank 3 [2,4,4], g8 -> scale [2,2]; the old same-rank shape is rejected
    q3 = [(i % 15) - 7 for i in range(32)]
    s3 = np.array([0.5, 0.25, 1, 2], dtype=np.float32)
    out3 = oracle.decode_i4(oracle.pack_i4(q3), [2, 4, 4], s3, [2, 2], 8).reshape(-1)
    want3 = [np.float32(v * float(s3[(i // 16) * 2 + (i % 16) // 8])) for i, v in enumerate(q3)]
    assert out3.tolist() == want3
    with pytest.raises(oracle.OracleError):
        oracle.decode_i4(oracle.pack_i4(q3), [2, 4, 4], [1.0] * 8, [2, 4, 1], 4)


def test_single_rounding():
    # format_i4_test.ts:98-106: scale 0.1 (not exact in f32), q = +-7 -> 0x1F
    s = np.float32(0.1)
    out = oracle.decode_i4(bytes([0x1F]), [1, 2], [s], [1, 1], 2).reshape(-1)
    assert out[0] == np.float32(7 * float(s))
    assert out[1] == np.float32(-7 * float(s))


def test_decode_rejections():
    # format_i4_test.ts:108-141
    raw = bytes(8)
    with pytest.raises(oracle.OracleError):
        oracle.decode_i4(bytes(7), [2, 8], [1, 1], [2, 1], 8)
    with pytest.raises(oracle.OracleError):
        oracle.decode_i4(raw, [2, 8], [1, 1], [2, 1], 4)
    with pytest.raises(oracle.OracleError):
        oracle.decode_i4(raw, [2, 8], [1, 1], [2, 1], 3)
    with pytest.raises(oracle.OracleError):
        oracle.decode_i4(raw, [2, 8], [1], [2, 2], 4)
    with pytest.raises(oracle.OracleError):
        oracle.decode_i4(b"", [], [], [], 16)


def test_decode_total_over_all_sixteen_codes():
    """The decode formula is total over u in [0, 15] (u = 0 -> q = -8): brute force in
    float64 with one rounding, every code at every in-word position."""
    q = np.array([(r + c) % 16 - 8 for r in range(16) for c in range(32)], dtype=np.int8)
    scale = np.array([[0.1 + 0.017 * r + 0.31 * g for g in range(2)] for r in range(16)],
                     dtype=np.float32)
    out = oracle.decode_i4(oracle.pack_i4(q), [16, 32], scale, [16, 2], 16)
    want = (q.reshape(16, 2, 16).astype(np.float64) * scale.astype(np.float64)[:, :, None]
            ).astype(np.float32).reshape(16, 32)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    for pos in range(8):
        assert len({int(v) for v in q.reshape(-1)[pos::8]}) == 16


def test_nibble_coverage_table_of_the_reference():
    # gpu_i4_weights_test.ts:404-427: q(row,col) = ((row+col) % 15) - 7 with row x group
    # amplitudes; the test-side quantiser must recover those codes and every code must appear
    # at each of the 8 in-word positions.
    vocab, hidden, g = 16, 32, 16
    w = np.array([(((i // hidden + i % hidden) % 15) - 7) *
                  (0.1 + (i // hidden) * 0.017 + ((i % hidden) // g) * 0.31)
                  for i in range(vocab * hidden)], dtype=np.float32)
    packed, q, scale = helpers.quantize_i4(w, (vocab, hidden), g)
    for pos in range(8):
        seen = set()
        for i in range(pos, vocab * hidden, 8):
            byte = int(packed[i >> 1])
            seen.add(byte >> 4 if i & 1 else byte & 0x0F)
        assert len(seen) == 15
    dec = oracle.decode_i4(packed, [vocab, hidden], scale, [vocab, hidden // g], g).reshape(-1)
    assert np.allclose(dec, w, rtol=1e-6, atol=1e-6)


# ---- f16 -----------------------------------------------------------------------------------

def test_f16_bits_to_f32_all_patterns_match_ieee():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_bits_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_rounding_matches_ieee():
    rng = np.random.default_rng(3)
    values = np.concatenate([
        rng.normal(0, 1, 4000), rng.normal(0, 1e-5, 2000), rng.normal(0, 3e4, 2000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 2 ** -24, 2 ** -25, 1.5 * 2 ** -24,
                  2.5 * 2 ** -24, 2 ** -14, 1.00048828125, 1.0009765625 + 2 ** -12]),
    ]).astype(np.float32)
    want = values.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16_bits(float(v)) for v in values], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---- linear --------------------------------------------------------------------------------

def test_linear_known_answer():
    # packages/runtime/tests/reference_ops_test.ts:585-596
    out = oracle.linear(np.array([[1, 2, 3], [4, 5, 6]]), np.array([[1, 0, -1], [2, 2, 2]]),
                        np.array([10, -1]))
    assert out.tolist() == [[8, 11], [8, 29]]
    out3 = oracle.linear(np.array([[[1, 2, 3]], [[4, 5, 6]]]), np.array([[1, 0, -1], [2, 2, 2]]),
                         np.array([10, -1]))
    assert out3.shape == (2, 1, 2) and out3.reshape(-1).tolist() == [8, 11, 8, 29]


def test_linear_golden_argmax_pick():
    """Torch-CPU golden: linear -> argmax, plus argmax over a tensor with ties
    (packages/runtime/tests/fixtures/golden/argmax_pick)."""
    model = load_file(f"{helpers.GOLDEN}/argmax_pick/model.safetensors")
    io = load_file(f"{helpers.GOLDEN}/argmax_pick/io.safetensors")
    logits = oracle.linear(io["input.x"], model["head.weight"], model["head.bias"])
    assert np.array_equal(oracle.argmax(logits), io["output.0"])
    tied = io["input.tied"]
    assert np.array_equal(oracle.argmax(np.concatenate([tied, tied], axis=1)), io["output.1"])


def test_linear_golden_rms_norm_block():
    """Torch-CPU golden: rms_norm(eps 1e-6) -> linear -> rms_norm(eps 1e-5) twice
    (packages/runtime/tests/fixtures/golden/rms_norm_block), atol 1e-6 rtol 1e-5."""
    model = load_file(f"{helpers.GOLDEN}/rms_norm_block/model.safetensors")
    io = load_file(f"{helpers.GOLDEN}/rms_norm_block/io.safetensors")
    h = oracle.rms_norm(io["input.x"], model["weight"], 1e-6)
    lin = oracle.linear(h, model["dense.weight"], model["const.316c8c74afaf9d19"])
    out0 = oracle.rms_norm(lin, model["affine.weight"], 1e-5)
    out1 = oracle.rms_norm(lin, model["const.bfd1c1e2f6cab2be"], 1e-5)
    for got, want in ((out0, io["output.0"]), (out1, io["output.1"])):
        ok, fails, max_abs, _ = oracle.allclose(got, want, atol=1e-6, rtol=1e-5)
        assert ok, (fails, max_abs)


def test_linear_matches_float64_matmul_and_threads_agree():
    rng = np.random.default_rng(11)
    x = rng.normal(size=(5, 96)).astype(np.float32)
    w = rng.normal(size=(20, 96)).astype(np.float32)
    b = rng.normal(size=20).astype(np.float32)
    want = (x.astype(np.float64) @ w.astype(np.float64).T + b.astype(np.float64))
    got = oracle.linear(x, w, b)
    assert np.max(np.abs(got - want)) <= 2e-6
    assert np.array_equal(oracle.linear(x, w, b, threads=True), got)


def test_linear_i4_row_streaming_equals_decode_then_linear():
    for case in helpers.I4_LINEAR_CASES:
        x, packed, _q, scale, bias = helpers.make_i4_linear(case)
        w = oracle.decode_i4(packed, [case.n, case.k], scale, [case.n, case.k // case.group],
                             case.group)
        want = oracle.linear(x, w, bias)
        got = oracle.linear_i4(x, packed, scale, bias, case.n, case.k, case.group)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), case.name


def test_linear_i4_sensitive_to_nibble_and_group_mistakes():
    """A swapped nibble order or a wrong scale index must move the result far beyond the
    tolerance used on the GPU side — otherwise a green parity run proves nothing."""
    case = helpers.I4_LINEAR_CASES[0]
    x, packed, q, scale, bias = helpers.make_i4_linear(case)
    good = oracle.linear_i4(x, packed, scale, bias, case.n, case.k, case.group)
    swapped = ((packed >> 4) | (packed << 4)).astype(np.uint8)
    bad_nibbles = oracle.linear_i4(x, swapped, scale, bias, case.n, case.k, case.group)
    bad_scale = oracle.linear_i4(x, packed, np.roll(scale, 1, axis=1), bias, case.n, case.k,
                                 case.group)
    assert np.max(np.abs(bad_nibbles - good)) > 1.0
    assert np.max(np.abs(bad_scale - good)) > 1.0


def test_allclose_rule():
    # packages/runtime/src/reference/allclose.ts:47-82
    ok, fails, max_abs, worst = oracle.allclose([1.0, 2.0], [1.0, 2.002], atol=1e-5, rtol=1e-3)
    assert ok and fails == 0 and abs(max_abs - 0.002) < 1e-6 and worst == 1
    assert not oracle.allclose([1.0], [1.1])[0]
    ok, fails, max_abs, _ = oracle.allclose([np.nan, 1.0], [np.nan, 1.0])
    assert not ok and fails == 1 and np.isinf(max_abs)
    assert not oracle.allclose([np.inf], [np.inf])[0]
    with pytest.raises(oracle.OracleError):
        oracle.allclose([1.0], [1.0, 2.0])


def test_glue_ops_known_answers():
    # argmax fixed behaviour (packages/runtime/src/reference/ops.ts:520-560)
    assert oracle.argmax(np.array([[1, 3, 3, 2]], dtype=np.float32)).tolist() == [[1]]
    assert oracle.argmax(np.array([[1, np.nan, 3, np.nan]], dtype=np.float32)).tolist() == [[1]]
    assert oracle.argmax(np.full((1, 4), -np.inf, dtype=np.float32)).tolist() == [[0]]
    # rope half split: rotate_half(x) = cat(-x[D/2:], x[:D/2])
    x = np.arange(8, dtype=np.float32).reshape(1, 1, 2, 4) + 1
    cos = np.full((2, 4), 0.5, dtype=np.float32)
    sin = np.full((2, 4), 2.0, dtype=np.float32)
    got = oracle.rope_half(x, cos, sin).reshape(2, 4)
    want = np.array([[1 * .5 - 3 * 2, 2 * .5 - 4 * 2, 3 * .5 + 1 * 2, 4 * .5 + 2 * 2],
                     [5 * .5 - 7 * 2, 6 * .5 - 8 * 2, 7 * .5 + 5 * 2, 8 * .5 + 6 * 2]])
    assert np.array_equal(got, want.astype(np.float32))
    # silu(g) * u against float64
    g = np.linspace(-6, 6, 25).astype(np.float32)
    u = np.linspace(2, -2, 25).astype(np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.max(np.abs(oracle.silu_mul(g, u) - want)) < 1e-6
    # embedding gathers rows and rejects an out-of-range index
    table = np.arange(12, dtype=np.float32).reshape(4, 3)
    assert oracle.embedding(table, [[2, 0]]).tolist() == [[[6, 7, 8], [0, 1, 2]]]
    with pytest.raises(oracle.OracleError):
        oracle.embedding(table, [4])
