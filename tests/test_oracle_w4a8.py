"""Pins the CPU oracle's activation quantiser and w4a8 `linear` against the known answers the
reference's own tests hold (packages/runtime/tests/i8a8_reference_test.ts) and against an
independent integer restatement.  CPU only."""
import numpy as np
import pytest

import helpers
from helpers import oracle

F32_TINY = 1.1754943508222875e-38


# ---- quantizeRowsReference: i8a8_reference_test.ts:42-96 --------------------------------------

def test_all_zero_row_gets_the_tiny_scale():
    q, scale = oracle.quantize_rows([0, 0, 0, 0], 4)
    assert float(scale[0]) == F32_TINY
    assert q.tolist() == [[0, 0, 0, 0]]


def test_non_finite_values_reach_the_row_scale_only():
    x = [1, np.nan, -3, 2, np.inf, 1, 2, -np.inf, 1, 1, 2, 3]
    q, scale = oracle.quantize_rows(x, 3)
    assert np.isnan(scale[0])
    assert scale[1] == np.inf and scale[2] == np.inf
    assert float(scale[3]) == 0.023622047156095505
    assert q[3].tolist() == [42, 85, 127]


def test_largest_magnitude_lands_on_127_exactly():
    q, scale = oracle.quantize_rows([127, -127, 3, 0], 4)
    assert float(scale[0]) == 1.0
    assert q.tolist() == [[127, -127, 3, 0]]
    # i8a8_reference_test.ts:98-104: x = [8, 3] -> s = f32(8/127), q = [127, 48]
    q, scale = oracle.quantize_rows([8, 3], 2)
    assert float(scale[0]) == 0.06299212574958801 and q.tolist() == [[127, 48]]


def test_ties_round_to_even():
    # gpu_i8a8_test.ts:216-238: amax = 127 makes s exactly 1, so the ties are the inputs
    values = [127, 0.5, 1.5, -0.5, -1.5, 2.5, 3.5, -3.5]
    q, scale = oracle.quantize_rows(values, len(values))
    assert float(scale[0]) == 1.0
    assert q.tolist() == [[127, 0, 2, 0, -2, 2, 4, -4]]


def test_tie_margin_of_the_reference_generators():
    # gpu_i8a8_test.ts:244-259: the 7 x 20 block, every row scaled differently, row 3 zero
    rows, dim = 7, 20
    x = np.array([[0 if r == 3 else helpers.SIGNED_A8(r * dim + i) * (1 + r * 3)
                   for i in range(dim)] for r in range(rows)], dtype=np.float32)
    assert oracle.quantize_rows_tie_margin(x, dim) > helpers.TIE_MARGIN
    q, scale = oracle.quantize_rows(x, dim)
    assert len(set(scale.tolist())) >= rows - 1
    assert float(scale[3]) == F32_TINY and not q[3].any()
    for r in range(rows):
        if r != 3:
            assert np.abs(q[r][np.abs(x[r]) == np.abs(x[r]).max()]).tolist() == [127] * int(
                (np.abs(x[r]) == np.abs(x[r]).max()).sum())


# ---- referenceLinearW4a8: i8a8_reference_test.ts:141-189 --------------------------------------

@pytest.mark.parametrize("fused", [True, False])
def test_w4a8_known_answer(fused):
    # group 2, power-of-two scales: every step up to the last product is exact in f32
    out = oracle.linear_w4a8([8, 3, -2, 5], oracle.pack_i4([1, 2, -3, 4, 7, -7, 5, -6]),
                             [0.5, 0.25, 0.125, 2], [1, -1], 2, 4, 2, fused=fused)
    assert [float(v) for v in out] == [14.511811256408691, -76.51968383789062]


@pytest.mark.parametrize("fused", [True, False])
def test_w4a8_flushes_every_group_on_its_own(fused):
    # s = 1 and q = x: only the order of the roundings is left in the output
    scale = 0.017009999603033066
    out = oracle.linear_w4a8([127, 37, 121, 20], oracle.pack_i4([-7, -3, -7, -6]),
                             [scale, scale], [0], 1, 4, 2, fused=fused)
    assert float(out[0]) == -33.45867156982422
    assert float(out[0]) != -33.45866775512695  # one integer sum over both groups


def independent_w4a8(x, q, scale, bias, group):
    """The formula again with numpy integers and an exact-rational fma (fractions), sharing
    no code with the C oracle."""
    from fractions import Fraction
    x = np.asarray(x, dtype=np.float32)
    m, k = x.shape
    n = q.shape[0]
    out = np.empty((m, n), dtype=np.float32)

    def fma(a, b, c):  # one rounding of the exact a * b + c
        exact = Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c))
        return np.float32(float(exact))

    for r in range(m):
        amax = np.float32(np.abs(x[r]).max())
        s = max(np.float32(amax * np.float32(1.0 / 127.0)), np.float32(F32_TINY))
        xq = np.clip(np.rint((x[r] / s).astype(np.float32)), -127, 127).astype(np.int64)
        for c in range(n):
            accf = np.float32(0)
            for g in range(k // group):
                acci = int((xq[g * group:(g + 1) * group] *
                            q[c, g * group:(g + 1) * group].astype(np.int64)).sum())
                accf = fma(np.float32(acci), scale[c, g], accf)
            out[r, c] = fma(accf, s, bias[c])
    return out


def test_w4a8_matches_an_independent_restatement():
    # float(Fraction) rounds to double first; the exact sums here fit a double (products of
    # 24-bit significands plus an addend of similar size), so the second rounding is the only one
    case = helpers.W4a8Case("small", 5, 6, 64, 16)
    x, packed, q, scale, bias = helpers.make_w4a8(case)
    want = independent_w4a8(x, q.reshape(case.n, case.k), scale, bias, case.group)
    for fused in (True, False):
        got = oracle.linear_w4a8(x, packed, scale, bias, case.n, case.k, case.group, fused=fused)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("case", helpers.W4A8_CASES, ids=lambda c: c.name)
def test_reference_cases_have_margin_and_alternating_signs(case):
    # the gates the reference puts in front of its atol = 0 claim (gpu_i8a8_test.ts:785-808)
    x, packed, q, scale, bias = helpers.make_w4a8(case)
    assert oracle.quantize_rows_tie_margin(x, case.k) > helpers.TIE_MARGIN
    alternating = int(((q[:-1] > 0) & (q[1:] < 0)).sum())
    assert alternating * 4 >= q.size
    fused = oracle.linear_w4a8(x, packed, scale, bias, case.n, case.k, case.group, fused=True)
    plain = oracle.linear_w4a8(x, packed, scale, bias, case.n, case.k, case.group, fused=False)
    assert np.array_equal(fused, plain)  # the double stand-in for fma agrees on this data
    assert len(set(fused.reshape(-1).tolist())) > 1
    # activations stay f32 on the default path: its values must differ (the quantiser acts)
    f32_path = oracle.linear_i4(x, packed, scale, bias, case.n, case.k, case.group)
    assert not np.array_equal(f32_path, fused)


def test_nan_row_spreads_over_its_outputs_only():
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
    out = oracle.linear_w4a8(x, packed, scale, bias, case.n, case.k, case.group)
    assert np.isnan(out[nan_row]).all() and np.isfinite(out[nan_row + 1]).all()
    assert np.array_equal(out[zero_row], bias)  # fma(0, tiny, bias)
