"""Pins the CPU oracle's states-form attention and state_append.  CPU only.

Sources of truth, none of which share code with the oracle's loops:
  * hand-computed probes of the reference's own unit tests
    (packages/runtime/tests/kernel_state_attention_test.ts:341-503);
  * the torch-CPU golden fixture `fused_attention`;
  * a float64 NumPy einsum restatement with an explicit mask (textbook attention);
  * the cross-oracle of packages/runtime/tests/gpu_state_acceptance_test.ts:371-585: a
    prefill -> decode chain through attention + append equals ONE full-history masked
    attention, and widening the window by one breaks it;
  * the reference's mutation checklist
    (packages/runtime/tests/gpu_state_attention_test.ts:714-765,793-815): the parity
    fixtures must move when the oracle is run with each fault.
"""
import numpy as np
import pytest
from safetensors.numpy import load_file

import helpers
from helpers import PARITY_CASES, StateCase, make_state_inputs, oracle, oracle_state_attention


def test_live_range_closed_forms():
    # kernel_state_attention_test.ts:341-354
    assert oracle.state_column_base(0, 100) == 0
    assert oracle.state_live_columns(0, 100, 8) == 108
    assert oracle.state_column_base(4, 2) == 0
    assert oracle.state_live_columns(4, 2, 1) == 3
    assert oracle.state_column_base(4, 9) == 6
    assert oracle.state_live_columns(4, 9, 1) == 4
    assert oracle.state_live_columns(4, 1000, 1) == 4
    assert oracle.state_effective_rows(4, 8, 9) == 1
    assert oracle.state_effective_rows(4, 8, 8) == 0
    assert oracle.state_effective_rows(4, 0, 9) == 4


def window_probe(window, past, query, chunk_rows, capacity, poison):
    """D = 1, all keys 1 (uniform weights), V(col) = col at its physical row
    (kernel_state_attention_test.ts:356-400)."""
    slot_k = np.ones(capacity, dtype=np.float32)
    slot_v = np.full(capacity, poison, dtype=np.float32)
    ins_k = np.ones(chunk_rows, dtype=np.float32)
    ins_v = np.full(chunk_rows, poison, dtype=np.float32)
    for col in range(oracle.state_column_base(window, past), past):
        slot_v[col % window if window else col] = col
    for row in range(query):
        ins_v[row] = past + row
    return oracle.state_attention(
        np.ones(chunk_rows, dtype=np.float32), ins_k, ins_v, slot_k, slot_v, batch=1, heads=1,
        kv_heads=1, chunk_rows=chunk_rows, depth=1, capacity=capacity, window=window, past=past,
        query=query, scale=1.0).reshape(-1)


def test_probe_sliding_window_is_two_sided():
    # kernel_state_attention_test.ts:402-417: W=4, P=5, Q=1 -> mean of {2,3,4,5} = 3.5
    assert abs(window_probe(4, 5, 1, 1, 4, 1e6)[0] - 3.5) < 1e-6


def test_probe_full_causal_and_pad_row_zero():
    # kernel_state_attention_test.ts:419-438: P=3,Q=2,M=3 -> 1.5, 2, exact +0
    out = window_probe(0, 3, 2, 3, 8, 0)
    assert abs(out[0] - 1.5) < 1e-6 and abs(out[1] - 2.0) < 1e-6
    assert out[2] == 0.0 and not np.signbit(out[2])


def test_probe_empty_row_is_exact_zero():
    # kernel_state_attention_test.ts:440-456: W=2,P=0,Q=1,M=3
    out = window_probe(2, 0, 1, 3, 2, 1e6)
    assert out[2] == 0.0 and not np.signbit(out[2])
    assert abs(out[0]) < 1e-6


def test_probe_gqa_plane_is_floor_division():
    # kernel_state_attention_test.ts:458-479
    batch, heads, kv_heads = 2, 4, 2
    ins_v = np.array([10, 20, 30, 40], dtype=np.float32)
    out = oracle.state_attention(
        np.ones(batch * heads, dtype=np.float32), np.ones(batch * kv_heads, dtype=np.float32),
        ins_v, np.zeros(batch * kv_heads, dtype=np.float32),
        np.zeros(batch * kv_heads, dtype=np.float32), batch=batch, heads=heads,
        kv_heads=kv_heads, chunk_rows=1, depth=1, capacity=1, window=0, past=0, query=1,
        scale=1.0).reshape(-1)
    for z in range(batch * heads):
        assert abs(out[z] - ins_v[z // (heads // kv_heads)]) < 1e-6


def test_append_vectors():
    # kernel_state_attention_test.ts:481-503
    spec = dict(kv_planes=1, chunk_rows=4, depth=1, capacity=4, window=4)
    slot = np.array([-1, -2, -3, -4], dtype=np.float32)
    x = np.array([100, 200, 300, 400], dtype=np.float32)
    after = oracle.state_append(x, slot, past=2, query=2, **spec)
    assert after.reshape(-1).tolist() == [-1, -2, 100, 200]
    assert slot.tolist() == [-1, -2, -3, -4]
    wrapped = oracle.state_append(x, slot, past=3, query=3, **spec)
    assert wrapped.reshape(-1).tolist() == [200, 300, -3, 100]
    collide = oracle.state_append(x, np.array([-1, -2], dtype=np.float32), kv_planes=1,
                                  chunk_rows=4, depth=1, capacity=2, window=2, past=0, query=4)
    assert collide.reshape(-1).tolist() == [300, 400]


def test_shape_rejections():
    # packages/runtime/src/reference/state-attention.ts:63-86
    case = StateCase("bad", 1, 3, 2, 1, 4, 4, 0, 0, 1)
    with pytest.raises(oracle.OracleError):  # H % Hkv
        oracle_state_attention(case, {k: np.zeros(64, dtype=np.float32) for k in
                                      ("q", "ins_k", "ins_v", "slot_k", "slot_v")})
    ok = StateCase("ok", 1, 2, 2, 2, 4, 4, 0, 3, 2)  # P + Q > C on a full slot
    with pytest.raises(oracle.OracleError):
        oracle_state_attention(ok, make_state_inputs(StateCase("ok", 1, 2, 2, 2, 4, 4, 0, 1, 2)))
    with pytest.raises(oracle.OracleError):  # window > capacity
        oracle.state_append(np.zeros(4, dtype=np.float32), np.zeros(4, dtype=np.float32),
                            kv_planes=1, chunk_rows=1, depth=4, capacity=1, window=2, past=0,
                            query=1)
    with pytest.raises(oracle.OracleError):  # query outside 1..M
        oracle.state_append(np.zeros(4, dtype=np.float32), np.zeros(4, dtype=np.float32),
                            kv_planes=1, chunk_rows=1, depth=4, capacity=1, window=0, past=0,
                            query=2)


def test_golden_fused_attention_row_by_row():
    """Torch-CPU golden (packages/runtime/tests/fixtures/golden/fused_attention): q [2,3,5,4],
    k/v [2,3,7,4], scale attr 0.70710677 = the half-scale of D = 4.  With window = 0, Q = 1,
    P = 6 one states-form row is ordinary attention over the 7 keys (6 in the slot, 1 in ins)."""
    io = load_file(f"{helpers.GOLDEN}/fused_attention/io.safetensors")
    q, k, v, want = io["input.query"], io["input.key"], io["input.value"], io["output.0"]
    half = np.float32(0.7071067690849304)
    slot_k, slot_v = k.copy(), v.copy()
    slot_k[:, :, 6] = 9.0    # the 7th key comes from ins; its slot row must not be read
    slot_v[:, :, 6] = 400.0
    for row in range(q.shape[2]):
        got = oracle.state_attention(
            q[:, :, row:row + 1, :], k[:, :, 6:7, :], v[:, :, 6:7, :], slot_k, slot_v,
            batch=2, heads=3, kv_heads=3, chunk_rows=1, depth=4, capacity=7,
            window=0, past=6, query=1, scale=half)
        ok, fails, max_abs, _ = oracle.allclose(got, want[:, :, row:row + 1, :], atol=1e-6,
                                                rtol=1e-5)
        assert ok, (row, fails, max_abs)


def dense_reference(case: StateCase, x: dict) -> np.ndarray:
    """Independent float64 restatement: gather the live columns into a dense K/V, build the
    boolean mask from the contract's predicate, run textbook attention."""
    b, h, hkv, m, d = case.batch, case.heads, case.kv_heads, case.chunk_rows, case.depth
    r = h // hkv
    base = oracle.state_column_base(case.window, case.past)
    cols = list(range(base, case.past + case.query))
    kd = np.zeros((b, hkv, len(cols), d))
    vd = np.zeros((b, hkv, len(cols), d))
    for j, col in enumerate(cols):
        if col < case.past:
            prow = col % case.window if case.window else col
            kd[:, :, j] = x["slot_k"][:, :, prow]
            vd[:, :, j] = x["slot_v"][:, :, prow]
        else:
            kd[:, :, j] = x["ins_k"][:, :, col - case.past]
            vd[:, :, j] = x["ins_v"][:, :, col - case.past]
    mask = np.zeros((case.query, len(cols)), dtype=bool)
    for row in range(case.query):
        for j, col in enumerate(cols):
            limit = case.past + row
            mask[row, j] = col <= limit and (case.window == 0 or limit - col < case.window)
    kd = np.repeat(kd, r, axis=1)
    vd = np.repeat(vd, r, axis=1)
    s = float(oracle.half_scale(d))
    out = np.zeros((b, h, m, d))
    out[:, :, :case.query] = helpers.dense_attention_f64(
        x["q"][:, :, :case.query].astype(np.float64), kd, vd, mask, s * s)
    return out


@pytest.mark.parametrize("case", PARITY_CASES, ids=lambda c: c.name)
def test_parity_grid_against_dense_float64(case):
    """The reference's 17-case grid: the oracle equals the dense float64 restatement, pad rows
    are exact +0, and no poison value leaks into the result."""
    x = make_state_inputs(case)
    got = oracle_state_attention(case, x)
    want = dense_reference(case, x)
    assert np.max(np.abs(got - want)) < 2e-6
    pad = got[:, :, case.query:, :]
    assert np.all(pad == 0.0) and not np.any(np.signbit(pad))
    assert np.max(np.abs(got)) < 50  # V poison is 400


MUTATION_WITNESS = {
    oracle.MUT_DROP_LOWER_BOUND: "sliding W4 P10 wrap",
    oracle.MUT_RING_MOD_CAPACITY: "sliding W4 C8 wrap",
    oracle.MUT_PAD_ROWS_COMPUTED: "full r2 pad B2 D6",
    oracle.MUT_IGNORE_KV_REPEAT: "full r2 pad B2 D6",
    oracle.MUT_SCALE_ONE_SIDE: "full r1 prefill B2",
    oracle.MUT_OVERFLOW_FORM: "sliding W2 P near u32 max",
}


@pytest.mark.parametrize("mutation,name", MUTATION_WITNESS.items())
def test_fixtures_are_sensitive_to_each_fault(mutation, name):
    """Every fault of the reference's checklist moves at least its witness case by far more
    than the GPU tolerance (5e-6); faults must not be invisible to the fixtures."""
    case = next(c for c in PARITY_CASES if c.name == name)
    x = make_state_inputs(case)
    good = oracle_state_attention(case, x)
    bad = oracle_state_attention(case, x, mutation=mutation)
    assert np.max(np.abs(bad - good)) > 1e-3


def test_append_ring_mutation_is_visible():
    slot = np.arange(8 * 2, dtype=np.float32).reshape(1, 8, 2)
    x = np.full((1, 2, 2), 77, dtype=np.float32)
    spec = dict(kv_planes=1, chunk_rows=2, depth=2, capacity=8, window=4, past=5, query=2)
    good = oracle.state_append(x, slot, **spec)
    bad = oracle.state_append(x, slot, mutation=oracle.MUT_APPEND_NO_RING, **spec)
    assert not np.array_equal(good, bad)
    assert good[0, 1].tolist() == [77, 77] and good[0, 2].tolist() == [77, 77]


def run_chain(window: int, capacity: int, steps, heads=4, kv_heads=2, depth=8, widen=0,
              with_slots=False):
    """Prefill -> decode chain carried on the host: each step reads the slots, then appends
    (packages/runtime/tests/gpu_state_execution_test.ts:152-212).  Returns the outputs of the
    valid rows of every step and the full K/V history that was fed in (and the final slots
    with `with_slots`).  Only the valid rows are drawn from the generator, so two chains whose
    steps differ in pad rows alone see the same values."""
    rng = np.random.default_rng(5)
    r = heads // kv_heads
    slot_k = np.zeros((1, kv_heads, capacity, depth), dtype=np.float32)
    slot_v = np.zeros_like(slot_k)
    past = 0
    outs, qs, ks, vs = [], [], [], []
    for chunk_rows, query in steps:
        q = np.full((1, heads, chunk_rows, depth), 0.5, dtype=np.float32)
        k = np.full((1, kv_heads, chunk_rows, depth), 9.0, dtype=np.float32)    # pad rows carry
        v = np.full((1, kv_heads, chunk_rows, depth), 400.0, dtype=np.float32)  # poison
        q[:, :, :query] = rng.normal(size=(1, heads, query, depth))
        k[:, :, :query] = rng.normal(size=(1, kv_heads, query, depth))
        v[:, :, :query] = rng.normal(size=(1, kv_heads, query, depth))
        out = oracle.state_attention(q, k, v, slot_k, slot_v, batch=1, heads=heads,
                                     kv_heads=kv_heads, chunk_rows=chunk_rows, depth=depth,
                                     capacity=capacity, window=window + widen if window else 0,
                                     past=past, query=query, scale=oracle.half_scale(depth))
        spec = dict(kv_planes=kv_heads, chunk_rows=chunk_rows, depth=depth, capacity=capacity,
                    window=window, past=past, query=query)
        slot_k = oracle.state_append(k, slot_k, **spec).reshape(1, kv_heads, capacity, depth)
        slot_v = oracle.state_append(v, slot_v, **spec).reshape(1, kv_heads, capacity, depth)
        outs.append(out[:, :, :query])
        qs.append(q[:, :, :query])
        ks.append(k[:, :, :query])
        vs.append(v[:, :, :query])
        past += query
    cat = lambda parts: np.concatenate(parts, axis=2)  # noqa: E731
    result = (cat(outs), cat(qs), np.repeat(cat(ks), r, axis=1), np.repeat(cat(vs), r, axis=1))
    return result + (slot_k, slot_v) if with_slots else result


@pytest.mark.parametrize("window,capacity", [(0, 32), (5, 5), (5, 8)])
def test_cross_oracle_chain_equals_full_history_attention(window, capacity):
    steps = [(6, 6), (6, 3), (1, 1), (1, 1), (4, 2), (1, 1)]
    out, q, k, v = run_chain(window, capacity, steps)
    total = q.shape[2]
    i = np.arange(total)
    mask = i[None, :] <= i[:, None]
    if window:
        mask &= (i[:, None] - i[None, :]) < window
    s = float(oracle.half_scale(8))
    want = helpers.dense_attention_f64(q, k, v, mask, s * s)
    assert np.max(np.abs(out - want)) < 2e-6
    if window:  # a window one wider is a different function (fault injection of the reference)
        wide, *_ = run_chain(window, capacity + 1, steps, widen=1)
        assert np.max(np.abs(wide - want)) > 1e-3


def test_capacity_and_pad_rows_do_not_change_results():
    """Outputs are bit-identical for C = 8 and C = 4096, and with or without pad rows
    (packages/runtime/tests/gpu_state_acceptance_test.ts:586-708,780-833)."""
    steps_pad = [(8, 5), (1, 1), (1, 1)]
    steps_tight = [(5, 5), (1, 1), (1, 1)]
    small, *_, small_k, small_v = run_chain(0, 8, steps_pad, with_slots=True)
    large, *_ = run_chain(0, 4096, steps_pad)
    tight, *_, tight_k, tight_v = run_chain(0, 8, steps_tight, with_slots=True)
    assert np.array_equal(small.view(np.uint32), large.view(np.uint32))
    # pad rows change neither the valid rows' outputs nor a byte of the KV slots
    assert small.shape == tight.shape == (1, 4, 7, 8)
    assert np.array_equal(small.view(np.uint32), tight.view(np.uint32))
    assert np.array_equal(small_k.view(np.uint32), tight_k.view(np.uint32))
    assert np.array_equal(small_v.view(np.uint32), tight_v.view(np.uint32))
    assert not np.any(small_k == 9.0) and not np.any(small_v == 400.0)
