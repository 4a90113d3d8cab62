"""Host-side greedy loop and generation context against a fake session (no GPU).

The cases restate packages/models/tests/generation_greedy_test.ts:152-560: what the host puts
together for one step — fixed-length chunks, zero pad rows, absolute positions, the fed-back
token, the life of the context — seen through the calls a fake session receives.  The fake
returns next_token[0, row, 0] = call * 1000 + row, so one value tells which run and which row
was read.
"""
import numpy as np
import pytest

from karume_amd.generation import (GenerationContext, GenerationContextError, generate_greedy,
                                   plan_prefill_chunks)
from karume_amd.runtime import ExecutionError


class FakeContext:
    def __init__(self):
        self.disposals = 0

    def dispose(self):
        self.disposals += 1


class FakeSession:
    """Records every run; all-rows form ([1, M, 1]) unless `token_only`."""

    def __init__(self, outputs=None, fail_at=None, token_only=False):
        self.calls, self.specs = [], []
        self.context = FakeContext()
        self.outputs, self.fail_at, self.token_only = outputs, fail_at, token_only

    def create_generation_context(self, **spec):
        self.specs.append(spec)
        return self.context

    def run(self, input_ids, position_ids, last_row, *, context, query_length):
        for name, arr in (("input_ids", input_ids), ("position_ids", position_ids)):
            assert isinstance(arr, np.ndarray) and arr.dtype == np.int32, name
        call = len(self.calls)
        self.calls.append(dict(ids=input_ids[0].tolist(), ids_shape=list(input_ids.shape),
                               positions=position_ids[0].tolist(),
                               positions_shape=list(position_ids.shape), last_row=last_row,
                               query_length=query_length, same_context=context is self.context))
        if self.fail_at == call:
            raise RuntimeError("the run failed")
        rows = input_ids.shape[1]
        if self.outputs is not None:
            return self.outputs(call, rows)
        if self.token_only:
            return np.array([[[5000 + call]]], dtype=np.int32)
        return (call * 1000 + np.arange(rows, dtype=np.int32)).reshape(1, rows, 1)


def prompt_of(length, base=100):
    return [base + i for i in range(length)]


def greedy(fake, **kw):
    args = dict(prompt=[10, 11], max_new_tokens=2, chunk_length=4, max_position=512,
                last_row=False)
    args.update(kw)
    return generate_greedy(fake, **args)


# ---- plan_prefill_chunks (generation_greedy_test.ts:108-150) --------------------------------

def test_plan_prefill_chunks_splits_and_invariants():
    as_pairs = lambda chunks: [(c.position, c.query_length) for c in chunks]  # noqa: E731
    assert as_pairs(plan_prefill_chunks(87, 32)) == [(0, 32), (32, 32), (64, 23)]
    assert as_pairs(plan_prefill_chunks(32, 32)) == [(0, 32)]
    assert as_pairs(plan_prefill_chunks(64, 32)) == [(0, 32), (32, 32)]
    assert as_pairs(plan_prefill_chunks(1, 32)) == [(0, 1)]
    assert as_pairs(plan_prefill_chunks(31, 32)) == [(0, 31)]
    assert as_pairs(plan_prefill_chunks(10, 4)) == [(0, 4), (4, 4), (8, 2)]
    for length, chunk_length in [(87, 32), (1, 1), (5, 7), (64, 8), (9, 4)]:
        expected = 0
        for chunk in plan_prefill_chunks(length, chunk_length):
            assert chunk.position == expected
            assert 1 <= chunk.query_length <= chunk_length
            expected += chunk.query_length
        assert expected == length


@pytest.mark.parametrize("length,chunk", [(0, 32), (-1, 32), (1.5, 32), (8, 0), (8, 2.5)])
def test_plan_prefill_chunks_rejects_non_positive_integers(length, chunk):
    with pytest.raises(ValueError):
        plan_prefill_chunks(length, chunk)


# ---- generate_greedy, all-rows exit (generation_greedy_test.ts:152-330) -----------------------

def test_prefill_runs_fixed_length_chunks_with_zero_pad_rows_and_absolute_positions():
    fake, prompt = FakeSession(), prompt_of(87)
    generated = greedy(fake, prompt=prompt, max_new_tokens=1, chunk_length=32)
    assert len(fake.calls) == 3
    assert [c["query_length"] for c in fake.calls] == [32, 32, 23]
    assert [c["ids_shape"] for c in fake.calls] == [[1, 32]] * 3
    assert [c["positions_shape"] for c in fake.calls] == [[1, 32]] * 3
    assert fake.calls[0]["ids"] == prompt[:32]
    assert fake.calls[1]["ids"] == prompt[32:64]
    assert fake.calls[2]["ids"] == prompt[64:87] + [0] * 9
    assert fake.calls[0]["positions"] == list(range(32))
    assert fake.calls[1]["positions"] == list(range(32, 64))
    assert fake.calls[2]["positions"] == list(range(64, 87)) + [0] * 9
    # the first generated token is read from the last valid row of the last chunk
    assert generated == [2022]
    assert all(c["last_row"] is None for c in fake.calls)


def test_prompt_of_exactly_one_chunk_has_no_pad_rows():
    fake, prompt = FakeSession(), prompt_of(4)
    assert greedy(fake, prompt=prompt, max_new_tokens=1) == [3]
    assert len(fake.calls) == 1 and fake.calls[0]["query_length"] == 4
    assert fake.calls[0]["ids"] == prompt and fake.calls[0]["positions"] == [0, 1, 2, 3]


def test_prompt_shorter_than_a_chunk_is_padded_with_zeros():
    fake = FakeSession()
    assert greedy(fake, prompt=[7, 8], max_new_tokens=1) == [1]   # row 1, not a pad row
    assert len(fake.calls) == 1 and fake.calls[0]["query_length"] == 2
    assert fake.calls[0]["ids"] == [7, 8, 0, 0] and fake.calls[0]["positions"] == [0, 1, 0, 0]


def test_decode_steps_are_one_row_with_positions_t_t_plus_1_and_token_feedback():
    fake = FakeSession()
    generated = greedy(fake, prompt=[10, 11, 12], max_new_tokens=3)
    assert len(fake.calls) == 3
    assert [c["query_length"] for c in fake.calls] == [3, 1, 1]
    assert fake.calls[1]["ids_shape"] == [1, 1] and fake.calls[2]["ids_shape"] == [1, 1]
    assert fake.calls[1]["positions"] == [3] and fake.calls[2]["positions"] == [4]
    assert generated == [2, 1000, 2000]
    assert fake.calls[1]["ids"] == [generated[0]] and fake.calls[2]["ids"] == [generated[1]]


def test_one_new_token_runs_no_decode_step():
    fake = FakeSession()
    assert len(greedy(fake, prompt=[10, 11, 12], max_new_tokens=1)) == 1
    assert len(fake.calls) == 1


def test_capacity_goes_to_the_context_only_and_every_step_shares_it():
    fake = FakeSession()
    greedy(fake, capacity=8)
    assert fake.specs == [dict(capacity=8, chunk_length=4)]
    assert all(c["same_context"] for c in fake.calls)
    fake = FakeSession()
    greedy(fake, max_position=64)
    assert fake.specs == [dict(capacity=64, chunk_length=4)]  # default: the position limit


def test_context_is_disposed_exactly_once_on_success():
    fake = FakeSession()
    greedy(fake, max_new_tokens=3)
    assert fake.context.disposals == 1


@pytest.mark.parametrize("fail_at", [0, 1])
def test_a_failing_run_still_disposes_the_context_and_propagates(fail_at):
    fake = FakeSession(fail_at=fail_at)
    with pytest.raises(RuntimeError, match="the run failed"):
        greedy(fake, max_new_tokens=3)
    assert len(fake.calls) == fail_at + 1
    assert fake.context.disposals == 1


@pytest.mark.parametrize("name,outputs", [
    ("no token output", lambda call, rows: None),
    ("f32 dtype", lambda call, rows: np.zeros((1, rows, 1), dtype=np.float32)),
    ("rank 2", lambda call, rows: np.zeros((1, rows), dtype=np.int32)),
    ("row count differs from the chunk", lambda call, rows: np.zeros((1, rows + 1, 1), np.int32)),
    ("last axis is not 1", lambda call, rows: np.zeros((1, rows, 2), dtype=np.int32)),
])
def test_a_token_output_of_the_wrong_dtype_or_shape_fails_loudly(name, outputs):
    fake = FakeSession(outputs=outputs)
    with pytest.raises((TypeError, ValueError)):
        greedy(fake)
    assert fake.context.disposals == 1, name


@pytest.mark.parametrize("override", [
    dict(prompt=[]), dict(chunk_length=0), dict(chunk_length=2.5), dict(max_new_tokens=0),
    dict(max_new_tokens=-1), dict(max_new_tokens=1.5), dict(max_position=0),
    dict(max_position=2.5), dict(prompt=[10, 1.5]), dict(prompt=[10, 4294967297]),
    dict(prompt=[-1, 10]),
    dict(max_position=2),   # the last position T + K - 2 = 2 is reached: exclusive upper bound
])
def test_entry_checks_fail_before_a_context_exists(override):
    fake = FakeSession()
    with pytest.raises(ValueError):
        greedy(fake, **override)
    assert fake.specs == [] and fake.calls == []


def test_max_position_is_an_exclusive_bound():
    fake = FakeSession()
    generated = greedy(fake, max_position=3)   # T = 2, K = 2: last position 2
    assert len(generated) == 2 and fake.calls[1]["positions"] == [2]


# ---- token-only exit (generation_greedy_test.ts:462-560) --------------------------------------

def test_last_row_is_the_last_valid_row_in_prefill_and_zero_in_decode():
    fake = FakeSession(token_only=True)
    generated = generate_greedy(fake, prompt=prompt_of(6), max_new_tokens=3, chunk_length=4,
                                max_position=64)
    assert [c["last_row"] for c in fake.calls] == [3, 1, 0, 0]
    assert generated == [5001, 5002, 5003]
    assert fake.context.disposals == 1


def test_token_only_exit_rejects_an_all_rows_output():
    fake = FakeSession(outputs=lambda call, rows: np.zeros((1, 4, 1), dtype=np.int32))
    with pytest.raises(ValueError, match=r"not \[1, 1, 1\]"):
        generate_greedy(fake, prompt=prompt_of(4), max_new_tokens=1, chunk_length=4,
                        max_position=64)


def test_without_last_row_no_row_index_is_handed_over():
    fake = FakeSession()
    greedy(fake, prompt=prompt_of(6), max_new_tokens=2, max_position=64)
    assert [c["last_row"] for c in fake.calls] == [None, None, None]


# ---- GenerationContext bookkeeping (packages/runtime/src/runtime/generation-context.ts) -------

class _NoDevice:
    """Stands where the GPU context does; hands out buffers that only remember being freed."""

    class _Buf:
        def __init__(self, nbytes):
            self.nbytes, self.freed = nbytes, False

        def free(self):
            self.freed = True

    def zeros(self, nbytes):
        return self._Buf(nbytes)


def _context(**kw):
    args = dict(layers=2, kv_planes=2, depth=4, capacity=8, chunk_length=4)
    args.update(kw)
    return GenerationContext(_NoDevice(), **args)


def test_context_advances_on_success_only_and_checks_the_run_contract():
    ctx = _context()
    assert ctx.begin_run(4, 3) == 0
    ctx.advance(0, 3)
    assert ctx.past == 3
    with pytest.raises(ExecutionError):
        ctx.begin_run(3, 3)            # neither chunkLength nor 1
    with pytest.raises(ExecutionError):
        ctx.begin_run(4, 5)            # queryLength > M
    with pytest.raises(ExecutionError):
        ctx.begin_run(1, 0)
    assert ctx.begin_run(4, 4) == 3
    ctx.advance(3, 4)
    assert ctx.begin_run(1, 1) == 7
    ctx.advance(7, 1)
    with pytest.raises(ExecutionError, match="exceeds capacity"):
        ctx.begin_run(1, 1)            # 8 + 1 > 8 on a full (non-sliding) context
    with pytest.raises(GenerationContextError):
        ctx.advance(3, 1)              # stale pastLength
    sliding = _context(window=4)
    sliding.past = 100
    assert sliding.begin_run(1, 1) == 100  # a ring never fills up


def test_rewind_only_on_a_usable_full_context():
    # generation-context.ts:486-512: rewind asserts the context is usable first
    ctx = _context()
    ctx.advance(ctx.begin_run(4, 4), 4)
    ctx.rewind(2)
    assert ctx.past == 2
    with pytest.raises(ExecutionError):
        ctx.rewind(3)
    with pytest.raises(ExecutionError):
        _context(window=4).rewind(0)
    ctx.poison()
    with pytest.raises(GenerationContextError, match="poisoned"):
        ctx.rewind(0)
    with pytest.raises(GenerationContextError, match="poisoned"):
        ctx.begin_run(1, 1)
    other = _context()
    slots = other.slots_k + other.slots_v + [other.lengths]
    other.dispose()
    other.dispose()                    # idempotent
    assert all(b.freed for b in slots)
    with pytest.raises(GenerationContextError, match="disposed"):
        other.rewind(0)
    with pytest.raises(GenerationContextError, match="disposed"):
        other.begin_run(1, 1)
