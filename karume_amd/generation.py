"""Generation context and greedy loop — host-side mirror of the reference's control flow.

* ``GenerationContext`` follows packages/runtime/src/runtime/generation-context.ts: it owns the
  zero-initialised KV state slots (one K and one V slot per layer, ``[B, Hkv, C, D]``) and the
  run-time lengths, advances ``past`` only after a successful run, is *poisoned* by a failed
  run that may already have written state (no rollback; recover with a new context), and can
  ``rewind`` a full (non-sliding) context.
* ``plan_prefill_chunks`` / ``generate_greedy`` follow
  packages/models/src/generation/greedy.ts:106-117,196-259: fixed-length prefill chunks with
  zero-filled pad rows, then one-row decode steps feeding each token back.

Nothing here computes on tensors; the session object does the device work.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Protocol, Sequence

import numpy as np

from .runtime import DeviceBuffer, ExecutionError, GpuContext, KarumeError


class GenerationContextError(KarumeError):
    """Use of a poisoned or disposed generation context."""


@dataclass(frozen=True)
class PrefillChunk:
    position: int       # absolute position of the chunk's first valid row
    query_length: int   # valid rows, 1..chunk_length (only the last chunk may be shorter)


def _assert_positive_integer(value, where: str) -> None:
    if not isinstance(value, (int, np.integer)) or isinstance(value, bool) or value < 1:
        raise ValueError(f"{where} {value!r} is not an integer >= 1")


def plan_prefill_chunks(prompt_length: int, chunk_length: int) -> List[PrefillChunk]:
    """Fixed-length chunks; only the last may have query_length < chunk_length
    (packages/models/src/generation/greedy.ts:106-117)."""
    _assert_positive_integer(prompt_length, "prompt length")
    _assert_positive_integer(chunk_length, "chunkLength")
    return [PrefillChunk(pos, min(chunk_length, prompt_length - pos))
            for pos in range(0, prompt_length, chunk_length)]


class GenerationContext:
    """KV state slots + lengths of one sequence."""

    def __init__(self, gpu: GpuContext, *, layers: int, kv_planes: int, depth: int,
                 capacity: int, chunk_length: int, window: int = 0, kv_itemsize: int = 4,
                 layer_depths: Optional[Sequence[int]] = None,
                 layer_windows: Optional[Sequence[int]] = None,
                 layer_owners: Optional[Sequence[int]] = None):
        """`layer_depths` / `layer_windows` / `layer_owners` (each one entry per layer) describe
        decoders whose layers differ: a sliding layer's slots are rings of `window` rows (their
        capacity is the window, not the context's: the ring map is col % window whatever the
        capacity, docs/ir-v1.md:296-351), and a layer whose owner is an earlier layer has no
        slots of its own — it reads the owner's (KV-sharing: two readers, one append,
        packages/runtime/tests/gpu_state_acceptance_test.ts:866-977)."""
        _assert_positive_integer(capacity, "capacity")
        _assert_positive_integer(chunk_length, "chunkLength")
        depths = [depth] * layers if layer_depths is None else [int(v) for v in layer_depths]
        windows = [window] * layers if layer_windows is None else [int(v) for v in layer_windows]
        owners = list(range(layers)) if layer_owners is None else [int(v) for v in layer_owners]
        if not (len(depths) == len(windows) == len(owners) == layers):
            raise ExecutionError("per-layer depths / windows / owners must have one entry per layer")
        self.gpu = gpu
        self.capacity = capacity
        self.chunk_length = chunk_length
        # full layers bound the sequence by the capacity; a context of sliding layers only never
        # runs out of rows
        self.window = 0 if any(w == 0 for w in windows) else min(windows)
        self.layer_window: List[int] = windows
        self.layer_capacity: List[int] = [w if w else capacity for w in windows]
        self.past = 0
        self.poisoned = False
        self.disposed = False
        self.slots_k: List[DeviceBuffer] = []
        self.slots_v: List[DeviceBuffer] = []
        self._owned: List[DeviceBuffer] = []
        for layer in range(layers):
            owner = owners[layer]
            if owner != layer:
                if not 0 <= owner < layer or owners[owner] != owner:
                    raise ExecutionError(f"layer {layer} cannot share the slots of layer {owner}")
                self.slots_k.append(self.slots_k[owner])
                self.slots_v.append(self.slots_v[owner])
                continue
            slot_bytes = kv_planes * self.layer_capacity[layer] * depths[layer] * kv_itemsize
            # zero-initialised at creation
            # (packages/runtime/tests/gpu_state_execution_test.ts:159-164)
            k, v = gpu.zeros(slot_bytes), gpu.zeros(slot_bytes)
            self.slots_k.append(k)
            self.slots_v.append(v)
            self._owned += [k, v]
        self.lengths: DeviceBuffer = gpu.zeros(16)

    # -- run protocol (generation-context.ts:330-345,559-604) --------------------------------
    def begin_run(self, chunk_rows: int, query_length: int) -> int:
        """Checks of assertGenerationRun (packages/runtime/src/runtime/recipe.ts:252-281);
        returns the pastLength the run must use."""
        if self.disposed:
            raise GenerationContextError("the generation context was disposed")
        if self.poisoned:
            raise GenerationContextError(
                "the generation context is poisoned by a failed run; create a new one")
        if chunk_rows not in (self.chunk_length, 1):
            raise ExecutionError(
                f"chunk rows {chunk_rows} is neither chunkLength {self.chunk_length} nor 1")
        if query_length < 1 or query_length > chunk_rows:
            raise ExecutionError(f"queryLength {query_length} is outside 1..{chunk_rows}")
        if self.window == 0 and self.past + query_length > self.capacity:
            raise ExecutionError(
                f"pastLength {self.past} + queryLength {query_length} exceeds capacity "
                f"{self.capacity}")
        return self.past

    def advance(self, past: int, query_length: int) -> None:
        if past != self.past:
            raise GenerationContextError("advance() with a stale pastLength")
        self.past = past + query_length

    def poison(self) -> None:
        self.poisoned = True

    def rewind(self, position: int) -> None:
        """Forget everything at and after `position` (full contexts only,
        generation-context.ts:486-512)."""
        if self.disposed:
            raise GenerationContextError("the generation context was disposed")
        if self.poisoned:
            raise GenerationContextError(
                "the generation context is poisoned by a failed run; create a new one")
        if any(self.layer_window):
            raise ExecutionError("a sliding-window context cannot be rewound")
        if position < 0 or position > self.past:
            raise ExecutionError(f"rewind position {position} is outside 0..{self.past}")
        self.past = position

    def dispose(self) -> None:
        if self.disposed:
            return
        for buf in self._owned + [self.lengths]:
            buf.free()
        self.slots_k, self.slots_v, self._owned = [], [], []
        self.disposed = True


class GreedySession(Protocol):
    """What the greedy loop needs from a session (greedy.ts:40-47)."""

    def create_generation_context(self, *, capacity: int, chunk_length: int): ...

    def run(self, input_ids: np.ndarray, position_ids: np.ndarray, last_row: Optional[int], *,
            context, query_length: int) -> np.ndarray: ...


def generate_greedy(session: GreedySession, *, prompt: Sequence[int], max_new_tokens: int,
                    chunk_length: int, max_position: int, capacity: Optional[int] = None,
                    last_row: bool = True) -> List[int]:
    """Greedy continuation of `prompt` (packages/models/src/generation/greedy.ts:196-259).

    `session.run` receives i32 ids/positions of shape [1, M] (pad rows zero) and, with
    `last_row` (the token-only exit, the reference's default asset form), the index of the last
    valid row; it then returns the argmax token as an i32 array of shape [1, 1, 1].  Without
    `last_row` the session is handed None there and returns the argmax of every row,
    [1, M, 1], of which the last valid row is read (greedy.ts:228-236).  Entry checks run
    before the context is created; the context is disposed exactly once, also on failure."""
    _assert_positive_integer(len(prompt), "prompt length")
    chunks = plan_prefill_chunks(len(prompt), chunk_length)
    _assert_positive_integer(max_new_tokens, "maxNewTokens")
    _assert_positive_integer(max_position, "maxPosition")
    for index, token in enumerate(prompt):
        if (not isinstance(token, (int, np.integer)) or isinstance(token, bool) or token < 0
                or token > 0x7FFFFFFF):
            raise ValueError(f"prompt[{index}] {token!r} is not an integer in 0..2147483647")
    last_position = len(prompt) + max_new_tokens - 2
    if last_position >= max_position:
        raise ValueError(
            f"prompt {len(prompt)} + maxNewTokens {max_new_tokens} reaches position "
            f"{last_position}, outside 0..{max_position - 1}")
    context = session.create_generation_context(
        capacity=capacity if capacity is not None else max_position, chunk_length=chunk_length)
    try:
        token = 0
        for chunk in chunks:
            ids = np.zeros((1, chunk_length), dtype=np.int32)       # pad rows stay 0
            positions = np.zeros((1, chunk_length), dtype=np.int32)
            n = chunk.query_length
            ids[0, :n] = prompt[chunk.position:chunk.position + n]
            positions[0, :n] = np.arange(chunk.position, chunk.position + n)
            out = session.run(ids, positions, n - 1 if last_row else None, context=context,
                              query_length=n)
            token = (_read_token(out, 1, 0) if last_row
                     else _read_token(out, chunk_length, n - 1))
        generated = [token]
        for index in range(max_new_tokens - 1):
            out = session.run(np.array([[generated[index]]], dtype=np.int32),
                              np.array([[len(prompt) + index]], dtype=np.int32),
                              0 if last_row else None, context=context, query_length=1)
            generated.append(_read_token(out, 1, 0))
        return generated
    finally:
        context.dispose()


def _read_token(out, rows: int, row: int) -> int:
    """One row of the argmax output; dtype and shape are checked so that a wrong output (the
    logits, the other exit form) fails instead of yielding tokens (greedy.ts:171-188)."""
    if out is None:
        raise ValueError("the run returned no token output")
    arr = np.asarray(out)
    if arr.dtype != np.int32:
        raise TypeError(f"the token output is {arr.dtype}, not int32")
    if arr.shape != (1, rows, 1):
        raise ValueError(f"the token output has shape {list(arr.shape)}, not [1, {rows}, 1]")
    return int(arr[0, row, 0])
