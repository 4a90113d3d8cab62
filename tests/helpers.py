"""Deterministic input generators shared by the tests.

They restate the generators of the reference's own hot-path tests so the same cases can be
replayed here (paths relative to the reference tree):
  * states attention: QUERY/KEY/VALUE, poison placement, the parity grid —
    packages/runtime/tests/gpu_state_attention_test.ts:56-103,119-347
  * int4 linear: SIGNED, groupVarying, the tile-edge shapes, the test-side quantiser —
    packages/runtime/tests/gpu_i4_weights_test.ts:34-45,116-145,
    packages/runtime/tests/helpers/i4.ts:43-85
"""
from __future__ import annotations

import os
import sys
from dataclasses import dataclass
from typing import Optional

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import oracle  # noqa: E402

GOLDEN = os.path.join(ROOT, "tests", "golden")
F32_TINY = np.float32(1.1754943508222875e-38)


def seeded(count: int, fn) -> np.ndarray:
    return np.array([fn(i) for i in range(count)], dtype=np.float32)


# ---------------------------------------------------------------------------- states form

def QUERY(i: int) -> float:
    return (((i * 7) % 23) - 11) * 0.17


def KEY(i: int) -> float:
    return (((i * 11) % 19) - 9) * 0.23


def VALUE(i: int) -> float:
    return (((i * 5) % 17) - 8) * 0.31


SLOT_POISON_K = 9.0
SLOT_POISON_V = 400.0


@dataclass(frozen=True)
class StateCase:
    name: str
    batch: int
    heads: int
    kv_heads: int
    chunk_rows: int
    depth: int
    capacity: int
    window: int
    past: int
    query: int
    rows_block: Optional[int] = None

    def kwargs(self) -> dict:
        return dict(batch=self.batch, heads=self.heads, kv_heads=self.kv_heads,
                    chunk_rows=self.chunk_rows, depth=self.depth, capacity=self.capacity,
                    window=self.window, past=self.past, query=self.query)


def _sc(name, b, h, hkv, m, d, c, w, p, q, rb=None) -> StateCase:
    return StateCase(name, b, h, hkv, m, d, c, w, p, q, rb)


# packages/runtime/tests/gpu_state_attention_test.ts:119-347
PARITY_CASES = [
    _sc("full r1 decode P0", 1, 2, 2, 1, 4, 16, 0, 0, 1),
    _sc("full r1 prefill B2", 2, 4, 4, 6, 8, 32, 0, 0, 6),
    _sc("full r2 pad B2 D6", 2, 4, 2, 6, 6, 32, 0, 5, 3),
    _sc("full r8 MQA decode", 2, 8, 1, 1, 16, 64, 0, 17, 1),
    _sc("full r1 rowblock 4x3", 1, 2, 2, 9, 8, 32, 0, 3, 9, 4),
    _sc("full r2 tile exact", 1, 4, 2, 16, 32, 64, 0, 16, 16),
    _sc("sliding W8 P0 decode", 1, 2, 2, 1, 4, 8, 8, 0, 1),
    _sc("sliding W8 P3 pad", 2, 4, 4, 4, 8, 8, 8, 3, 2),
    _sc("sliding W4 P3 edge", 1, 2, 2, 3, 4, 4, 4, 3, 2),
    _sc("sliding W4 P10 wrap", 2, 4, 4, 4, 8, 4, 4, 10, 2),
    _sc("sliding W4 C8 wrap", 1, 2, 2, 3, 4, 8, 4, 9, 2),
    _sc("sliding W6 r2 wrap pad", 2, 4, 2, 5, 6, 6, 6, 13, 3),
    _sc("sliding W8 r8 MQA", 2, 8, 1, 1, 16, 8, 8, 21, 1),
    _sc("sliding W2 empty rows", 1, 2, 2, 4, 4, 2, 2, 0, 1),
    _sc("sliding W2 Q4 gt W", 1, 2, 2, 4, 4, 2, 2, 5, 4),
    _sc("sliding W6 rowblock", 1, 2, 2, 8, 8, 6, 6, 20, 8, 5),
    _sc("sliding W2 P near u32 max", 1, 2, 2, 1, 4, 2, 2, 0xFFFFFFFE, 1),
]


def make_state_inputs(case: StateCase, salt: int = 0, poison: bool = True) -> dict:
    """The five arrays the attention reads, with poison in every place it must not read:
    non-resident slot rows and ins pad rows (gpu_state_attention_test.ts:72-103)."""
    b, h, hkv, m, d, c = (case.batch, case.heads, case.kv_heads, case.chunk_rows, case.depth,
                          case.capacity)
    planes = b * hkv
    q = seeded(b * h * m * d, lambda i: QUERY(i + salt))
    ins_k = seeded(planes * m * d, lambda i: KEY(i + salt))
    ins_v = seeded(planes * m * d, lambda i: VALUE(i + salt))
    slot_k = seeded(planes * c * d, lambda i: KEY(i + 3 + salt)).reshape(planes, c, d)
    slot_v = seeded(planes * c * d, lambda i: VALUE(i + 5 + salt)).reshape(planes, c, d)
    ins_k = ins_k.reshape(planes, m, d)
    ins_v = ins_v.reshape(planes, m, d)
    if poison:
        base = oracle.state_column_base(case.window, case.past)
        resident = {col % case.window if case.window else col
                    for col in range(base, case.past)}
        for row in range(c):
            if row not in resident:
                slot_k[:, row, :] = SLOT_POISON_K
                slot_v[:, row, :] = SLOT_POISON_V
        ins_k[:, case.query:, :] = SLOT_POISON_K
        ins_v[:, case.query:, :] = SLOT_POISON_V
    return dict(q=q.reshape(b, h, m, d), ins_k=ins_k.reshape(b, hkv, m, d),
                ins_v=ins_v.reshape(b, hkv, m, d), slot_k=slot_k.reshape(b, hkv, c, d),
                slot_v=slot_v.reshape(b, hkv, c, d))


def oracle_state_attention(case: StateCase, inputs: dict, mutation: int = 0,
                           scale: Optional[float] = None) -> np.ndarray:
    return oracle.state_attention(
        inputs["q"], inputs["ins_k"], inputs["ins_v"], inputs["slot_k"], inputs["slot_v"],
        scale=oracle.half_scale(case.depth) if scale is None else scale, mutation=mutation,
        **case.kwargs())


def dense_attention_f64(q, k, v, mask, scale_full: float) -> np.ndarray:
    """Textbook softmax(q k^T * scale + mask) v in float64 (independent of the oracle's loops).
    q [..., Lq, D], k/v [..., Lk, D], mask [Lq, Lk] boolean (True = visible)."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    s = np.einsum("...qd,...kd->...qk", q, k) * scale_full
    s = np.where(mask, s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p = p / p.sum(axis=-1, keepdims=True)
    return np.einsum("...qk,...kd->...qd", p, v)


# ---------------------------------------------------------------------------- int4 linear

def SIGNED(i: int) -> float:
    return ((i % 13) - 6) * 0.75


def group_varying(cols: int, group: int):
    def fn(i: int) -> float:
        g = (i % cols) // group
        row = i // cols
        base = (0.125 + (i % 11) * 0.5) * (1 if i % 2 == 0 else -1)
        return base * (1 + g * 0.75 + (row % 5) * 0.25)
    return fn


def quantize_i4(values: np.ndarray, shape, group: int):
    """Test-side quantiser: scale = max(fround(amax/7), tiny), q = round-half-away(w/scale)
    clamped to +-7, packed low nibble first (packages/runtime/tests/helpers/i4.ts:43-85).
    Returns (packed bytes, q int8, scale f32 [rows, groups])."""
    values = np.asarray(values, dtype=np.float32).reshape(-1)
    rows = shape[0]
    width = values.size // rows
    assert width % group == 0
    groups = width // group
    v = values.reshape(rows, groups, group).astype(np.float64)
    amax = np.abs(v).max(axis=2)
    scale = np.maximum((amax / 7.0).astype(np.float32), F32_TINY)
    ratio = v / scale.astype(np.float64)[:, :, None]
    rounded = np.sign(ratio) * np.floor(np.abs(ratio) + 0.5)
    q = np.clip(rounded, -7, 7).astype(np.int8).reshape(-1)
    return oracle.pack_i4(q), q, scale


@dataclass(frozen=True)
class I4LinearCase:
    name: str
    m: int
    k: int
    n: int
    group: int


# packages/runtime/tests/gpu_i4_weights_test.ts:116-145
I4_LINEAR_CASES = [
    I4LinearCase("v4 [65,48] x W[68,48] g16", 65, 48, 68, 16),
    I4LinearCase("scalar [17,32] x W[19,32] g16", 17, 32, 19, 16),
    I4LinearCase("v4 [9,96] x W[20,96] g32", 9, 96, 20, 32),
]


def make_i4_linear(case: I4LinearCase):
    x = seeded(case.m * case.k, SIGNED).reshape(case.m, case.k)
    w = seeded(case.n * case.k, group_varying(case.k, case.group)).reshape(case.n, case.k)
    bias = seeded(case.n, SIGNED)
    packed, q, scale = quantize_i4(w, (case.n, case.k), case.group)
    return x, packed, q, scale, bias


def synthetic_int4(rng: np.random.Generator, n: int, k: int, group: int, scale_f16: bool = True):
    """Benchmark-style weights: codes uniform in [-8, 7], scales |N(0, 0.02)| kept in fp16."""
    q = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    scale = np.abs(rng.normal(0.0, 0.02, size=(n, k // group))).astype(np.float32)
    if scale_f16:
        scale = np.maximum(scale.astype(np.float16), np.float16(6.104e-05))
    else:
        scale = np.maximum(scale, F32_TINY)
    return oracle.pack_i4(q), q, scale


# ---------------------------------------------------------------------------- decoder oracle

def oracle_decoder_logits(weights, ids, rows=None) -> np.ndarray:
    """Full re-forward WITHOUT a KV cache over the whole id sequence (the way the reference
    derives its greedy goldens, tools/export-recipes/_shared/decode_series.py:51-73): every op
    is the CPU oracle's; attention is one causal pass (P = 0, Q = M = T).  Returns logits [T, V]
    in float32, or [len(rows), V] for the listed positions only (the lm_head is the largest
    linear; a long sequence needs it on few rows)."""
    c = weights.config
    ids = np.asarray(ids, dtype=np.int32)
    t = ids.size
    g = c.group_size

    def lin(x, l):
        return oracle.linear_i4(x, l.packed.reshape(-1), l.scales.astype(np.float32),
                                np.zeros(l.n, dtype=np.float32), l.n, l.k, g)

    h = oracle.embedding(weights.embedding.astype(np.float32), ids)          # [T, d]
    step_kv = {}     # owner layer -> (roped k, v) of the whole sequence
    for li, lw in enumerate(weights.layers):
        depth, owner, window = c.depth_of(li), c.owner_of(li), c.window_of(li)
        cos, sin = (table[:t] for table in weights.rope_of(depth))
        xn = oracle.rms_norm(h, lw["attn_norm"], c.rms_eps)
        q = lin(xn, lw["q"]).reshape(t, c.heads, depth).transpose(1, 0, 2)
        q = oracle.rope_half(q[None], cos, sin)
        if owner == li:
            k = lin(xn, lw["k"]).reshape(t, c.kv_heads, depth).transpose(1, 0, 2)
            v = lin(xn, lw["v"]).reshape(t, c.kv_heads, depth).transpose(1, 0, 2)
            step_kv[li] = (oracle.rope_half(k[None], cos, sin), np.ascontiguousarray(v[None]))
        k, v = step_kv[owner]     # a KV-sharing layer attends over its owner's rows
        slot_rows = max(t, window)  # the slots stay unread (past = 0); window <= capacity holds
        zeros = np.zeros((1, c.kv_heads, slot_rows, depth), dtype=np.float32)
        # one causal pass over the whole sequence; `window` is the explicit band
        # (col <= row and row - col < window), no ring involved: nothing comes from a slot
        att = oracle.state_attention(q, k, v, zeros, zeros, batch=1, heads=c.heads,
                                     kv_heads=c.kv_heads, chunk_rows=t, depth=depth,
                                     capacity=slot_rows, window=window, past=0, query=t,
                                     scale=np.float32(c.half_scale_of(li)))
        att = att[0].transpose(1, 0, 2).reshape(t, c.heads * depth)
        h = (h + lin(att, lw["o"])).astype(np.float32)
        xn = oracle.rms_norm(h, lw["ffn_norm"], c.rms_eps)
        act = oracle.silu_mul(lin(xn, lw["gate"]), lin(xn, lw["up"]))
        h = (h + lin(act, lw["down"])).astype(np.float32)
    if rows is not None:
        h = np.ascontiguousarray(h[np.asarray(rows, dtype=np.int64)])
    xn = oracle.rms_norm(h, weights.final_norm, c.rms_eps)
    return lin(xn, weights.lm_head)


# ---------------------------------------------------------------------------- w4a8

def SIGNED_A8(i: int) -> float:
    """x / bias generator of the integer-dot tests (packages/runtime/tests/gpu_i8a8_test.ts:82)."""
    return ((i % 29) - 14) * 0.3717 + 0.0131


TIE_MARGIN = 1e-3  # gpu_i8a8_test.ts:86


@dataclass(frozen=True)
class W4a8Case:
    name: str
    m: int
    n: int
    k: int
    group: int


# packages/runtime/tests/gpu_i8a8_test.ts:758-769
W4A8_CASES = [
    W4a8Case("v4 [130,96] x W[68,96] g32", 130, 68, 96, 32),
    W4a8Case("scalar [129,48] x W[67,48] g16", 129, 67, 48, 16),
    W4a8Case("v4 small [3,32] x W[8,32] g32", 3, 8, 32, 32),
    W4a8Case("scalar small [17,96] x W[19,96] g32", 17, 19, 96, 32),
]


def make_w4a8(case: W4a8Case, x_value=None):
    """Inputs of one case as the reference prepares them (gpu_i8a8_test.ts:777-821): weights
    from group_varying through the test-side quantiser, bias and x from SIGNED_A8.
    x_value(index, m, k) replaces single elements of x."""
    w = seeded(case.n * case.k, group_varying(case.k, case.group)).reshape(case.n, case.k)
    packed, q, scale = quantize_i4(w, (case.n, case.k), case.group)
    bias = seeded(case.n, SIGNED_A8)
    fn = (lambda i: x_value(i, case.m, case.k)) if x_value else SIGNED_A8
    x = seeded(case.m * case.k, fn).reshape(case.m, case.k)
    return x, packed, q, scale, bias
