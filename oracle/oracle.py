"""ctypes front-end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Loads ``oracle/libkarume_oracle.so`` (built by ``make -C oracle``) and exposes each C function
as a NumPy-in / NumPy-out call.  Nothing in the product package imports this module; it is
used by ``tests/``, by the smoke check and by the benchmark's CPU-baseline leg only.

Reference citations live next to each C function in ``oracle/karume_oracle.c``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libkarume_oracle.so")

MUT_NONE = 0
MUT_DROP_LOWER_BOUND = 1
MUT_RING_MOD_CAPACITY = 2
MUT_PAD_ROWS_COMPUTED = 3
MUT_IGNORE_KV_REPEAT = 4
MUT_SCALE_ONE_SIDE = 6
MUT_APPEND_NO_RING = 7
MUT_OVERFLOW_FORM = 8


class OracleError(ValueError):
    """The oracle rejected the shapes (mirrors the reference's ReferenceOpError / I4Error)."""


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside it and return the library path."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
        os.path.join(_HERE, "karume_oracle.c")
    ):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True,
                       stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _declare(_lib)
    return _lib


def _declare(L: C.CDLL) -> None:
    p = C.c_void_p
    z = C.c_size_t
    u64 = C.c_uint64
    L.krmo_f16_bits_to_f32.restype = C.c_float
    L.krmo_f16_bits_to_f32.argtypes = [C.c_uint16]
    L.krmo_f32_to_f16_bits.restype = C.c_uint16
    L.krmo_f32_to_f16_bits.argtypes = [C.c_float]
    L.krmo_decode_i4.restype = C.c_int
    L.krmo_decode_i4.argtypes = [p, z, z, z, p, z, p]
    L.krmo_pack_i4.restype = C.c_int
    L.krmo_pack_i4.argtypes = [p, z, p]
    for name in ("krmo_linear", "krmo_linear_mt"):
        f = getattr(L, name)
        f.restype = None
        f.argtypes = [p, p, p, z, z, z, p]
    L.krmo_linear_i4_mt.restype = C.c_int
    L.krmo_linear_i4_mt.argtypes = [p, p, p, p, z, z, z, z, p]
    L.krmo_quantize_rows.restype = None
    L.krmo_quantize_rows.argtypes = [p, z, z, p, p]
    L.krmo_quantize_rows_tie_margin.restype = C.c_double
    L.krmo_quantize_rows_tie_margin.argtypes = [p, z, z]
    L.krmo_linear_w4a8.restype = C.c_int
    L.krmo_linear_w4a8.argtypes = [p, p, p, p, z, z, z, z, C.c_int, p]
    L.krmo_state_column_base.restype = u64
    L.krmo_state_column_base.argtypes = [u64, u64]
    L.krmo_state_live_columns.restype = u64
    L.krmo_state_live_columns.argtypes = [u64, u64, u64]
    L.krmo_state_effective_rows.restype = u64
    L.krmo_state_effective_rows.argtypes = [u64, u64, u64]
    L.krmo_state_attention_mut.restype = C.c_int
    L.krmo_state_attention_mut.argtypes = [p] * 6 + [u64] * 9 + [C.c_float, p, C.c_int]
    L.krmo_state_append_mut.restype = C.c_int
    L.krmo_state_append_mut.argtypes = [p, p] + [u64] * 7 + [C.c_int]
    L.krmo_allclose.restype = z
    L.krmo_allclose.argtypes = [p, p, z, C.c_double, C.c_double, C.POINTER(C.c_double),
                                C.POINTER(z)]
    L.krmo_rms_norm.restype = None
    L.krmo_rms_norm.argtypes = [p, p, z, z, C.c_double, p]
    L.krmo_argmax.restype = None
    L.krmo_argmax.argtypes = [p, z, z, p]
    L.krmo_rope_half.restype = None
    L.krmo_rope_half.argtypes = [p, p, p, z, z, z, p]
    L.krmo_silu_mul.restype = None
    L.krmo_silu_mul.argtypes = [p, p, z, p]
    L.krmo_embedding.restype = C.c_int
    L.krmo_embedding.argtypes = [p, p, z, z, z, p]


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


# ---------------------------------------------------------------------------- formats

def f16_bits_to_f32(bits: int) -> float:
    return float(lib().krmo_f16_bits_to_f32(int(bits) & 0xFFFF))


def f32_to_f16_bits(value: float) -> int:
    return int(lib().krmo_f32_to_f16_bits(np.float32(value)))


def group_scale_shape(shape, group: int):
    """[shape[0], (numel/shape[0]) / group] — packages/runtime/src/format/i4.ts:44-50."""
    dims = [int(d) for d in shape]
    numel = int(np.prod(dims)) if dims else 1
    return [dims[0], (numel / dims[0]) / group]


def decode_i4(data: bytes | np.ndarray, shape, scale, scale_shape, group: int) -> np.ndarray:
    """decodeI4 with its rejections — packages/runtime/src/format/i4.ts:63-118."""
    shape = [int(d) for d in shape]
    if len(shape) == 0:
        raise OracleError("rank 0 int4 weight has no quantisation axis")
    raw = np.frombuffer(bytes(data), dtype=np.uint8) if not isinstance(data, np.ndarray) \
        else np.ascontiguousarray(data, dtype=np.uint8)
    count = int(np.prod(shape))
    if count % 2 != 0 or raw.size * 2 != count:
        raise OracleError(f"payload of {raw.size} bytes does not match shape {shape}")
    width = count // shape[0] if shape[0] else 0
    if not isinstance(group, (int, np.integer)) or group < 1 or width % group != 0:
        raise OracleError(f"group_size {group} does not divide the row length {width}")
    expected = [shape[0], width // group]
    if list(scale_shape) != expected:
        raise OracleError(f"scale {list(scale_shape)} is not the group shape {expected}")
    scale = _f32(scale).reshape(-1)
    if scale.size != int(np.prod(scale_shape)):
        raise OracleError("scale element count does not match its shape")
    out = np.empty(count, dtype=np.float32)
    rc = lib().krmo_decode_i4(_ptr(raw), raw.size, shape[0], width, _ptr(scale), group, _ptr(out))
    if rc != 0:
        raise OracleError("decode_i4 rejected the shapes")
    return out.reshape(shape)


def pack_i4(q) -> np.ndarray:
    """q in [-8, 7] (any shape, even count) -> packed bytes; emit.py:292-322."""
    q = np.ascontiguousarray(q, dtype=np.int8).reshape(-1)
    out = np.empty(q.size // 2, dtype=np.uint8)
    if lib().krmo_pack_i4(_ptr(q), q.size, _ptr(out)) != 0:
        raise OracleError("pack_i4: odd count or value outside [-8, 7]")
    return out


# ---------------------------------------------------------------------------- linear

def linear(x, w, bias, threads: bool = False) -> np.ndarray:
    """referenceLinear — x[..., K] · w[N, K]^T + bias[N], double accumulate."""
    x = _f32(x)
    w = _f32(w)
    bias = _f32(bias)
    n, k = w.shape
    if x.shape[-1] != k or bias.shape != (n,):
        raise OracleError(f"linear shapes x{x.shape} w{w.shape} b{bias.shape}")
    m = x.size // k if k else 0
    out = np.empty((m, n), dtype=np.float32)
    fn = lib().krmo_linear_mt if threads else lib().krmo_linear
    fn(_ptr(x), _ptr(w), _ptr(bias), m, n, k, _ptr(out))
    return out.reshape(x.shape[:-1] + (n,))


def linear_i4(x, packed, scale, bias, n: int, k: int, group: int) -> np.ndarray:
    """decode_i4 followed by linear, one weight row at a time (OpenMP over output columns)."""
    x = _f32(x)
    packed = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
    scale = _f32(scale).reshape(-1)
    bias = _f32(bias)
    if packed.size * 2 != n * k or scale.size * group != n * k or x.shape[-1] != k:
        raise OracleError("linear_i4 shapes")
    m = x.size // k
    out = np.empty((m, n), dtype=np.float32)
    rc = lib().krmo_linear_i4_mt(_ptr(x), _ptr(packed), _ptr(scale), _ptr(bias), m, n, k, group,
                                 _ptr(out))
    if rc != 0:
        raise OracleError("linear_i4 rejected the shapes")
    return out.reshape(x.shape[:-1] + (n,))


def quantize_rows(x, dim: int):
    """Per-row symmetric int8 quantisation -> (q int8 [rows, dim], scale f32 [rows])."""
    x = _f32(x).reshape(-1, dim) if dim else _f32(x).reshape(0, 0)
    rows = x.shape[0]
    q = np.empty((rows, dim), dtype=np.int8)
    scale = np.empty(rows, dtype=np.float32)
    lib().krmo_quantize_rows(_ptr(x), rows, dim, _ptr(q), _ptr(scale))
    return q, scale


def quantize_rows_tie_margin(x, dim: int) -> float:
    x = _f32(x).reshape(-1, dim)
    return float(lib().krmo_quantize_rows_tie_margin(_ptr(x), x.shape[0], dim))


def linear_w4a8(x, packed, scale, bias, n: int, k: int, group: int, fused: bool = True):
    """w4a8 linear: int8 rows of x against packed int4 weights, one f32 flush per group."""
    x = _f32(x)
    packed = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
    scale = _f32(scale).reshape(-1)
    bias = _f32(bias) if bias is not None else np.zeros(n, dtype=np.float32)
    if packed.size * 2 != n * k or scale.size * group != n * k or x.shape[-1] != k:
        raise OracleError("linear_w4a8 shapes")
    m = x.size // k
    out = np.empty((m, n), dtype=np.float32)
    rc = lib().krmo_linear_w4a8(_ptr(x), _ptr(packed), _ptr(scale), _ptr(bias), m, n, k, group,
                                1 if fused else 0, _ptr(out))
    if rc != 0:
        raise OracleError("linear_w4a8 rejected the shapes")
    return out.reshape(x.shape[:-1] + (n,))


# ---------------------------------------------------------------------------- states form

def state_column_base(window: int, past: int) -> int:
    return int(lib().krmo_state_column_base(window, past))


def state_live_columns(window: int, past: int, query: int) -> int:
    return int(lib().krmo_state_live_columns(window, past, query))


def state_effective_rows(rows_block: int, row_offset: int, query: int) -> int:
    return int(lib().krmo_state_effective_rows(rows_block, row_offset, query))


def state_attention(q, ins_k, ins_v, slot_k, slot_v, *, batch, heads, kv_heads, chunk_rows,
                    depth, capacity, window, past, query, scale, mutation: int = MUT_NONE
                    ) -> np.ndarray:
    """referenceStateAttention; returns out[B, H, M, D] (pad rows exact 0)."""
    q, ins_k, ins_v, slot_k, slot_v = map(_f32, (q, ins_k, ins_v, slot_k, slot_v))
    for name, arr, want in (
        ("q", q, batch * heads * chunk_rows * depth),
        ("insK", ins_k, batch * kv_heads * chunk_rows * depth),
        ("insV", ins_v, batch * kv_heads * chunk_rows * depth),
        ("slotK", slot_k, batch * kv_heads * capacity * depth),
        ("slotV", slot_v, batch * kv_heads * capacity * depth),
    ):
        if arr.size != want:
            raise OracleError(f"{name}: {arr.size} elements, expected {want}")
    out = np.empty((batch, heads, chunk_rows, depth), dtype=np.float32)
    live = max(1, state_live_columns(window, past, query))
    scratch = np.empty(2 * live, dtype=np.float32)
    rc = lib().krmo_state_attention_mut(
        _ptr(q), _ptr(ins_k), _ptr(ins_v), _ptr(slot_k), _ptr(slot_v), _ptr(out),
        batch, heads, kv_heads, chunk_rows, depth, capacity, window, past, query,
        np.float32(scale), _ptr(scratch), mutation)
    if rc != 0:
        raise OracleError("state_attention rejected the shapes")
    return out


def state_append(x, slot, *, kv_planes, chunk_rows, depth, capacity, window, past, query,
                 mutation: int = MUT_NONE) -> np.ndarray:
    """referenceStateAppend; returns a COPY of the slot after the write."""
    x = _f32(x)
    out = _f32(slot).copy()
    if x.size != kv_planes * chunk_rows * depth or out.size != kv_planes * capacity * depth:
        raise OracleError("state_append element counts")
    rc = lib().krmo_state_append_mut(_ptr(x), _ptr(out), kv_planes, chunk_rows, depth, capacity,
                                     window, past, query, mutation)
    if rc != 0:
        raise OracleError("state_append rejected the shapes")
    return out.reshape(kv_planes, capacity, depth)


def half_scale(depth: int) -> np.float32:
    """fround(sqrt(1/sqrt(D))) — packages/runtime/tests/helpers/state-dispatch.ts:63."""
    return np.float32(np.sqrt(1.0 / np.sqrt(float(depth))))


def allclose(actual, expected, atol: float = 1e-5, rtol: float = 1e-3):
    """allclose report (pass, fail_count, max_abs, worst_index) — reference/allclose.ts:47-82."""
    a = _f32(actual).reshape(-1)
    e = _f32(expected).reshape(-1)
    if a.size != e.size:
        raise OracleError(f"length mismatch {a.size} vs {e.size}")
    max_abs = C.c_double(0)
    worst = C.c_size_t(0)
    fail = lib().krmo_allclose(_ptr(a), _ptr(e), a.size, atol, rtol, C.byref(max_abs),
                               C.byref(worst))
    return fail == 0, int(fail), float(max_abs.value), int(worst.value)


# ---------------------------------------------------------------------------- decoder glue

def rms_norm(x, weight, eps: float) -> np.ndarray:
    x = _f32(x)
    weight = _f32(weight)
    dim = x.shape[-1]
    out = np.empty_like(x)
    lib().krmo_rms_norm(_ptr(x), _ptr(weight), x.size // dim, dim, eps, _ptr(out))
    return out


def argmax(x) -> np.ndarray:
    x = _f32(x)
    dim = x.shape[-1]
    out = np.empty(x.size // dim, dtype=np.int32)
    lib().krmo_argmax(_ptr(x), x.size // dim, dim, _ptr(out))
    return out.reshape(x.shape[:-1] + (1,))


def rope_half(x, cos, sin) -> np.ndarray:
    """x[B,H,S,D], cos/sin[S,D] -> x*cos + rotate_half(x)*sin."""
    x = _f32(x)
    cos = _f32(cos)
    sin = _f32(sin)
    b, h, s, d = x.shape
    out = np.empty_like(x)
    lib().krmo_rope_half(_ptr(x), _ptr(cos), _ptr(sin), b * h, s, d, _ptr(out))
    return out


def silu_mul(gate, up) -> np.ndarray:
    gate = _f32(gate)
    up = _f32(up)
    out = np.empty_like(gate)
    lib().krmo_silu_mul(_ptr(gate), _ptr(up), gate.size, _ptr(out))
    return out


def embedding(weight, index) -> np.ndarray:
    weight = _f32(weight)
    index = np.ascontiguousarray(index, dtype=np.int32)
    vocab, hidden = weight.shape
    out = np.empty((index.size, hidden), dtype=np.float32)
    if lib().krmo_embedding(_ptr(weight), _ptr(index), index.size, vocab, hidden, _ptr(out)) != 0:
        raise OracleError("embedding index out of range")
    return out.reshape(index.shape + (hidden,))
