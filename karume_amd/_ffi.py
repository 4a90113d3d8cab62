"""ctypes binding of libkarume_hip.so — one prototype per symbol of include/karume_hip.h.

The library is built in-tree (``python -m karume_amd.build``).  There is no fallback: if the
shared object is missing or a symbol is absent, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libkarume_hip.so")

c_ctx = C.c_void_p
c_buf = C.c_uint64
c_evt = C.c_void_p
i32 = C.c_int32
u32 = C.c_uint32
u64 = C.c_uint64
size_t = C.c_size_t

# name -> (restype, argtypes); mirrors include/karume_hip.h declaration by declaration.
PROTOTYPES = {
    "krm_version": (C.c_char_p, []),
    "krm_ctx_create": (i32, [i32, C.POINTER(c_ctx)]),
    "krm_ctx_create_on_stream": (i32, [i32, C.c_void_p, C.POINTER(c_ctx)]),
    "krm_ctx_destroy": (i32, [c_ctx]),
    "krm_last_error": (C.c_char_p, [c_ctx]),
    "krm_sync": (i32, [c_ctx]),
    "krm_buf_alloc": (i32, [c_ctx, size_t, C.POINTER(c_buf)]),
    "krm_buf_free": (i32, [c_ctx, c_buf]),
    "krm_buf_upload": (i32, [c_ctx, c_buf, size_t, C.c_void_p, size_t]),
    "krm_buf_download": (i32, [c_ctx, c_buf, size_t, C.c_void_p, size_t]),
    "krm_buf_zero": (i32, [c_ctx, c_buf, size_t, size_t]),
    "krm_buf_copy": (i32, [c_ctx, c_buf, c_buf, size_t]),
    "krm_event_create": (i32, [c_ctx, C.POINTER(c_evt)]),
    "krm_event_record": (i32, [c_ctx, c_evt]),
    "krm_event_elapsed_ms": (i32, [c_ctx, c_evt, c_evt, C.POINTER(C.c_float)]),
    "krm_event_destroy": (i32, [c_ctx, c_evt]),
    "krm_probe_launch": (i32, [c_ctx, i32, c_buf, size_t, u32, u32]),
    "krm_probe_exchange": (i32, [c_ctx, c_buf, size_t, u32, u32, u32]),
    "krm_probe_linear_series": (i32, [c_ctx, c_buf, C.POINTER(c_buf), C.POINTER(c_buf), u32, c_buf,
                                      u32, u32, u32, u32, u32, i32, i32]),
    "krm_graph_begin": (i32, [c_ctx]),
    "krm_graph_branch": (i32, [c_ctx, u32]),
    "krm_graph_end": (i32, [c_ctx, C.POINTER(C.c_void_p)]),
    "krm_graph_launch": (i32, [c_ctx, C.c_void_p]),
    "krm_graph_destroy": (i32, [c_ctx, C.c_void_p]),
    "krm_dequant_i4": (i32, [c_ctx, c_buf, c_buf, c_buf, u64, u64, u32, i32]),
    "krm_linear_i4": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, u32, u32, u32, u32, i32,
                            i32, i32]),
    "krm_linear_i4_fused": (i32, [c_ctx, c_buf, c_buf, C.c_float, c_buf, c_buf, c_buf, c_buf,
                                  c_buf, u32, u32, u32, u32, i32, i32, i32]),
    "krm_linear_i4_rows": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, u32, u32, u32,
                                 u32, i32, i32, i32, i32, i32]),
    "krm_prefill_qkv": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf,
                              c_buf, u32, u32, u32, u32, u32, u32, u32, i32, i32, i32, i32]),
    "krm_quantize_rows": (i32, [c_ctx, c_buf, c_buf, c_buf, u32, u32]),
    "krm_linear_w4a8": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, u32, u32, u32, u32,
                              i32]),
    "krm_linear_w4a8_fused": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, u32,
                                    u32, u32, u32, i32]),
    "krm_attention_state_workspace": (i32, [u32, u32, u32, u32, u32, u32, u32, u32,
                                            C.POINTER(size_t)]),
    "krm_attention_state": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, u32, u32, u32,
                                  u32, u32, u32, u32, C.c_float, u32, u32, i32, i32, c_buf,
                                  size_t]),
    "krm_attention_chunk": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, u32, u32, u32,
                                  u32, u32, u32, u32, C.c_float, u32, u32, c_buf, i32, i32, u32]),
    "krm_attention_state_noalloc": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, u32,
                                          u32, u32, u32, u32, u32, u32, C.c_float, u32, u32, i32,
                                          i32]),
    "krm_state_append": (i32, [c_ctx, c_buf, c_buf, u32, u32, u32, u32, u32, u32, u32, i32, i32]),
    "krm_attention_varlen_workspace": (i32, [u32, u32, u32, u32, u64, C.POINTER(size_t)]),
    "krm_attention_varlen": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf,
                                   C.POINTER(i32), u32, u32, u32, u32, u64, C.c_float, i32, i32,
                                   c_buf, size_t]),
    "krm_attention_varlen_plan_bytes": (i32, [u32, C.POINTER(size_t)]),
    "krm_attention_varlen_max_splits": (i32, [u32, u32, i32, u64, C.POINTER(u32)]),
    "krm_attention_varlen_plan": (i32, [c_ctx, c_buf, c_buf, u32, u32, i32, u64, u32]),
    "krm_attention_varlen_planned": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf,
                                           u32, u32, u32, u32, u64, u32, C.c_float, i32, i32,
                                           c_buf, size_t]),
    "krm_lengths_set": (i32, [c_ctx, c_buf, u32, u32]),
    "krm_lengths_advance": (i32, [c_ctx, c_buf]),
    "krm_lengths_positions": (i32, [c_ctx, c_buf, c_buf, u32]),
    "krm_lengths_log_token": (i32, [c_ctx, c_buf, c_buf, c_buf, u32]),
    "krm_lengths_step_end": (i32, [c_ctx, c_buf, c_buf, c_buf, u32, c_buf]),
    "krm_decode_head": (i32, [c_ctx, c_buf, c_buf, C.c_float, c_buf, c_buf, c_buf, c_buf, c_buf,
                              size_t, C.POINTER(u32), u32, u32, u32, i32, i32]),
    "krm_decode_tail": (i32, [c_ctx, c_buf, u32, c_buf, c_buf, c_buf, u32, c_buf, c_buf, u32, u32,
                              c_buf, i32, i32]),
    "krm_attention_state_lengths": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, u32,
                                          u32, u32, u32, u32, u32, u32, C.c_float, c_buf, u32,
                                          i32, i32, c_buf, size_t]),
    "krm_state_append_lengths": (i32, [c_ctx, c_buf, c_buf, u32, u32, u32, u32, u32, c_buf, i32,
                                       i32]),
    "krm_rms_norm": (i32, [c_ctx, c_buf, c_buf, c_buf, u32, u32, C.c_float, i32]),
    "krm_rms_norm_cast": (i32, [c_ctx, c_buf, c_buf, c_buf, u32, u32, C.c_float, i32, i32]),
    "krm_rope_half": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, u32, u32, u32, u32, i32,
                            i32]),
    "krm_decode_rope_append": (i32, [c_ctx, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, u32,
                                     u32, u32, u32, u32, u32, u32, c_buf, i32, i32]),
    "krm_decode_qkv": (i32, [c_ctx, c_buf, c_buf, C.c_float, c_buf, c_buf, c_buf, c_buf, c_buf,
                             c_buf, c_buf, c_buf, c_buf, u32, u32, u32, u32, u32, u32, u32, u32,
                             u32, c_buf, i32, i32, i32]),
    "krm_transpose_01": (i32, [c_ctx, c_buf, c_buf, u32, u32, u32, i32]),
    "krm_silu_mul": (i32, [c_ctx, c_buf, c_buf, c_buf, u64, i32]),
    "krm_add": (i32, [c_ctx, c_buf, c_buf, c_buf, u64, i32]),
    "krm_embedding": (i32, [c_ctx, c_buf, c_buf, c_buf, u32, u32, u32, i32, i32]),
    "krm_argmax": (i32, [c_ctx, c_buf, c_buf, u32, u32, i32]),
}

_lib = None


class LibraryMissingError(RuntimeError):
    """libkarume_hip.so has not been built (or lacks a declared symbol)."""


def load() -> C.CDLL:
    """Load the shared library and bind every prototype.  No computation happens here."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LibraryMissingError(
            f"{LIB_PATH} is missing: build it with `python -m karume_amd.build` "
            "(there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise LibraryMissingError(f"{LIB_PATH} does not export {name}") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib
