"""Host-side mirror of the reference's device layer for the ops this backend serves.

``acquire_gpu`` / ``GpuContext`` stand where the reference has ``acquireGpu`` / ``GpuContext``
(packages/runtime/mod.ts:13-113, packages/runtime/src/gpu/device.ts); the error classes are the
reference's public ones (packages/runtime/mod.ts:25-35,112).  Everything below is plumbing
around the C ABI: no arithmetic happens in Python.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence, Union

import numpy as np

from . import _ffi

F32 = 0
F16 = 1
COMPUTE_F32 = 0
COMPUTE_F16 = 1
PROBE_EMPTY = 0
PROBE_READ = 1
EPILOGUE_NONE = 0
CHUNK_OUT_ROW_MAJOR, CHUNK_APPEND, CHUNK_OUT_F16 = 1, 2, 4
EPILOGUE_SILU_PAIRS = 1

_NP_DTYPE_CODE = {np.dtype(np.float32): F32, np.dtype(np.float16): F16}


class KarumeError(RuntimeError):
    """Base of the errors raised by this backend."""


class GpuValidationError(KarumeError):
    """Shapes, attributes or alignment rejected before launch (status -1)."""


class GpuOutOfMemoryError(KarumeError):
    """Device allocation failed (status -2)."""


class GpuDeviceLostError(KarumeError):
    """The HIP runtime reported a failure; the context should be discarded (status -3)."""


class ExecutionError(KarumeError):
    """A run violated its contract, e.g. pastLength + queryLength > capacity (status -4)."""


_ERRORS = {-1: GpuValidationError, -2: GpuOutOfMemoryError, -3: GpuDeviceLostError,
           -4: ExecutionError}


def dtype_code(dtype) -> int:
    """KRM_F32 / KRM_F16 for a NumPy dtype."""
    try:
        return _NP_DTYPE_CODE[np.dtype(dtype)]
    except KeyError as exc:
        raise GpuValidationError(f"unsupported element type {dtype}") from exc


class DeviceBuffer:
    """A device allocation (or a borrowed device address) of ``nbytes`` bytes."""

    def __init__(self, ctx: "GpuContext", address: int, nbytes: int, owned: bool):
        self.ctx = ctx
        self.address = int(address)
        self.nbytes = int(nbytes)
        self._owned = owned

    def __int__(self) -> int:
        return self.address

    def offset(self, byte_offset: int) -> int:
        if byte_offset < 0 or byte_offset > self.nbytes:
            raise GpuValidationError(f"offset {byte_offset} outside a {self.nbytes}-byte buffer")
        return self.address + byte_offset

    def upload(self, array: np.ndarray, byte_offset: int = 0) -> None:
        data = np.ascontiguousarray(array)
        if byte_offset + data.nbytes > self.nbytes:
            raise GpuValidationError("upload past the end of the buffer")
        self.ctx._check(self.ctx._lib.krm_buf_upload(
            self.ctx._handle, self.address, byte_offset, data.ctypes.data, data.nbytes))

    def download(self, dtype, shape: Sequence[int], byte_offset: int = 0) -> np.ndarray:
        out = np.empty(tuple(shape), dtype=dtype)
        if byte_offset + out.nbytes > self.nbytes:
            raise GpuValidationError("download past the end of the buffer")
        self.ctx._check(self.ctx._lib.krm_buf_download(
            self.ctx._handle, self.address, byte_offset, out.ctypes.data, out.nbytes))
        return out

    def zero(self) -> None:
        self.ctx._check(self.ctx._lib.krm_buf_zero(self.ctx._handle, self.address, 0,
                                                    self.nbytes - self.nbytes % 4))

    def free(self) -> None:
        if self._owned and self.address:
            self.ctx._check(self.ctx._lib.krm_buf_free(self.ctx._handle, self.address))
            self.ctx._buffers.discard(self)
        self.address = 0
        self._owned = False


BufferLike = Union[DeviceBuffer, int, None]


def _addr(buf: BufferLike) -> int:
    if buf is None:
        return 0
    return int(buf)


class GpuEvent:
    def __init__(self, ctx: "GpuContext"):
        self.ctx = ctx
        handle = C.c_void_p()
        ctx._check(ctx._lib.krm_event_create(ctx._handle, C.byref(handle)))
        self._handle = handle

    def record(self) -> None:
        self.ctx._check(self.ctx._lib.krm_event_record(self.ctx._handle, self._handle))

    def elapsed_ms(self, stop: "GpuEvent") -> float:
        ms = C.c_float()
        self.ctx._check(self.ctx._lib.krm_event_elapsed_ms(
            self.ctx._handle, self._handle, stop._handle, C.byref(ms)))
        return float(ms.value)

    def destroy(self) -> None:
        if self._handle:
            self.ctx._lib.krm_event_destroy(self.ctx._handle, self._handle)
            self._handle = None


class GpuGraph:
    """A recorded launch sequence (see GpuContext.record)."""

    def __init__(self, ctx: "GpuContext", handle):
        self.ctx = ctx
        self._handle = handle

    def launch(self) -> None:
        self.ctx._check(self.ctx._lib.krm_graph_launch(self.ctx._handle, self._handle))

    def destroy(self) -> None:
        if self._handle:
            self.ctx._lib.krm_graph_destroy(self.ctx._handle, self._handle)
            self._handle = None


class _Recording:
    def __init__(self, ctx: "GpuContext"):
        self.ctx = ctx
        self.graph: Optional[GpuGraph] = None

    def branch(self, index: int) -> None:
        """The ops that follow go to parallel branch `index` (0 = main, 1..3 = side branches
        that fork from the main branch here and join it when the recording ends)."""
        self.ctx._check(self.ctx._lib.krm_graph_branch(self.ctx._handle, index))

    def __enter__(self) -> "_Recording":
        self.ctx._check(self.ctx._lib.krm_graph_begin(self.ctx._handle))
        return self

    def __exit__(self, exc_type, exc, tb) -> None:
        handle = C.c_void_p()
        status = self.ctx._lib.krm_graph_end(self.ctx._handle, C.byref(handle))
        if exc_type is None:
            self.ctx._check(status)
            self.graph = GpuGraph(self.ctx, handle)
        elif status == 0:
            self.ctx._lib.krm_graph_destroy(self.ctx._handle, handle)


class GpuContext:
    """One device + one stream; every op of this backend is queued through it."""

    def __init__(self, device: int = 0, stream: Optional[int] = None):
        self._lib = _ffi.load()
        handle = C.c_void_p()
        if stream is None:
            status = self._lib.krm_ctx_create(device, C.byref(handle))
        else:
            status = self._lib.krm_ctx_create_on_stream(device, C.c_void_p(stream), C.byref(handle))
        if status != 0:
            message = self._lib.krm_last_error(None).decode("utf-8", "replace")
            raise _ERRORS.get(status, KarumeError)(message)
        self._handle = handle
        self.device = device
        self._buffers: set[DeviceBuffer] = set()

    # -- lifecycle -------------------------------------------------------------------------
    def destroy(self) -> None:
        if self._handle:
            for buf in list(self._buffers):
                buf.free()
            self._buffers.clear()
            self._lib.krm_ctx_destroy(self._handle)
            self._handle = None

    def __enter__(self) -> "GpuContext":
        return self

    def __exit__(self, *exc) -> None:
        self.destroy()

    def _check(self, status: int) -> None:
        if status != 0:
            message = self._lib.krm_last_error(self._handle).decode("utf-8", "replace")
            raise _ERRORS.get(status, KarumeError)(message)

    def sync(self) -> None:
        self._check(self._lib.krm_sync(self._handle))

    def event(self) -> GpuEvent:
        return GpuEvent(self)

    def record(self) -> _Recording:
        """``with ctx.record() as rec: ...ops...`` then ``rec.graph.launch()`` replays them."""
        return _Recording(self)

    # -- buffers ---------------------------------------------------------------------------
    def alloc(self, nbytes: int) -> DeviceBuffer:
        address = C.c_uint64()
        self._check(self._lib.krm_buf_alloc(self._handle, nbytes, C.byref(address)))
        buf = DeviceBuffer(self, address.value, nbytes, owned=True)
        self._buffers.add(buf)
        return buf

    def upload(self, array: np.ndarray) -> DeviceBuffer:
        data = np.ascontiguousarray(array)
        buf = self.alloc(max(data.nbytes, 16))
        if data.nbytes:
            buf.upload(data)
        return buf

    def zeros(self, nbytes: int) -> DeviceBuffer:
        buf = self.alloc((nbytes + 3) // 4 * 4)
        buf.zero()
        return buf

    def copy(self, dst: BufferLike, src: BufferLike, nbytes: int) -> None:
        self._check(self._lib.krm_buf_copy(self._handle, _addr(dst), _addr(src), nbytes))

    def probe_launch(self, kind: int, src: BufferLike = None, nbytes: int = 0, grid: int = 1,
                     block: int = 256) -> None:
        """Measurement floors: PROBE_EMPTY launches a kernel that does nothing, PROBE_READ one
        that streams `nbytes` at `src` with 16-byte loads."""
        self._check(self._lib.krm_probe_launch(self._handle, kind, _addr(src), nbytes, grid,
                                               block))

    def probe_exchange(self, work: DeviceBuffer, entries: int, phases: int,
                       spin_limit: int = 1 << 16) -> None:
        """`phases` all-to-all hand-overs of a vector between the workgroups of one launch."""
        self._check(self._lib.krm_probe_exchange(self._handle, _addr(work), work.nbytes, entries,
                                                 phases, spin_limit))

    def probe_linear_series(self, x: BufferLike, weights: Sequence[BufferLike],
                            scales: Sequence[BufferLike], out: BufferLike, count: int, m: int,
                            n: int, k: int, group: int, io_dtype: int = F32,
                            scale_dtype: int = F32) -> None:
        """`count` plain launches of linear_i4 from one call, rotating over the weight copies."""
        copies = len(weights)
        w_list = (C.c_uint64 * copies)(*[_addr(b) for b in weights])
        s_list = (C.c_uint64 * copies)(*[_addr(b) for b in scales])
        self._check(self._lib.krm_probe_linear_series(
            self._handle, _addr(x), w_list, s_list, copies, _addr(out), count, m, n, k, group,
            io_dtype, scale_dtype))

    def borrow(self, address: int, nbytes: int) -> DeviceBuffer:
        """Wrap device memory owned by someone else (for example a torch tensor's data_ptr)."""
        return DeviceBuffer(self, address, nbytes, owned=False)

    # -- ops (argument order = the C ABI's) ---------------------------------------------------
    def dequant_i4(self, w: BufferLike, scales: BufferLike, out_f32: BufferLike, rows: int,
                   width: int, group: int, scale_dtype: int = F32) -> None:
        self._check(self._lib.krm_dequant_i4(self._handle, _addr(w), _addr(scales),
                                             _addr(out_f32), rows, width, group, scale_dtype))

    def linear_i4(self, x: BufferLike, w: BufferLike, scales: BufferLike, bias: BufferLike,
                  out: BufferLike, m: int, n: int, k: int, group: int, io_dtype: int = F32,
                  scale_dtype: int = F32, compute: int = COMPUTE_F32) -> None:
        self._check(self._lib.krm_linear_i4(self._handle, _addr(x), _addr(w), _addr(scales),
                                            _addr(bias), _addr(out), m, n, k, group, io_dtype,
                                            scale_dtype, compute))

    def linear_i4_fused(self, x: BufferLike, w: BufferLike, scales: BufferLike, out: BufferLike,
                        m: int, n: int, k: int, group: int, *, norm_weight: BufferLike = None,
                        norm_eps: float = 0.0, bias: BufferLike = None,
                        residual: BufferLike = None, io_dtype: int = F32, scale_dtype: int = F32,
                        epilogue: int = EPILOGUE_NONE) -> None:
        self._check(self._lib.krm_linear_i4_fused(
            self._handle, _addr(x), _addr(norm_weight), float(norm_eps), _addr(w), _addr(scales),
            _addr(bias), _addr(residual), _addr(out), m, n, k, group, io_dtype, scale_dtype,
            epilogue))

    def quantize_rows(self, x_f32: BufferLike, xq_i8: BufferLike, xs_f32: BufferLike, rows: int,
                      dim: int) -> None:
        self._check(self._lib.krm_quantize_rows(self._handle, _addr(x_f32), _addr(xq_i8),
                                                _addr(xs_f32), rows, dim))

    def linear_w4a8(self, xq_i8: BufferLike, xs_f32: BufferLike, w: BufferLike,
                    scales: BufferLike, bias_f32: BufferLike, out_f32: BufferLike, m: int, n: int,
                    k: int, group: int, scale_dtype: int = F32) -> None:
        self._check(self._lib.krm_linear_w4a8(self._handle, _addr(xq_i8), _addr(xs_f32), _addr(w),
                                              _addr(scales), _addr(bias_f32), _addr(out_f32), m, n,
                                              k, group, scale_dtype))

    def linear_w4a8_fused(self, x_f32: BufferLike, w: BufferLike, scales: BufferLike,
                          bias_f32: BufferLike, out_f32: BufferLike, m: int, n: int, k: int,
                          group: int, scale_dtype: int = F32, *, xq_i8: BufferLike = None,
                          xs_f32: BufferLike = None) -> None:
        """quantize_rows + linear_w4a8 behind one call (one launch for few rows); xq / xs are the
        work buffers of the shapes that take two launches."""
        self._check(self._lib.krm_linear_w4a8_fused(self._handle, _addr(x_f32), _addr(xq_i8),
                                                    _addr(xs_f32), _addr(w), _addr(scales),
                                                    _addr(bias_f32), _addr(out_f32), m, n, k,
                                                    group, scale_dtype))

    def attention_state_workspace(self, batch: int, heads: int, kv_heads: int, chunk_rows: int,
                                  depth: int, window: int, max_past: int, max_query: int = 1
                                  ) -> int:
        nbytes = C.c_size_t()
        self._check(self._lib.krm_attention_state_workspace(
            batch, heads, kv_heads, chunk_rows, depth, window, max_past, max_query,
            C.byref(nbytes)))
        return int(nbytes.value)

    def attention_state(self, q: BufferLike, ins_k: BufferLike, ins_v: BufferLike,
                        slot_k: BufferLike, slot_v: BufferLike, out: BufferLike, *, batch: int,
                        heads: int, kv_heads: int, chunk_rows: int, depth: int, capacity: int,
                        window: int, half_scale: float, past: int, query: int,
                        io_dtype: int = F32, kv_dtype: int = F32,
                        workspace: BufferLike = None, workspace_bytes: int = 0) -> None:
        if isinstance(workspace, DeviceBuffer) and not workspace_bytes:
            workspace_bytes = workspace.nbytes
        self._check(self._lib.krm_attention_state(
            self._handle, _addr(q), _addr(ins_k), _addr(ins_v), _addr(slot_k), _addr(slot_v),
            _addr(out), batch, heads, kv_heads, chunk_rows, depth, capacity, window,
            float(half_scale), past, query, io_dtype, kv_dtype, _addr(workspace),
            workspace_bytes))

    def attention_chunk(self, q: BufferLike, ins_k: BufferLike, ins_v: BufferLike,
                        slot_k: BufferLike, slot_v: BufferLike, out: BufferLike, *, batch: int,
                        heads: int, kv_heads: int, chunk_rows: int, depth: int, capacity: int,
                        window: int, half_scale: float, past: int = 0, query: int = 0,
                        lengths: Optional[BufferLike] = None, io_dtype: int = F32,
                        kv_dtype: int = F32, row_major: bool = False,
                        append: bool = False, out_f16: bool = False) -> None:
        """The attention of a chunk of rows with the output permute and the state appends
        folded in (D = 64 / 128); out_f16 stores the result as fp16 whatever io_dtype is."""
        flags = ((CHUNK_OUT_ROW_MAJOR if row_major else 0) | (CHUNK_APPEND if append else 0)
                 | (CHUNK_OUT_F16 if out_f16 else 0))
        self._check(self._lib.krm_attention_chunk(
            self._handle, _addr(q), _addr(ins_k), _addr(ins_v), _addr(slot_k), _addr(slot_v),
            _addr(out), batch, heads, kv_heads, chunk_rows, depth, capacity, window,
            float(half_scale), past, query, _addr(lengths), io_dtype, kv_dtype, flags))

    def attention_state_noalloc(self, q: BufferLike, ins_k: BufferLike, ins_v: BufferLike,
                                slot_k: BufferLike, slot_v: BufferLike, out: BufferLike, *,
                                batch: int, heads: int, kv_heads: int, chunk_rows: int,
                                depth: int, capacity: int, window: int, half_scale: float,
                                past: int, query: int, io_dtype: int = F32,
                                kv_dtype: int = F32) -> None:
        """attention_state without a workspace: partials and counters in the library's own
        device array (for callers that cannot allocate); rejects calls beyond its fixed size."""
        self._check(self._lib.krm_attention_state_noalloc(
            self._handle, _addr(q), _addr(ins_k), _addr(ins_v), _addr(slot_k), _addr(slot_v),
            _addr(out), batch, heads, kv_heads, chunk_rows, depth, capacity, window,
            float(half_scale), past, query, io_dtype, kv_dtype))

    def state_append(self, x: BufferLike, slot: BufferLike, *, kv_planes: int, chunk_rows: int,
                     depth: int, capacity: int, window: int, past: int, query: int,
                     x_dtype: int = F32, slot_dtype: int = F32) -> None:
        self._check(self._lib.krm_state_append(
            self._handle, _addr(x), _addr(slot), kv_planes, chunk_rows, depth, capacity, window,
            past, query, x_dtype, slot_dtype))

    def attention_varlen_workspace(self, nseq: int, heads: int, kv_heads: int, depth: int,
                                   total_rows: int) -> int:
        nbytes = C.c_size_t()
        self._check(self._lib.krm_attention_varlen_workspace(
            nseq, heads, kv_heads, depth, total_rows, C.byref(nbytes)))
        return int(nbytes.value)

    def attention_varlen(self, q: BufferLike, ins_k: BufferLike, ins_v: BufferLike,
                         slot_k: BufferLike, slot_v: BufferLike, out: BufferLike,
                         cu_seqlens: Sequence[int], *, heads: int, kv_heads: int, depth: int,
                         total_rows: int, half_scale: float, io_dtype: int = F32,
                         kv_dtype: int = F32, workspace: BufferLike = None,
                         workspace_bytes: int = 0) -> None:
        cu = np.ascontiguousarray(cu_seqlens, dtype=np.int32)
        if isinstance(workspace, DeviceBuffer) and not workspace_bytes:
            workspace_bytes = workspace.nbytes
        self._check(self._lib.krm_attention_varlen(
            self._handle, _addr(q), _addr(ins_k), _addr(ins_v), _addr(slot_k), _addr(slot_v),
            _addr(out), cu.ctypes.data_as(C.POINTER(C.c_int32)), cu.size - 1, heads, kv_heads,
            depth, total_rows, float(half_scale), io_dtype, kv_dtype, _addr(workspace),
            workspace_bytes))

    def attention_varlen_plan_bytes(self, nseq: int) -> int:
        nbytes = C.c_size_t()
        self._check(self._lib.krm_attention_varlen_plan_bytes(nseq, C.byref(nbytes)))
        return int(nbytes.value)

    def attention_varlen_max_splits(self, nseq: int, depth: int, kv_dtype: int,
                                    total_rows: int) -> int:
        splits = C.c_uint32()
        self._check(self._lib.krm_attention_varlen_max_splits(nseq, depth, kv_dtype, total_rows,
                                                              C.byref(splits)))
        return int(splits.value)

    def attention_varlen_plan(self, cu_seqlens: BufferLike, plan: BufferLike, *, nseq: int,
                              depth: int, kv_dtype: int, total_rows: int, max_splits: int) -> None:
        """Launch tables of a ragged step from a DEVICE cu_seqlens array (recordable)."""
        self._check(self._lib.krm_attention_varlen_plan(
            self._handle, _addr(cu_seqlens), _addr(plan), nseq, depth, kv_dtype, total_rows,
            max_splits))

    def attention_varlen_planned(self, q: BufferLike, ins_k: BufferLike, ins_v: BufferLike,
                                 slot_k: BufferLike, slot_v: BufferLike, out: BufferLike,
                                 plan: BufferLike, *, nseq: int, heads: int, kv_heads: int,
                                 depth: int, total_rows: int, max_splits: int, half_scale: float,
                                 io_dtype: int = F32, kv_dtype: int = F32,
                                 workspace: BufferLike = None, workspace_bytes: int = 0) -> None:
        if isinstance(workspace, DeviceBuffer) and not workspace_bytes:
            workspace_bytes = workspace.nbytes
        self._check(self._lib.krm_attention_varlen_planned(
            self._handle, _addr(q), _addr(ins_k), _addr(ins_v), _addr(slot_k), _addr(slot_v),
            _addr(out), _addr(plan), nseq, heads, kv_heads, depth, total_rows, max_splits,
            float(half_scale), io_dtype, kv_dtype, _addr(workspace), workspace_bytes))

    # -- run-time lengths on the device ----------------------------------------------------------
    def lengths_set(self, lengths: BufferLike, past: int, query: int) -> None:
        self._check(self._lib.krm_lengths_set(self._handle, _addr(lengths), past, query))

    def lengths_advance(self, lengths: BufferLike) -> None:
        self._check(self._lib.krm_lengths_advance(self._handle, _addr(lengths)))

    def lengths_positions(self, lengths: BufferLike, positions: BufferLike, rows: int) -> None:
        self._check(self._lib.krm_lengths_positions(self._handle, _addr(lengths),
                                                    _addr(positions), rows))

    def lengths_log_token(self, lengths: BufferLike, token: BufferLike, history: BufferLike,
                          history_len: int) -> None:
        self._check(self._lib.krm_lengths_log_token(self._handle, _addr(lengths), _addr(token),
                                                    _addr(history), history_len))

    def lengths_step_end(self, lengths: BufferLike, token: BufferLike, history: BufferLike,
                         history_len: int, positions: BufferLike) -> None:
        """log the token, advance the lengths, leave the next one-row step's position."""
        self._check(self._lib.krm_lengths_step_end(self._handle, _addr(lengths), _addr(token),
                                                   _addr(history), history_len,
                                                   _addr(positions)))

    def decode_head(self, x: BufferLike, w: BufferLike, scales: BufferLike, logits: BufferLike,
                    partials: DeviceBuffer, n: int, k: int, group: int, *,
                    norm_weight: BufferLike = None, norm_eps: float = 0.0,
                    bias: BufferLike = None, io_dtype: int = F32, scale_dtype: int = F16) -> int:
        """Final rms_norm + lm_head for one row, leaving per-workgroup argmax partials; returns
        how many partials the launch writes."""
        count = C.c_uint32()
        self._check(self._lib.krm_decode_head(
            self._handle, _addr(x), _addr(norm_weight), float(norm_eps), _addr(w), _addr(scales),
            _addr(bias), _addr(logits), _addr(partials), partials.nbytes, C.byref(count), n, k,
            group, io_dtype, scale_dtype))
        return int(count.value)

    def decode_tail(self, partials: BufferLike, partial_count: int, token: BufferLike,
                    lengths: BufferLike, history: BufferLike, history_len: int,
                    positions: BufferLike, table: BufferLike, vocab: int, hidden: int,
                    next_row: BufferLike, *, table_dtype: int = F16, out_dtype: int = F32) -> None:
        """argmax over the head's partials + the end of a recorded decode step + the next
        step's embedding row, one launch."""
        self._check(self._lib.krm_decode_tail(
            self._handle, _addr(partials), partial_count, _addr(token), _addr(lengths),
            _addr(history), history_len, _addr(positions), _addr(table), vocab, hidden,
            _addr(next_row), table_dtype, out_dtype))

    def attention_state_lengths(self, q: BufferLike, ins_k: BufferLike, ins_v: BufferLike,
                                slot_k: BufferLike, slot_v: BufferLike, out: BufferLike, *,
                                batch: int, heads: int, kv_heads: int, chunk_rows: int,
                                depth: int, capacity: int, window: int, half_scale: float,
                                lengths: BufferLike, max_past: int, io_dtype: int = F32,
                                kv_dtype: int = F32, workspace: BufferLike = None,
                                workspace_bytes: int = 0) -> None:
        if isinstance(workspace, DeviceBuffer) and not workspace_bytes:
            workspace_bytes = workspace.nbytes
        self._check(self._lib.krm_attention_state_lengths(
            self._handle, _addr(q), _addr(ins_k), _addr(ins_v), _addr(slot_k), _addr(slot_v),
            _addr(out), batch, heads, kv_heads, chunk_rows, depth, capacity, window,
            float(half_scale), _addr(lengths), max_past, io_dtype, kv_dtype, _addr(workspace),
            workspace_bytes))

    def state_append_lengths(self, x: BufferLike, slot: BufferLike, *, kv_planes: int,
                             chunk_rows: int, depth: int, capacity: int, window: int,
                             lengths: BufferLike, x_dtype: int = F32, slot_dtype: int = F32
                             ) -> None:
        self._check(self._lib.krm_state_append_lengths(
            self._handle, _addr(x), _addr(slot), kv_planes, chunk_rows, depth, capacity, window,
            _addr(lengths), x_dtype, slot_dtype))

    # -- decoder glue ops -----------------------------------------------------------------------
    def rms_norm(self, x: BufferLike, weight_f32: BufferLike, out: BufferLike, rows: int,
                 dim: int, eps: float, io_dtype: int = F32) -> None:
        self._check(self._lib.krm_rms_norm(self._handle, _addr(x), _addr(weight_f32), _addr(out),
                                           rows, dim, float(eps), io_dtype))

    def rms_norm_cast(self, x: BufferLike, weight_f32: BufferLike, out: BufferLike, rows: int,
                      dim: int, eps: float, io_dtype: int = F32, out_dtype: int = F16) -> None:
        """rms_norm with the result stored as out_dtype (fp16 beside f32 rows)."""
        self._check(self._lib.krm_rms_norm_cast(self._handle, _addr(x), _addr(weight_f32),
                                                _addr(out), rows, dim, float(eps), io_dtype,
                                                out_dtype))

    def rope_half(self, x: BufferLike, positions: BufferLike, cos_table: BufferLike,
                  sin_table: BufferLike, out: BufferLike, rows: int, heads: int, head_dim: int,
                  table_rows: int, to_head_major: bool = False, io_dtype: int = F32) -> None:
        self._check(self._lib.krm_rope_half(
            self._handle, _addr(x), _addr(positions), _addr(cos_table), _addr(sin_table),
            _addr(out), rows, heads, head_dim, table_rows, int(to_head_major), io_dtype))

    def decode_rope_append(self, qkv: BufferLike, positions: BufferLike, cos_table: BufferLike,
                           sin_table: BufferLike, qk_out: BufferLike, slot_k: BufferLike,
                           slot_v: BufferLike, *, heads: int, kv_heads: int, depth: int,
                           table_rows: int, capacity: int, window: int = 0, past: int = 0,
                           lengths: Optional[BufferLike] = None, io_dtype: int = F32,
                           kv_dtype: int = F32) -> None:
        """RoPE of the q and k heads of one [q; k; v] row + state_append of k and v."""
        self._check(self._lib.krm_decode_rope_append(
            self._handle, _addr(qkv), _addr(positions), _addr(cos_table), _addr(sin_table),
            _addr(qk_out), _addr(slot_k), _addr(slot_v), heads, kv_heads, depth, table_rows,
            capacity, window, past, _addr(lengths) if lengths is not None else 0, io_dtype,
            kv_dtype))

    def decode_qkv(self, x: BufferLike, w: BufferLike, scales: BufferLike, positions: BufferLike,
                   cos_table: BufferLike, sin_table: BufferLike, out: BufferLike,
                   slot_k: BufferLike, slot_v: BufferLike, *, heads: int, kv_heads: int,
                   depth: int, k: int, group: int, table_rows: int, capacity: int,
                   window: int = 0, past: int = 0, lengths: Optional[BufferLike] = None,
                   norm_weight: Optional[BufferLike] = None, norm_eps: float = 0.0,
                   bias: Optional[BufferLike] = None, io_dtype: int = F32,
                   scale_dtype: int = F32, kv_dtype: int = F32) -> None:
        """(rms_norm ->) fused [q; k; v] projection of one decode row -> RoPE of q and k ->
        state_append of k and v; q/k weight rows interleaved per head as (j, j + D/2)."""
        self._check(self._lib.krm_decode_qkv(
            self._handle, _addr(x), _addr(norm_weight) if norm_weight is not None else 0,
            float(norm_eps), _addr(w), _addr(scales), _addr(bias) if bias is not None else 0,
            _addr(positions), _addr(cos_table), _addr(sin_table), _addr(out), _addr(slot_k),
            _addr(slot_v), heads, kv_heads, depth, k, group, table_rows, capacity, window, past,
            _addr(lengths) if lengths is not None else 0, io_dtype, scale_dtype, kv_dtype))

    def linear_i4_rows(self, x: BufferLike, w: BufferLike, scales: BufferLike, out: BufferLike,
                       m: int, n: int, k: int, group: int, *, bias: Optional[BufferLike] = None,
                       residual: Optional[BufferLike] = None, io_dtype: int = F32,
                       scale_dtype: int = F32, compute: int = COMPUTE_F32,
                       epilogue: int = EPILOGUE_NONE, x_dtype: Optional[int] = None) -> None:
        """`linear` for a chunk of rows on the matrix cores, with the residual add or the
        gate/up silu-mul folded in.  x_dtype (default: io_dtype) may be F16 beside f32 io under
        COMPUTE_F16: an fp16 copy of the activations, same result."""
        self._check(self._lib.krm_linear_i4_rows(
            self._handle, _addr(x), _addr(w), _addr(scales),
            _addr(bias) if bias is not None else 0, _addr(residual) if residual is not None else 0,
            _addr(out), m, n, k, group, io_dtype, scale_dtype, compute, epilogue,
            io_dtype if x_dtype is None else x_dtype))

    def prefill_qkv(self, x: BufferLike, w: BufferLike, scales: BufferLike, positions: BufferLike,
                    cos_table: BufferLike, sin_table: BufferLike, q_out: BufferLike,
                    k_out: BufferLike, v_out: BufferLike, *, m: int, heads: int, kv_heads: int,
                    depth: int, k: int, group: int, table_rows: int,
                    bias: Optional[BufferLike] = None, io_dtype: int = F32, scale_dtype: int = F32,
                    compute: int = COMPUTE_F32, x_dtype: Optional[int] = None) -> None:
        """Fused [q; k; v] projection of m rows + RoPE of q and k, written head-major."""
        self._check(self._lib.krm_prefill_qkv(
            self._handle, _addr(x), _addr(w), _addr(scales),
            _addr(bias) if bias is not None else 0, _addr(positions), _addr(cos_table),
            _addr(sin_table), _addr(q_out), _addr(k_out), _addr(v_out), m, heads, kv_heads, depth,
            k, group, table_rows, io_dtype, scale_dtype, compute,
            io_dtype if x_dtype is None else x_dtype))

    def transpose_01(self, x: BufferLike, out: BufferLike, a: int, b: int, d: int,
                     io_dtype: int = F32) -> None:
        self._check(self._lib.krm_transpose_01(self._handle, _addr(x), _addr(out), a, b, d,
                                               io_dtype))

    def silu_mul(self, gate: BufferLike, up: BufferLike, out: BufferLike, count: int,
                 io_dtype: int = F32) -> None:
        self._check(self._lib.krm_silu_mul(self._handle, _addr(gate), _addr(up), _addr(out),
                                           count, io_dtype))

    def add(self, a: BufferLike, b: BufferLike, out: BufferLike, count: int,
            io_dtype: int = F32) -> None:
        self._check(self._lib.krm_add(self._handle, _addr(a), _addr(b), _addr(out), count,
                                      io_dtype))

    def embedding(self, table: BufferLike, index: BufferLike, out: BufferLike, rows: int,
                  vocab: int, hidden: int, table_dtype: int = F32, out_dtype: int = F32) -> None:
        self._check(self._lib.krm_embedding(self._handle, _addr(table), _addr(index), _addr(out),
                                            rows, vocab, hidden, table_dtype, out_dtype))

    def argmax(self, x: BufferLike, out_i32: BufferLike, rows: int, dim: int,
               io_dtype: int = F32) -> None:
        self._check(self._lib.krm_argmax(self._handle, _addr(x), _addr(out_i32), rows, dim,
                                         io_dtype))


def acquire_gpu(device: int = 0, stream: Optional[int] = None) -> GpuContext:
    """Create a context on ``device`` (optionally on an existing hipStream_t handle)."""
    return GpuContext(device, stream)


def version() -> str:
    return _ffi.load().krm_version().decode()
