"""On-disk model reader: safetensors container + the `karume_ir` weight table.

Host-side mirror of the reference's loader for the parts the int4 hot path needs — it reads
nothing from disk itself (the caller hands over the bytes) and copies nothing (tensor payloads
are memoryview slices of the caller's buffer):

* ``parse_safetensors`` follows packages/runtime/src/format/safetensors.ts:10-276: layout
  ``[u64 LE header length][header JSON][data]``, ``data_offsets`` relative to the data section,
  byte length = ``numel * bits / 8`` exactly (``I4`` is 4 bits per element with the LOGICAL
  shape), the data section covered by the declarations without gaps, overlaps or a tail, and a
  start alignment per dtype (``I4`` tensors start on 4 bytes because the kernels bind them as
  u32 words).
* ``open_model`` follows packages/runtime/src/format/container.ts:96-130,215-384 and the storage
  rules of packages/runtime/src/format/ir.ts:268-305,620-650 (docs/ir-v1.md:125-206): every
  initializer names a tensor whose safetensors dtype and shape match its declaration; ``i8`` and
  ``i4`` storage carry a companion F32 scale tensor (``storage.scale``), ``i4`` also a
  ``storage.group_size`` (power of two >= 16 dividing the row length ``numel / shape[0]``) and a
  rank-2 scale ``[shape[0], row length / group_size]``; tensors that no initializer references
  are rejected.  Only the weight table of the graph is validated here — nodes are read as far
  as the residency rule needs them.
* ``i4_resident_initializers`` is the residency rule of
  packages/runtime/src/runtime/plan.ts:366-431: an int4 initializer stays packed on the device
  only if every use is the weight slot of ``linear`` / ``embedding`` / ``conv1d`` with
  ``groups == 1`` and it is not a graph output; anything else is expanded to f32 at load.
"""
from __future__ import annotations

import json
import struct
from dataclasses import dataclass
from typing import Dict, List, Mapping, Optional, Sequence, Set, Tuple

import numpy as np

from .format_i4 import I4Error, check_int4, group_scale_shape

# dtype -> bits per element / required alignment of the tensor's first byte
# (packages/runtime/src/format/safetensors.ts:26-56)
_DTYPE_BITS = {"F32": 32, "F16": 16, "BF16": 16, "I8": 8, "I4": 4, "U8": 8, "I32": 32,
               "U32": 32, "I64": 64, "BOOL": 8}
_DTYPE_ALIGN = {"F32": 4, "F16": 2, "BF16": 2, "I8": 1, "I4": 4, "U8": 1, "I32": 4, "U32": 4,
                "I64": 8, "BOOL": 1}
# storage dtype of the IR -> safetensors dtype (container.ts:96-104)
_STORAGE_ENCODING = {"f32": "F32", "f16": "F16", "bf16": "BF16", "i8": "I8", "i4": "I4",
                     "i32": "I32"}
_QUANTIZED = ("i8", "i4")
_MIN_GROUP_SIZE = 16
_MAX_SAFE_INTEGER = 2 ** 53 - 1
IR_METADATA_KEY = "karume_ir"
# op -> input slot that holds the weight (packages/runtime/src/ops/names.ts:356-362)
_WEIGHT_SLOTS = {"linear": 1, "conv1d": 1, "conv2d": 1, "conv_transpose1d": 1, "embedding": 0}
_I4_WEIGHT_OPS = ("linear", "embedding", "conv1d")


class SafetensorsError(ValueError):
    """The file is not a well-formed safetensors container."""


class ContainerError(ValueError):
    """The container and its karume_ir weight table do not agree."""


class IrError(ValueError):
    """The karume_ir JSON breaks a declaration rule."""


@dataclass(frozen=True)
class TensorView:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    byte_offset: int   # absolute, from the start of the buffer
    byte_length: int


@dataclass(frozen=True)
class SafetensorsFile:
    buffer: memoryview
    metadata: Mapping[str, str]
    tensors: Mapping[str, TensorView]


def _as_index(value, where: str, what: str) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 0 or \
            value > _MAX_SAFE_INTEGER:
        raise SafetensorsError(f"{where}: {what} {value!r} is not a non-negative integer")
    return value


def parse_safetensors(buffer) -> SafetensorsFile:
    """Strictly validated tensor table of one safetensors file held in memory."""
    view = memoryview(buffer).cast("B")
    if len(view) < 8:
        raise SafetensorsError(f"file too short: {len(view)} bytes (no header length)")
    (header_length,) = struct.unpack_from("<Q", view, 0)
    if header_length > _MAX_SAFE_INTEGER:
        raise SafetensorsError(f"header length {header_length} exceeds the safe integer range")
    data_start = 8 + header_length
    if data_start > len(view):
        raise SafetensorsError(f"header length {header_length} exceeds the file length "
                               f"{len(view)}")
    try:
        text = bytes(view[8:data_start]).decode("utf-8", errors="strict")
    except UnicodeDecodeError:
        raise SafetensorsError("the header is not valid UTF-8") from None
    try:
        header = json.loads(text)
    except json.JSONDecodeError as err:
        raise SafetensorsError(f"the header JSON cannot be parsed: {err}") from None
    if not isinstance(header, dict):
        raise SafetensorsError("the header JSON is not an object")

    metadata: Dict[str, str] = {}
    declared = []
    for name, raw in header.items():
        if name == "__metadata__":
            if not isinstance(raw, dict):
                raise SafetensorsError("__metadata__ is not an object")
            for key, item in raw.items():
                if not isinstance(item, str):
                    raise SafetensorsError(f"__metadata__.{key} is not a string")
                metadata[key] = item
            continue
        where = f"tensor '{name}'"
        if not isinstance(raw, dict):
            raise SafetensorsError(f"{where}: the header entry is not an object")
        dtype = raw.get("dtype")
        if not isinstance(dtype, str) or dtype not in _DTYPE_BITS:
            raise SafetensorsError(f"{where}: unsupported dtype {json.dumps(dtype)}")
        if not isinstance(raw.get("shape"), list):
            raise SafetensorsError(f"{where}: shape is not an array")
        shape = tuple(_as_index(dim, where, "shape element") for dim in raw["shape"])
        offsets = raw.get("data_offsets")
        if not isinstance(offsets, list):
            raise SafetensorsError(f"{where}: data_offsets is not an array")
        if len(offsets) != 2:
            raise SafetensorsError(f"{where}: data_offsets has {len(offsets)} entries (2 needed)")
        begin = _as_index(offsets[0], where, "data_offsets")
        end = _as_index(offsets[1], where, "data_offsets")
        if end < begin:
            raise SafetensorsError(f"{where}: data_offsets are reversed [{begin}, {end})")
        count = 1
        for dim in shape:
            count *= dim
            if count > _MAX_SAFE_INTEGER:
                raise SafetensorsError(f"{where}: the element count exceeds the safe range")
        bits = count * _DTYPE_BITS[dtype]
        if bits % 8 != 0:  # an odd number of I4 elements: the last one would stick out
            raise SafetensorsError(
                f"{where}: {count} elements of {dtype} ({_DTYPE_BITS[dtype]} bits each) do not "
                "end on a byte boundary")
        if end - begin != bits // 8:
            raise SafetensorsError(
                f"{where}: size mismatch, offsets={end - begin} expected={bits // 8} "
                f"({dtype} [{','.join(map(str, shape))}])")
        declared.append((begin, end, name, dtype, shape))

    data_length = len(view) - data_start
    tensors: Dict[str, TensorView] = {}
    cursor = 0
    for begin, end, name, dtype, shape in sorted(declared, key=lambda d: (d[0], d[1])):
        where = f"tensor '{name}'"
        if begin < cursor:
            raise SafetensorsError(f"{where}: overlaps the preceding tensor [{begin}, {end}), "
                                   f"used up to {cursor}")
        if begin > cursor:
            raise SafetensorsError(f"{where}: unused bytes [{cursor}, {begin}) in the data section")
        if end > data_length:
            raise SafetensorsError(f"{where}: [{begin}, {end}) lies outside the data section of "
                                   f"{data_length} bytes")
        align = _DTYPE_ALIGN[dtype]
        if (data_start + begin) % align != 0:
            raise SafetensorsError(f"{where}: absolute offset {data_start + begin} is not aligned "
                                   f"to the {align} bytes {dtype} needs")
        cursor = end
        tensors[name] = TensorView(name, dtype, shape, data_start + begin, end - begin)
    if cursor != data_length:
        raise SafetensorsError(f"{data_length - cursor} unused bytes at the end of the data section")
    return SafetensorsFile(view, metadata, tensors)


def tensor_bytes(file: SafetensorsFile, view: TensorView) -> memoryview:
    """The tensor's raw bytes (no copy; I4 has no element type of its own)."""
    return file.buffer[view.byte_offset:view.byte_offset + view.byte_length]


# ---------------------------------------------------------------------------------- karume_ir

@dataclass(frozen=True)
class Storage:
    dtype: str
    scale: Optional[str] = None
    group_size: Optional[int] = None


@dataclass(frozen=True)
class Initializer:
    name: str
    tensor: str
    storage: Storage
    dtype: str               # semantic dtype: f32 or i32
    shape: Tuple[int, ...]


@dataclass(frozen=True)
class KarumeModel:
    graph: dict                          # the parsed karume_ir JSON
    initializers: Mapping[str, Initializer]
    file: SafetensorsFile


def _reject_non_finite(text: str):
    def bad(token):
        raise IrError(f"non-finite number {token} in the graph JSON")
    return json.loads(text, parse_constant=bad)


def _parse_storage(raw, where: str) -> Storage:
    if not isinstance(raw, dict):
        raise IrError(f"{where}: not an object")
    unknown = set(raw) - {"dtype", "scale", "group_size"}
    if unknown or "dtype" not in raw:
        raise IrError(f"{where}: keys {sorted(raw)} (dtype required; scale, group_size optional)")
    dtype = raw["dtype"]
    if dtype not in _STORAGE_ENCODING:
        raise IrError(f"{where}.dtype: unknown storage dtype {dtype!r}")
    has_scale, has_group = "scale" in raw, "group_size" in raw
    if dtype not in _QUANTIZED and (has_scale or has_group):
        raise IrError(f"{where}: storage dtype '{dtype}' cannot carry scale / group_size")
    if dtype in _QUANTIZED and not has_scale:
        raise IrError(f"{where}: storage dtype '{dtype}' needs scale (the scale tensor's key)")
    if dtype == "i4" and not has_group:
        raise IrError(f"{where}: storage dtype 'i4' needs group_size")
    scale = None
    if has_scale:
        scale = raw["scale"]
        if not isinstance(scale, str) or not scale:
            raise IrError(f"{where}.scale: not a non-empty string")
    group = None
    if has_group:
        group = raw["group_size"]
        if isinstance(group, bool) or not isinstance(group, int) or group < 1:
            raise IrError(f"{where}.group_size: not a positive integer")
        if dtype == "i4" and (group & (group - 1) or group < _MIN_GROUP_SIZE):
            raise IrError(f"{where}.group_size: {group} is not a power of two >= "
                          f"{_MIN_GROUP_SIZE}")
    return Storage(dtype, scale, group)


def _parse_initializers(graph: dict) -> Dict[str, Initializer]:
    raw_inits = graph.get("initializers", {})
    values = graph.get("values", {})
    if not isinstance(raw_inits, dict) or not isinstance(values, dict):
        raise IrError("graph.initializers / graph.values: not objects")
    out: Dict[str, Initializer] = {}
    for name, raw in raw_inits.items():
        where = f"graph.initializers['{name}']"
        if not isinstance(raw, dict) or set(raw) != {"tensor", "storage"}:
            raise IrError(f"{where}: needs exactly the keys tensor and storage")
        tensor = raw["tensor"]
        if not isinstance(tensor, str) or not tensor:
            raise IrError(f"{where}.tensor: not a non-empty string")
        storage = _parse_storage(raw["storage"], f"{where}.storage")
        info = values.get(name)
        if not isinstance(info, dict) or "dtype" not in info or "shape" not in info:
            raise IrError(f"graph.values['{name}']: the initializer is not declared")
        dtype, shape = info["dtype"], info["shape"]
        if not isinstance(shape, list) or any(
                isinstance(d, bool) or not isinstance(d, int) or d < 0 for d in shape):
            raise IrError(f"graph.values['{name}']: an initializer needs a numeric shape")
        # semantic x storage: f32 x {f32, f16, bf16, i8, i4}; i32 x i32 (docs/ir-v1.md:186-195)
        if not ((dtype == "f32" and storage.dtype != "i32") or
                (dtype == "i32" and storage.dtype == "i32")):
            raise IrError(f"{where}: semantic dtype '{dtype}' cannot be combined with storage "
                          f"'{storage.dtype}'")
        if storage.dtype == "i4":
            if len(shape) == 0:
                raise IrError(f"graph.values['{name}']: an i4 initializer needs rank >= 1")
            numel = int(np.prod(shape, dtype=np.int64))
            width = numel // shape[0] if shape[0] else 0
            if shape[0] == 0 or width % storage.group_size:
                raise IrError(f"graph.values['{name}']: the i4 row length {width} "
                              f"(= numel / {shape[0]}) is not a multiple of group_size "
                              f"{storage.group_size}")
        out[name] = Initializer(name, tensor, storage, dtype, tuple(shape))
    return out


def _check_scale_tensor(init: Initializer, view: TensorView) -> None:
    where = f"initializer '{init.name}'"
    if view.dtype != "F32":
        raise ContainerError(f"{where}: scale tensor '{init.storage.scale}' is {view.dtype} "
                             "(F32 needed)")
    if init.storage.dtype == "i4":
        expected = [int(d) for d in group_scale_shape(init.shape, init.storage.group_size)]
        if len(view.shape) != len(expected):
            raise ContainerError(f"{where}: scale {list(view.shape)} does not have the rank of "
                                 f"the group shape {expected} (rank 2 whatever the weight's rank)")
        if list(view.shape) != expected:
            raise ContainerError(f"{where}: scale {list(view.shape)} is not the group shape "
                                 f"{expected} of weight {list(init.shape)} "
                                 f"(group_size={init.storage.group_size})")
        return
    if len(view.shape) != len(init.shape):
        raise ContainerError(f"{where}: scale {list(view.shape)} does not have the weight's rank "
                             f"{list(init.shape)} (keepdim broadcast shape needed)")
    if not all(d == 1 or d == w for d, w in zip(view.shape, init.shape)):
        raise ContainerError(f"{where}: scale {list(view.shape)} does not broadcast over weight "
                             f"{list(init.shape)}")


def open_model(buffer) -> KarumeModel:
    """One safetensors file -> the validated weight table of its karume_ir graph."""
    file = parse_safetensors(buffer)
    text = file.metadata.get(IR_METADATA_KEY)
    if text is None:
        raise ContainerError(f"__metadata__.{IR_METADATA_KEY} is missing (not a Karume model)")
    try:
        graph = _reject_non_finite(text)
    except json.JSONDecodeError as err:
        raise IrError(f"the graph JSON cannot be parsed: {err}") from None
    if not isinstance(graph, dict) or graph.get("format") != "karume-ir":
        raise IrError("graph.format is not 'karume-ir'")
    if graph.get("version") != 1:
        raise IrError(f"graph.version {graph.get('version')!r} is not 1")
    initializers = _parse_initializers(graph)

    tensor_keys = {init.tensor for init in initializers.values()}
    referenced: Set[str] = set(tensor_keys)
    for init in initializers.values():
        where = f"initializer '{init.name}'"
        view = file.tensors.get(init.tensor)
        if view is None:
            raise ContainerError(f"{where}: tensor '{init.tensor}' is not in the file")
        if view.dtype != _STORAGE_ENCODING[init.storage.dtype]:
            raise ContainerError(f"{where}: tensor '{init.tensor}' is {view.dtype}, the declared "
                                 f"storage '{init.storage.dtype}' needs "
                                 f"{_STORAGE_ENCODING[init.storage.dtype]}")
        if tuple(view.shape) != init.shape:
            raise ContainerError(f"{where}: declared shape {list(init.shape)} differs from the "
                                 f"tensor's {list(view.shape)}")
        if init.storage.scale is not None:
            if init.storage.scale in tensor_keys:
                raise ContainerError(f"{where}: scale key '{init.storage.scale}' collides with an "
                                     "initializer's tensor")
            scale = file.tensors.get(init.storage.scale)
            if scale is None:
                raise ContainerError(f"{where}: scale tensor '{init.storage.scale}' is not in the "
                                     f"file (it must sit beside '{init.tensor}')")
            _check_scale_tensor(init, scale)
            referenced.add(init.storage.scale)
    surplus = sorted(set(file.tensors) - referenced)
    if surplus:
        raise ContainerError(f"tensors no initializer references ({len(surplus)}): "
                             f"{', '.join(surplus)}")
    return KarumeModel(graph, initializers, file)


def i4_resident_initializers(model: KarumeModel) -> Set[str]:
    """Names of the int4 initializers that stay packed on the device."""
    graph = model.graph
    names = set(model.initializers)
    eligible: Set[str] = set()
    disqualified: Set[str] = set(graph.get("outputs", []))
    other_kernel: Set[str] = set()
    for node in graph.get("nodes", []):
        op, ins = node.get("op"), node.get("ins", [])
        slot = _WEIGHT_SLOTS.get(op)
        for index, name in enumerate(ins):
            if name not in names:
                continue
            if index == slot:
                eligible.add(name)
                expands = op in _I4_WEIGHT_OPS
                if op == "conv1d":
                    attrs = node.get("attrs", {})
                    if "groups" not in attrs:
                        raise IrError("nodes (conv1d): attrs.groups is missing")
                    expands = attrs["groups"] == 1
                if not expands:
                    other_kernel.add(name)
            else:
                disqualified.add(name)
    return {name for name in eligible - disqualified - other_kernel
            if model.initializers[name].storage.dtype == "i4"}


@dataclass(frozen=True)
class PackedInt4:
    """One int4 weight as the device kernels take it."""
    shape: Tuple[int, ...]
    group_size: int
    packed: np.ndarray   # uint8 [numel / 2], a view of the file
    scales: np.ndarray   # float32 [shape[0], row length / group_size], a view of the file


def packed_int4(model: KarumeModel, name: str) -> PackedInt4:
    """The packed payload and scales of an int4 initializer, checked against the storage
    contract (packages/runtime/src/format/i4.ts:70-97); views, not copies."""
    init = model.initializers.get(name)
    if init is None:
        raise ContainerError(f"no initializer named '{name}'")
    if init.storage.dtype != "i4":
        raise ContainerError(f"initializer '{name}' is stored as {init.storage.dtype}, not i4")
    weight = model.file.tensors[init.tensor]
    scale = model.file.tensors[init.storage.scale]
    check_int4(weight.byte_length, init.shape, scale.shape, init.storage.group_size)
    packed = np.frombuffer(tensor_bytes(model.file, weight), dtype=np.uint8)
    scales = np.frombuffer(tensor_bytes(model.file, scale), dtype="<f4").reshape(scale.shape)
    return PackedInt4(init.shape, init.storage.group_size, packed, scales)


def build_safetensors(tensors: Sequence[Tuple[str, str, Sequence[int], bytes]],
                      metadata: Optional[Mapping[str, str]] = None) -> bytes:
    """Writer used by tests and tools: tensors in the given order, the header padded with
    spaces so that the data section starts on 8 bytes (every dtype's alignment then follows
    from the offsets the caller's order produces)."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    cursor = 0
    for name, dtype, shape, data in tensors:
        header[name] = {"dtype": dtype, "shape": list(shape),
                        "data_offsets": [cursor, cursor + len(data)]}
        cursor += len(data)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * (-(8 + len(text)) % 8)
    return struct.pack("<Q", len(text)) + text + b"".join(bytes(d) for _, _, _, d in tensors)


__all__: List[str] = [
    "ContainerError", "I4Error", "IR_METADATA_KEY", "Initializer", "IrError", "KarumeModel",
    "PackedInt4", "SafetensorsError", "SafetensorsFile", "Storage", "TensorView",
    "build_safetensors", "i4_resident_initializers", "open_model", "packed_int4",
    "parse_safetensors", "tensor_bytes",
]
