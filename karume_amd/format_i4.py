"""Packed int4 weight format of IR v1 — host-side layout helpers (no dequantisation here).

Layout (docs/ir-v1.md:135-150, tools/exporter/src/karume/emit.py:292-322,
packages/runtime/src/format/i4.ts:44-50): codes q in [-8, 7] are stored as u = q + 8, two per
byte in flat row-major order — element 2j in the low nibble of byte j, element 2j+1 in the
high nibble; the scale tensor has shape [shape[0], (numel / shape[0]) / group_size].
Expansion to f32 is done on the device (``GpuContext.dequant_i4``).
"""
from __future__ import annotations

from typing import Sequence

import numpy as np


class I4Error(ValueError):
    """The packed payload, group size or scale shape breaks the storage contract."""


def group_scale_shape(shape: Sequence[int], group_size: int) -> list:
    """Rank-2 scale shape of an int4 tensor (packages/runtime/src/format/i4.ts:44-50)."""
    dims = [int(d) for d in shape]
    numel = int(np.prod(dims)) if dims else 1
    return [dims[0], (numel / dims[0]) / group_size]


def pack_int4(q: np.ndarray) -> np.ndarray:
    """Pack integer codes in [-8, 7] (flat row-major, even count) into bytes."""
    flat = np.ascontiguousarray(q).reshape(-1).astype(np.int16)
    if flat.size % 2 != 0:
        raise I4Error(f"an odd number of codes ({flat.size}) cannot be packed")
    if flat.size and (flat.min() < -8 or flat.max() > 7):
        raise I4Error("int4 codes must lie in [-8, 7]")
    u = (flat + 8).astype(np.uint8)
    return (u[0::2] | (u[1::2] << 4)).astype(np.uint8)


def check_int4(byte_len: int, shape: Sequence[int], scale_shape: Sequence[int],
               group_size: int) -> None:
    """Storage checks the loader performs before an int4 tensor is handed to the device
    (same rejections as packages/runtime/src/format/i4.ts:70-97)."""
    shape = [int(d) for d in shape]
    if len(shape) == 0:
        raise I4Error("a rank-0 int4 weight has no quantisation axis")
    count = int(np.prod(shape))
    if count % 2 != 0 or byte_len * 2 != count:
        raise I4Error(f"payload of {byte_len} bytes does not match shape {shape} "
                      f"({count / 2} bytes needed)")
    width = count // shape[0] if shape[0] else 0
    if not isinstance(group_size, (int, np.integer)) or group_size < 1 or width % group_size:
        raise I4Error(f"group_size {group_size} does not divide the row length {width}")
    expected = [shape[0], width // group_size]
    if list(scale_shape) != expected:
        raise I4Error(f"scale {list(scale_shape)} is not the group shape {expected} "
                      f"(group_size={group_size})")
