"""karume_amd — MI355X (gfx950) backend for the Karume IR runtime's int4 ``linear``,
states-form ``attention`` and ``state_append`` ops.

The compute lives in ``lib/libkarume_hip.so`` (hand-written HIP, built by
``python -m karume_amd.build``) behind the C ABI of ``include/karume_hip.h``; this package is
the host-side mirror of the reference's interface for those ops.
"""
from .format_i4 import I4Error, check_int4, group_scale_shape, pack_int4
from .format_model import (ContainerError, IrError, KarumeModel, PackedInt4, SafetensorsError,
                           i4_resident_initializers, open_model, packed_int4,
                           parse_safetensors, tensor_bytes)
from .runtime import (COMPUTE_F16, COMPUTE_F32, EPILOGUE_NONE, EPILOGUE_SILU_PAIRS, F16, F32,
                      PROBE_EMPTY, PROBE_READ, DeviceBuffer, ExecutionError,
                      GpuContext, GpuDeviceLostError, GpuEvent, GpuGraph, GpuOutOfMemoryError,
                      GpuValidationError, KarumeError, acquire_gpu, dtype_code, version)

from .decoder_loader import GraphShapeError, decoder_weights_from_model
from .generation import (GenerationContext, GenerationContextError, PrefillChunk,
                         generate_greedy, plan_prefill_chunks)

__all__ = [
    "GenerationContext", "GenerationContextError", "PrefillChunk", "generate_greedy",
    "plan_prefill_chunks",
    "I4Error", "check_int4", "group_scale_shape", "pack_int4",
    "GraphShapeError", "decoder_weights_from_model",
    "ContainerError", "IrError", "KarumeModel", "PackedInt4", "SafetensorsError",
    "i4_resident_initializers", "open_model", "packed_int4", "parse_safetensors", "tensor_bytes",
    "COMPUTE_F16", "COMPUTE_F32", "EPILOGUE_NONE", "EPILOGUE_SILU_PAIRS", "F16", "F32",
    "PROBE_EMPTY", "PROBE_READ", "DeviceBuffer", "ExecutionError", "GpuContext",
    "GpuDeviceLostError", "GpuEvent", "GpuGraph", "GpuOutOfMemoryError", "GpuValidationError", "KarumeError",
    "acquire_gpu", "dtype_code", "version",
]
