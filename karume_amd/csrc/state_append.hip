// state_append for gfx950: copies this step's K or V rows into the state slot.
//
// Follows packages/runtime/src/kernels/state-append.ts:47-96 (kernel) and :120-173 (params,
// grid): total work is kv_planes * query * depth elements (never proportional to the slot
// capacity or to `past`), destination row = slot_row(past + row) with the same ring map the
// attention kernels read through, and with query > window only the last logical row that maps
// to a physical row writes it.
#include "krm_internal.h"

using namespace krm;

namespace {

template <typename T>
__device__ inline float load_as_f32(const T* p, size_t i);
template <>
__device__ inline float load_as_f32<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ inline float load_as_f32<__half>(const __half* p, size_t i) {
  return __half2float(p[i]);
}
template <typename T>
__device__ inline void store_from_f32(T* p, size_t i, float v);
template <>
__device__ inline void store_from_f32<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ inline void store_from_f32<__half>(__half* p, size_t i, float v) {
  p[i] = __float2half_rn(v);
}

template <typename XT, typename ST>
__global__ __launch_bounds__(256) void state_append_kernel(
    const XT* __restrict__ x, ST* __restrict__ slot, uint32_t kv_planes, uint32_t chunk_rows,
    uint32_t depth, uint32_t capacity, uint32_t window, uint32_t past, uint32_t query) {
  const uint64_t total = (uint64_t)kv_planes * query * depth;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < total; i += stride) {
    const uint32_t d = (uint32_t)(i % depth);
    const uint64_t rest = i / depth;
    const uint32_t row = (uint32_t)(rest % query);
    const uint32_t plane = (uint32_t)(rest / query);
    const uint64_t logical = (uint64_t)past + row;
    const uint64_t prow = window ? logical % window : logical;
    // Ring overrun (query > window): several logical rows share a physical row; only the
    // last one writes, so the result does not depend on scheduling.
    if (window && (uint64_t)row + window < query) continue;
    const size_t src = ((size_t)plane * chunk_rows + row) * depth + d;
    const size_t dst = ((size_t)plane * capacity + prow) * depth + d;
    store_from_f32<ST>(slot, dst, load_as_f32<XT>(x, src));
  }
}

template <typename XT, typename ST>
int32_t launch(krm_ctx* ctx, krm_buf x, krm_buf slot, uint32_t kv_planes, uint32_t chunk_rows,
               uint32_t depth, uint32_t capacity, uint32_t window, uint32_t past,
               uint32_t query) {
  const uint64_t total = (uint64_t)kv_planes * query * depth;
  uint64_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  state_append_kernel<XT, ST><<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(
      ptr<const XT>(x), ptr<ST>(slot), kv_planes, chunk_rows, depth, capacity, window, past,
      query);
  return launched(ctx, "state_append_kernel");
}

}  // namespace

extern "C" {

int32_t krm_state_append(krm_ctx* ctx, krm_buf x, krm_buf slot, uint32_t kv_planes,
                         uint32_t chunk_rows, uint32_t depth, uint32_t capacity,
                         uint32_t window, uint32_t past, uint32_t query, int32_t x_dtype,
                         int32_t slot_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(x_dtype) && valid_dtype(slot_dtype),
              "krm_state_append: x_dtype %d / slot_dtype %d", x_dtype, slot_dtype);
  KRM_REQUIRE(ctx, kv_planes >= 1 && chunk_rows >= 1 && depth >= 1 && capacity >= 1,
              "krm_state_append: kv_planes / chunk_rows / depth / capacity must be positive "
              "(%u / %u / %u / %u)",
              kv_planes, chunk_rows, depth, capacity);
  KRM_REQUIRE(ctx, window <= capacity, "krm_state_append: window %u exceeds capacity %u", window,
              capacity);
  if (query < 1 || query > chunk_rows)
    return fail(ctx, KRM_ERR_EXECUTION, "krm_state_append: queryLength %u is outside 1..%u", query,
                chunk_rows);
  if (window == 0 && (uint64_t)past + query > capacity)
    return fail(ctx, KRM_ERR_EXECUTION,
                "krm_state_append: pastLength %u + queryLength %u exceeds capacity %u", past,
                query, capacity);
  KRM_REQUIRE(ctx, x && slot, "krm_state_append: NULL buffer");
  KRM_REQUIRE(ctx, aligned(x, dtype_bytes(x_dtype)) && aligned(slot, dtype_bytes(slot_dtype)),
              "krm_state_append: misaligned buffer");
  if (x_dtype == KRM_F32 && slot_dtype == KRM_F32)
    return launch<float, float>(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window,
                                past, query);
  if (x_dtype == KRM_F32 && slot_dtype == KRM_F16)
    return launch<float, __half>(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window,
                                 past, query);
  if (x_dtype == KRM_F16 && slot_dtype == KRM_F16)
    return launch<__half, __half>(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window,
                                  past, query);
  return launch<__half, float>(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window, past,
                               query);
}

}  // extern "C"
