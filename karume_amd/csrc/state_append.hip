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
    uint32_t depth, uint32_t capacity, uint32_t window, uint32_t past, uint32_t query,
    uint32_t* lengths) {
  if (lengths) {  // run-time lengths read on the device; same checks as the scalar form
    past = lengths[0];
    query = lengths[1];
    const bool ok = query >= 1 && query <= chunk_rows &&
                    (uint64_t)past + query <= 0xffffffffull &&
                    (window != 0 || (uint64_t)past + query <= capacity);
    if (!ok) {
      if (blockIdx.x == 0 && threadIdx.x == 0) lengths[2] = 1u;
      return;
    }
  }
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


// One decode row ([q; k; v] as a fused qkv linear writes it): half-split RoPE of the q and k
// heads (same roundings as rope_kernel: two rounded products, then the add;
// packages/runtime/src/kernels/rope.ts:5-20,52-80) and the state_append of the roped k row and
// the v row (packages/runtime/src/kernels/state-append.ts:47-96) in one launch.  Appending
// before the attention of the same step is safe for a one-row step: the attention reads slot
// columns c < past only, and the row written is column `past` (full context) or the physical
// row of column past - window, which has just left the window (ring).
template <typename XT, typename ST>
__global__ __launch_bounds__(256) void decode_rope_append_kernel(
    const XT* __restrict__ qkv, const int32_t* __restrict__ positions,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table,
    XT* __restrict__ qk_out, ST* __restrict__ slot_k, ST* __restrict__ slot_v, uint32_t heads,
    uint32_t kv_heads, uint32_t depth, uint32_t table_rows, uint32_t capacity, uint32_t window,
    uint32_t past, uint32_t* lengths) {
  bool append = true;
  if (lengths) {
    past = lengths[0];
    const uint32_t query = lengths[1];
    append = query == 1 && (uint64_t)past + 1 <= 0xffffffffull &&
             (window != 0 || (uint64_t)past + 1 <= capacity);
    if (!append && blockIdx.x == 0 && threadIdx.x == 0) lengths[2] = 1u;
  }
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t total = (heads + 2 * kv_heads) * depth;
  if (i >= total) return;
  const uint32_t head = i / depth, d = i - head * depth;
  const uint64_t prow = window ? (uint64_t)past % window : (uint64_t)past;
  if (head >= heads + kv_heads) {  // v: copy into the slot
    if (append) {
      const uint32_t plane = head - heads - kv_heads;
      store_from_f32<ST>(slot_v, ((size_t)plane * capacity + prow) * depth + d,
                         load_as_f32<XT>(qkv, i));
    }
    return;
  }
  const int32_t pos = positions[0];
  const uint32_t half = depth / 2;
  float value;
  if (pos < 0 || (uint32_t)pos >= table_rows) {
    value = NAN;
  } else {
    const float self = load_as_f32<XT>(qkv, i);
    const float other = d < half ? -load_as_f32<XT>(qkv, i + half) : load_as_f32<XT>(qkv, i - half);
    const size_t t = (size_t)pos * depth + d;
    const float direct = __fmul_rn(self, cos_table[t]);
    const float cross = __fmul_rn(other, sin_table[t]);
    value = __fadd_rn(direct, cross);
  }
  store_from_f32<XT>(qk_out, i, value);
  if (head >= heads && append) {
    // the slot holds what a separate state_append would copy from the stored (rounded) k row
    const float stored = sizeof(XT) == 2 ? __half2float(__float2half_rn(value)) : value;
    store_from_f32<ST>(slot_k, ((size_t)(head - heads) * capacity + prow) * depth + d, stored);
  }
}

template <typename XT, typename ST>
int32_t launch(krm_ctx* ctx, krm_buf x, krm_buf slot, uint32_t kv_planes, uint32_t chunk_rows,
               uint32_t depth, uint32_t capacity, uint32_t window, uint32_t past,
               uint32_t query, krm_buf lengths) {
  const uint64_t total = (uint64_t)kv_planes * query * depth;
  uint64_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  state_append_kernel<XT, ST><<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(
      ptr<const XT>(x), ptr<ST>(slot), kv_planes, chunk_rows, depth, capacity, window, past,
      query, ptr<uint32_t>(lengths));
  return launched(ctx, "state_append_kernel");
}

}  // namespace

// `lengths` == 0: past / query are this run's values; otherwise they are read on the device
// and `query` only sizes the launch (the chunk's physical rows).
static int32_t state_append_impl(krm_ctx* ctx, krm_buf x, krm_buf slot, uint32_t kv_planes,
                                 uint32_t chunk_rows, uint32_t depth, uint32_t capacity,
                                 uint32_t window, uint32_t past, uint32_t query, krm_buf lengths,
                                 int32_t x_dtype, int32_t slot_dtype) {
  KRM_TRY(enter(ctx));
  const bool dyn = lengths != 0;
  KRM_REQUIRE(ctx, valid_dtype(x_dtype) && valid_dtype(slot_dtype),
              "krm_state_append: x_dtype %d / slot_dtype %d", x_dtype, slot_dtype);
  KRM_REQUIRE(ctx, kv_planes >= 1 && chunk_rows >= 1 && depth >= 1 && capacity >= 1,
              "krm_state_append: kv_planes / chunk_rows / depth / capacity must be positive "
              "(%u / %u / %u / %u)",
              kv_planes, chunk_rows, depth, capacity);
  KRM_REQUIRE(ctx, window <= capacity, "krm_state_append: window %u exceeds capacity %u", window,
              capacity);
  if (!dyn && (query < 1 || query > chunk_rows))
    return fail(ctx, KRM_ERR_EXECUTION, "krm_state_append: queryLength %u is outside 1..%u", query,
                chunk_rows);
  if (!dyn && window == 0 && (uint64_t)past + query > capacity)
    return fail(ctx, KRM_ERR_EXECUTION,
                "krm_state_append: pastLength %u + queryLength %u exceeds capacity %u", past,
                query, capacity);
  KRM_REQUIRE(ctx, x && slot, "krm_state_append: NULL buffer");
  KRM_REQUIRE(ctx, aligned(x, dtype_bytes(x_dtype)) && aligned(slot, dtype_bytes(slot_dtype)),
              "krm_state_append: misaligned buffer");
  if (x_dtype == KRM_F32 && slot_dtype == KRM_F32)
    return launch<float, float>(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window,
                                past, query, lengths);
  if (x_dtype == KRM_F32 && slot_dtype == KRM_F16)
    return launch<float, __half>(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window,
                                 past, query, lengths);
  if (x_dtype == KRM_F16 && slot_dtype == KRM_F16)
    return launch<__half, __half>(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window,
                                  past, query, lengths);
  return launch<__half, float>(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window, past,
                               query, lengths);
}

template <typename XT, typename ST>
static int32_t launch_rope_append(krm_ctx* ctx, krm_buf qkv, krm_buf positions, krm_buf cos_table,
                                  krm_buf sin_table, krm_buf qk_out, krm_buf slot_k,
                                  krm_buf slot_v, uint32_t heads, uint32_t kv_heads,
                                  uint32_t depth, uint32_t table_rows, uint32_t capacity,
                                  uint32_t window, uint32_t past, krm_buf lengths) {
  const uint32_t total = (heads + 2 * kv_heads) * depth;
  decode_rope_append_kernel<XT, ST><<<dim3((total + 255) / 256), dim3(256), 0, ctx->stream>>>(
      ptr<const XT>(qkv), ptr<const int32_t>(positions), ptr<const float>(cos_table),
      ptr<const float>(sin_table), ptr<XT>(qk_out), ptr<ST>(slot_k), ptr<ST>(slot_v), heads,
      kv_heads, depth, table_rows, capacity, window, past, ptr<uint32_t>(lengths));
  return launched(ctx, "decode_rope_append_kernel");
}

extern "C" int32_t krm_decode_rope_append(krm_ctx* ctx, krm_buf qkv, krm_buf positions_i32,
                                          krm_buf cos_table_f32, krm_buf sin_table_f32,
                                          krm_buf qk_out, krm_buf slot_k, krm_buf slot_v,
                                          uint32_t heads, uint32_t kv_heads, uint32_t depth,
                                          uint32_t table_rows, uint32_t capacity, uint32_t window,
                                          uint32_t past, krm_buf lengths, int32_t io_dtype,
                                          int32_t kv_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(kv_dtype),
              "krm_decode_rope_append: io_dtype %d / kv_dtype %d", io_dtype, kv_dtype);
  KRM_REQUIRE(ctx, heads >= 1 && kv_heads >= 1 && depth >= 2 && depth % 2 == 0 && capacity >= 1 &&
                       table_rows >= 1,
              "krm_decode_rope_append: H / Hkv / D / C / table rows (%u / %u / %u / %u / %u)",
              heads, kv_heads, depth, capacity, table_rows);
  KRM_REQUIRE(ctx, ((uint64_t)heads + 2ull * kv_heads) * depth <= 0x7fffffffull,
              "krm_decode_rope_append: the row is too long");
  KRM_REQUIRE(ctx, window <= capacity, "krm_decode_rope_append: window %u exceeds capacity %u",
              window, capacity);
  if (!lengths && window == 0 && (uint64_t)past + 1 > capacity)
    return fail(ctx, KRM_ERR_EXECUTION,
                "krm_decode_rope_append: pastLength %u + queryLength 1 exceeds capacity %u", past,
                capacity);
  KRM_REQUIRE(ctx, qkv && positions_i32 && cos_table_f32 && sin_table_f32 && qk_out && slot_k &&
                       slot_v,
              "krm_decode_rope_append: NULL buffer");
  const size_t io_b = dtype_bytes(io_dtype), kv_b = dtype_bytes(kv_dtype);
  KRM_REQUIRE(ctx,
              aligned(qkv, io_b) && aligned(qk_out, io_b) && aligned(slot_k, kv_b) &&
                  aligned(slot_v, kv_b) && aligned(positions_i32, 4) &&
                  aligned(cos_table_f32, 4) && aligned(sin_table_f32, 4) && aligned(lengths, 4),
              "krm_decode_rope_append: misaligned buffer");
#define KRM_ROPE_APPEND(XT, ST)                                                              \
  return launch_rope_append<XT, ST>(ctx, qkv, positions_i32, cos_table_f32, sin_table_f32,   \
                                    qk_out, slot_k, slot_v, heads, kv_heads, depth,          \
                                    table_rows, capacity, window, past, lengths)
  if (io_dtype == KRM_F32 && kv_dtype == KRM_F32) KRM_ROPE_APPEND(float, float);
  if (io_dtype == KRM_F32 && kv_dtype == KRM_F16) KRM_ROPE_APPEND(float, __half);
  if (io_dtype == KRM_F16 && kv_dtype == KRM_F16) KRM_ROPE_APPEND(__half, __half);
  KRM_ROPE_APPEND(__half, float);
#undef KRM_ROPE_APPEND
}

// Run-time lengths {past, query, fault} kept in device memory so a recorded step can be
// replayed while the sequence grows (the reference keeps them in an 8-byte uniform owned by
// the generation context, packages/runtime/src/runtime/generation-context.ts:559-566).
__global__ void lengths_set_kernel(uint32_t* lengths, uint32_t past, uint32_t query) {
  lengths[0] = past;
  lengths[1] = query;
  lengths[2] = 0u;
  lengths[3] = 0u;
}
__global__ void lengths_advance_kernel(uint32_t* lengths) {
  // P advances by Q only when the step ran clean (generation-context.ts:576-591)
  if (lengths[2] == 0u) lengths[0] += lengths[1];
}
__global__ void lengths_positions_kernel(const uint32_t* lengths, int32_t* positions,
                                         uint32_t rows) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < rows) positions[i] = (int32_t)(lengths[0] + i);
}

__global__ void lengths_log_token_kernel(uint32_t* lengths, const int32_t* token,
                                         int32_t* history, uint32_t history_len) {
  const uint32_t at = lengths[3];
  if (at < history_len) history[at] = token[0];
  lengths[3] = at + 1;
}

// End of a one-row decode step in one launch: the three kernels above in their order.
__global__ void lengths_step_end_kernel(uint32_t* lengths, const int32_t* token, int32_t* history,
                                        uint32_t history_len, int32_t* positions) {
  const uint32_t at = lengths[3];
  if (at < history_len) history[at] = token[0];
  lengths[3] = at + 1;
  uint32_t past = lengths[0];
  if (lengths[2] == 0u) {
    past += lengths[1];
    lengths[0] = past;
  }
  positions[0] = (int32_t)past;
}

extern "C" {

int32_t krm_lengths_step_end(krm_ctx* ctx, krm_buf lengths, krm_buf token_i32,
                             krm_buf history_i32, uint32_t history_len, krm_buf positions_i32) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, lengths && token_i32 && history_i32 && positions_i32 && lengths % 4 == 0 &&
                       token_i32 % 4 == 0 && history_i32 % 4 == 0 && positions_i32 % 4 == 0,
              "krm_lengths_step_end: bad buffer");
  lengths_step_end_kernel<<<dim3(1), dim3(1), 0, ctx->stream>>>(
      ptr<uint32_t>(lengths), ptr<const int32_t>(token_i32), ptr<int32_t>(history_i32),
      history_len, ptr<int32_t>(positions_i32));
  return launched(ctx, "lengths_step_end_kernel");
}

int32_t krm_lengths_log_token(krm_ctx* ctx, krm_buf lengths, krm_buf token_i32,
                              krm_buf history_i32, uint32_t history_len) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, lengths && token_i32 && history_i32 && lengths % 4 == 0 &&
                       token_i32 % 4 == 0 && history_i32 % 4 == 0,
              "krm_lengths_log_token: bad buffer");
  lengths_log_token_kernel<<<dim3(1), dim3(1), 0, ctx->stream>>>(
      ptr<uint32_t>(lengths), ptr<const int32_t>(token_i32), ptr<int32_t>(history_i32),
      history_len);
  return launched(ctx, "lengths_log_token_kernel");
}

int32_t krm_state_append(krm_ctx* ctx, krm_buf x, krm_buf slot, uint32_t kv_planes,
                         uint32_t chunk_rows, uint32_t depth, uint32_t capacity,
                         uint32_t window, uint32_t past, uint32_t query, int32_t x_dtype,
                         int32_t slot_dtype) {
  return state_append_impl(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window, past,
                           query, 0, x_dtype, slot_dtype);
}

int32_t krm_state_append_lengths(krm_ctx* ctx, krm_buf x, krm_buf slot, uint32_t kv_planes,
                                 uint32_t chunk_rows, uint32_t depth, uint32_t capacity,
                                 uint32_t window, krm_buf lengths, int32_t x_dtype,
                                 int32_t slot_dtype) {
  if (!lengths || lengths % 4)
    return fail(ctx, KRM_ERR_VALIDATION, "krm_state_append_lengths: bad lengths buffer");
  return state_append_impl(ctx, x, slot, kv_planes, chunk_rows, depth, capacity, window, 0,
                           chunk_rows, lengths, x_dtype, slot_dtype);
}

int32_t krm_lengths_set(krm_ctx* ctx, krm_buf lengths, uint32_t past, uint32_t query) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, lengths && lengths % 4 == 0, "krm_lengths_set: bad lengths buffer");
  lengths_set_kernel<<<dim3(1), dim3(1), 0, ctx->stream>>>(ptr<uint32_t>(lengths), past, query);
  return launched(ctx, "lengths_set_kernel");
}

int32_t krm_lengths_advance(krm_ctx* ctx, krm_buf lengths) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, lengths && lengths % 4 == 0, "krm_lengths_advance: bad lengths buffer");
  lengths_advance_kernel<<<dim3(1), dim3(1), 0, ctx->stream>>>(ptr<uint32_t>(lengths));
  return launched(ctx, "lengths_advance_kernel");
}

int32_t krm_lengths_positions(krm_ctx* ctx, krm_buf lengths, krm_buf positions_i32,
                              uint32_t rows) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, lengths && positions_i32 && lengths % 4 == 0 && positions_i32 % 4 == 0,
              "krm_lengths_positions: bad buffer");
  if (rows == 0) return KRM_OK;
  lengths_positions_kernel<<<dim3((rows + 63) / 64), dim3(64), 0, ctx->stream>>>(
      ptr<const uint32_t>(lengths), ptr<int32_t>(positions_i32), rows);
  return launched(ctx, "lengths_positions_kernel");
}

}  // extern "C"
