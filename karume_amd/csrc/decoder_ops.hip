// The small ops a Llama-style decoder layer runs between the linears and the attention:
// rms_norm, half-split RoPE with a position table, SiLU-gate, residual add, embedding gather,
// argmax and the [rows, heads, D] <-> [heads, rows, D] transposition.  Each follows the
// reference kernel of the same name (cited per kernel); activations may be f32 or fp16,
// arithmetic is f32.
#include "krm_internal.h"

#include <cmath>

using namespace krm;

namespace {

constexpr int kThreads = 256;

template <typename T>
__device__ inline float ld(const T* p, size_t i);
template <>
__device__ inline float ld<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ inline float ld<__half>(const __half* p, size_t i) { return __half2float(p[i]); }
template <typename T>
__device__ inline void st(T* p, size_t i, float v);
template <>
__device__ inline void st<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ inline void st<__half>(__half* p, size_t i, float v) { p[i] = __float2half_rn(v); }

__device__ inline float block_sum(float v, float* scratch) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < kThreads / kWave; ++w) total += scratch[w];
  __syncthreads();
  return total;
}

// rms_norm: out = x * rsqrt(mean(x^2) + eps) * weight, one workgroup per row.
// packages/runtime/src/kernels/rms-norm.ts:35-91 (no mean subtraction; weight is f32).
// OT: the type the result is stored in (XT, or fp16 beside f32 rows: a copy for a consumer
// that would round the f32 result to fp16 anyway).
template <typename XT, typename OT = XT>
__global__ __launch_bounds__(kThreads) void rms_norm_kernel(const XT* __restrict__ x,
                                                           const float* __restrict__ weight,
                                                           OT* __restrict__ out, uint32_t dim,
                                                           float eps) {
  __shared__ float scratch[kThreads / kWave];
  const size_t base = (size_t)blockIdx.x * dim;
  // the fp16 copy of an f32 row is the f32 result rounded again, never a product rounded once
  auto keep_f32 = [](float v) { return sizeof(OT) == sizeof(XT) ? v : rounded_f32(v); };
  constexpr int kKeep = 16;  // rows up to 4096 elements stay in registers: one trip to memory
  if (dim <= (uint32_t)(kThreads * kKeep)) {
    float v[kKeep], wv[kKeep];
#pragma unroll
    for (int j = 0; j < kKeep; ++j) {
      const uint32_t i = threadIdx.x + j * kThreads;
      v[j] = i < dim ? ld<XT>(x, base + i) : 0.f;
      wv[j] = i < dim ? weight[i] : 0.f;
    }
    float squares = 0.f;  // the same elements in the same order as the loop below
#pragma unroll
    for (int j = 0; j < kKeep; ++j)
      if (threadIdx.x + j * kThreads < dim) squares = fmaf(v[j], v[j], squares);
    const float total = block_sum(squares, scratch);
    const float inv = 1.0f / sqrtf(total / (float)dim + eps);
#pragma unroll
    for (int j = 0; j < kKeep; ++j) {
      const uint32_t i = threadIdx.x + j * kThreads;
      if (i < dim) st<OT>(out, base + i, keep_f32(v[j] * inv * wv[j]));
    }
    return;
  }
  float squares = 0.f;
  for (uint32_t i = threadIdx.x; i < dim; i += kThreads) {
    const float v = ld<XT>(x, base + i);
    squares = fmaf(v, v, squares);
  }
  const float total = block_sum(squares, scratch);
  const float inv = 1.0f / sqrtf(total / (float)dim + eps);
  for (uint32_t i = threadIdx.x; i < dim; i += kThreads)
    st<OT>(out, base + i, keep_f32(ld<XT>(x, base + i) * inv * weight[i]));
}

// Half-split RoPE with the cos / sin rows looked up by absolute position:
//   out = x*cos[pos] + rotate_half(x)*sin[pos],  rotate_half(x) = cat(-x[D/2:], x[:D/2]).
// Both products are rounded before the add, as in the reference's fused kernel
// (packages/runtime/src/kernels/rope.ts:5-20,52-80); the table lookup is the decode graph's
// embedding(position_ids, table) (tools/export-recipes/minicpm5/export_decode.py:24-35).
// `x` is [rows, heads, D] (the layout a linear writes); `out` is [heads, rows, D] (the layout
// the attention reads) when to_head_major is set, otherwise the same layout as `x`.
template <typename XT>
__global__ __launch_bounds__(kThreads) void rope_kernel(
    const XT* __restrict__ x, const int32_t* __restrict__ positions,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table,
    XT* __restrict__ out, uint32_t rows, uint32_t heads, uint32_t head_dim,
    uint32_t table_rows, uint32_t to_head_major) {
  const size_t total = (size_t)rows * heads * head_dim;
  const uint32_t half = head_dim / 2;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += stride) {
    const uint32_t d = (uint32_t)(i % head_dim);
    const size_t rest = i / head_dim;
    const uint32_t head = (uint32_t)(rest % heads);
    const uint32_t row = (uint32_t)(rest / heads);
    const int32_t pos = positions[row];
    const size_t row_base = i - d;
    float value;
    if (pos < 0 || (uint32_t)pos >= table_rows) {
      value = NAN;  // a position outside the table must not look like a valid rotation
    } else {
      const float self = ld<XT>(x, i);
      const float other = d < half ? -ld<XT>(x, row_base + d + half) : ld<XT>(x, row_base + d - half);
      const size_t t = (size_t)pos * head_dim + d;
      const float direct = __fmul_rn(self, cos_table[t]);
      const float cross = __fmul_rn(other, sin_table[t]);
      value = __fadd_rn(direct, cross);
    }
    const size_t dst = to_head_major ? ((size_t)head * rows + row) * head_dim + d : i;
    st<XT>(out, dst, value);
  }
}

// [a, b, d] -> [b, a, d]
template <typename XT>
__global__ __launch_bounds__(kThreads) void transpose_kernel(const XT* __restrict__ x,
                                                            XT* __restrict__ out, uint32_t a,
                                                            uint32_t b, uint32_t d) {
  const size_t total = (size_t)a * b * d;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += stride) {
    const uint32_t e = (uint32_t)(i % d);
    const size_t rest = i / d;
    const uint32_t bi = (uint32_t)(rest % b);
    const uint32_t ai = (uint32_t)(rest / b);
    out[((size_t)bi * a + ai) * d + e] = x[i];
  }
}

// silu(gate) * up with the reference's roundings: s = sigmoid_stable(gate) is rounded, then
// gate*s, then *up (packages/runtime/src/kernels/silu.ts:47-93,
// packages/runtime/src/codegen/elementwise.ts:187-190).
__device__ inline float sigmoid_stable(float v) {
  const float t = expf(-fabsf(v));
  return v < 0.f ? t / (1.0f + t) : 1.0f / (1.0f + t);
}
template <typename XT>
__global__ __launch_bounds__(kThreads) void silu_mul_kernel(const XT* __restrict__ gate,
                                                           const XT* __restrict__ up,
                                                           XT* __restrict__ out, size_t count) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < count; i += stride) {
    const float g = ld<XT>(gate, i);
    const float act = __fmul_rn(g, sigmoid_stable(g));
    st<XT>(out, i, __fmul_rn(act, ld<XT>(up, i)));
  }
}

// elementwise add (the residual connections).  packages/runtime/src/codegen/elementwise.ts
template <typename XT>
__global__ __launch_bounds__(kThreads) void add_kernel(const XT* __restrict__ a,
                                                      const XT* __restrict__ b,
                                                      XT* __restrict__ out, size_t count) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < count; i += stride)
    st<XT>(out, i, __fadd_rn(ld<XT>(a, i), ld<XT>(b, i)));
}

// embedding row gather; an index outside [0, vocab) writes NaN to that row, it is never
// clamped (packages/runtime/src/kernels/embedding.ts:1-43).
template <typename WT, typename XT>
__global__ __launch_bounds__(kThreads) void embedding_kernel(const WT* __restrict__ table,
                                                            const int32_t* __restrict__ index,
                                                            XT* __restrict__ out, uint32_t rows,
                                                            uint32_t vocab, uint32_t hidden) {
  const size_t total = (size_t)rows * hidden;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += stride) {
    const uint32_t col = (uint32_t)(i % hidden);
    const int32_t pick = index[i / hidden];
    const float v = (pick < 0 || (uint32_t)pick >= vocab) ? NAN
                                                          : ld<WT>(table, (size_t)pick * hidden + col);
    st<XT>(out, i, v);
  }
}

// argmax over the last dim: ties -> smallest index, NaN counts as the maximum, a row of -inf
// gives 0 (packages/runtime/src/kernels/argmax.ts:16-34).  (value, index) pairs are ordered
// lexicographically (value descending, index ascending), so the tree shape does not matter.
__device__ inline bool beats(float va, uint32_t ia, float vb, uint32_t ib) {
  return argmax_beats(va, ia, vb, ib);
}
constexpr int kArgmaxThreads = 1024;
constexpr int kArgmaxUnroll = 32;  // independent loads in flight per thread (one pass up to 32768)
template <typename XT>
__global__ __launch_bounds__(kArgmaxThreads) void argmax_kernel(const XT* __restrict__ x,
                                                               int32_t* __restrict__ out,
                                                               uint32_t dim) {
  __shared__ float s_val[kArgmaxThreads / kWave];
  __shared__ uint32_t s_idx[kArgmaxThreads / kWave];
  const size_t base = (size_t)blockIdx.x * dim;
  float best = -INFINITY;
  uint32_t at = dim;  // sentinel: any real element beats it on the index comparison
  // f32 rows of whole 16-byte pieces: four elements a load (a quarter of the load instructions —
  // one workgroup's vector-memory path is what a 128 KB row costs)
  if constexpr (sizeof(XT) == 4) {
    if ((dim & 3u) == 0 && (((uintptr_t)(x + base)) & 15u) == 0) {
      const uint32_t pieces = dim >> 2;
      const float4* src = reinterpret_cast<const float4*>(x + base);
      constexpr int kWide = 8;
      for (uint32_t p0 = threadIdx.x; p0 < pieces; p0 += kArgmaxThreads * kWide) {
        float4 v[kWide];
#pragma unroll
        for (int u = 0; u < kWide; ++u) {
          const uint32_t p = p0 + u * kArgmaxThreads;
          v[u] = src[p < pieces ? p : p0];
        }
#pragma unroll
        for (int u = 0; u < kWide; ++u) {
          const uint32_t p = p0 + u * kArgmaxThreads;
          if (p < pieces) {
            const float e[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (beats(e[j], 4 * p + j, best, at)) {
                best = e[j];
                at = 4 * p + j;
              }
          }
        }
      }
      dim = 0;  // the scalar walk below has nothing left
    }
  }
  for (uint32_t i0 = threadIdx.x; i0 < dim; i0 += kArgmaxThreads * kArgmaxUnroll) {
    float v[kArgmaxUnroll];
#pragma unroll
    for (int u = 0; u < kArgmaxUnroll; ++u) {
      const uint32_t i = i0 + u * kArgmaxThreads;
      v[u] = ld<XT>(x, base + (i < dim ? i : i0));  // past the end: re-read, never wins (index)
    }
#pragma unroll
    for (int u = 0; u < kArgmaxUnroll; ++u) {
      const uint32_t i = i0 + u * kArgmaxThreads;
      if (i < dim && beats(v[u], i, best, at)) {
        best = v[u];
        at = i;
      }
    }
  }
  // Any tree gives the same pair.  Inside a 16-lane row the partners come through DPP (lane ^ 1,
  // lane ^ 2, rotations by 4 and 8), the rows 16 and 32 lanes apart through the LDS crossbar.
  auto take = [&](float ov, uint32_t oi) {
    if (beats(ov, oi, best, at)) {
      best = ov;
      at = oi;
    }
  };
  auto fold_row = [&]() {
#define KRM_ARGMAX_DPP(CTRL)                                                                      \
  take(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, best),   \
                                                            CTRL, 0xf, 0xf, true)),              \
       (uint32_t)__builtin_amdgcn_update_dpp(0, (int)at, CTRL, 0xf, 0xf, true))
    KRM_ARGMAX_DPP(0xB1);   // quad_perm [1,0,3,2]
    KRM_ARGMAX_DPP(0x4E);   // quad_perm [2,3,0,1]
    KRM_ARGMAX_DPP(0x124);  // row_ror:4
    KRM_ARGMAX_DPP(0x128);  // row_ror:8
#undef KRM_ARGMAX_DPP
  };
  fold_row();
  for (int off = 16; off <= 32; off <<= 1)
    take(__shfl_xor(best, off, kWave), (uint32_t)__shfl_xor((int)at, off, kWave));
  if ((threadIdx.x & 63) == 0) {
    s_val[threadIdx.x >> 6] = best;
    s_idx[threadIdx.x >> 6] = at;
  }
  __syncthreads();
  if (threadIdx.x < kWave) {  // the 16 wave results, one per lane of the first row
    static_assert(kArgmaxThreads / kWave == 16, "one 16-lane row holds the wave results");
    const int w = threadIdx.x & 15;
    best = s_val[w];
    at = s_idx[w];
    fold_row();
    if (threadIdx.x == 0) out[blockIdx.x] = (int32_t)at;
  }
}

// End of a one-row decode step in one launch: the argmax over the per-workgroup partials the
// head projection left (krm_decode_head), the step's bookkeeping (what lengths_step_end_kernel
// does: token logged, lengths advanced when the step ran clean, the next position written) and
// the next step's embedding row.  One workgroup; the partials are a few thousand pairs.
template <typename WT, typename XT>
__global__ __launch_bounds__(kArgmaxThreads) void decode_tail_kernel(
    const uint2* __restrict__ partials, uint32_t count, int32_t* __restrict__ token,
    uint32_t* __restrict__ lengths, int32_t* __restrict__ history, uint32_t history_len,
    int32_t* __restrict__ positions, const WT* __restrict__ table, uint32_t vocab,
    uint32_t hidden, XT* __restrict__ next_row) {
  __shared__ float s_val[kArgmaxThreads / kWave];
  __shared__ uint32_t s_idx[kArgmaxThreads / kWave];
  __shared__ uint32_t s_token;
  // the bookkeeping words are requested now, beside the partials, not after the reduction
  const uint32_t len_past = lengths[0], len_query = lengths[1], len_fault = lengths[2],
                 len_slot = lengths[3];
  float best = -INFINITY;
  uint32_t at = 0xffffffffu;
  constexpr int kWide = 8;
  for (uint32_t p0 = threadIdx.x; p0 < count; p0 += kArgmaxThreads * kWide) {
    uint2 v[kWide];
#pragma unroll
    for (int u = 0; u < kWide; ++u) {
      const uint32_t p = p0 + u * kArgmaxThreads;
      v[u] = partials[p < count ? p : p0];
    }
#pragma unroll
    for (int u = 0; u < kWide; ++u) {
      const uint32_t p = p0 + u * kArgmaxThreads;
      if (p < count && beats(__uint_as_float(v[u].x), v[u].y, best, at)) {
        best = __uint_as_float(v[u].x);
        at = v[u].y;
      }
    }
  }
  auto take = [&](float ov, uint32_t oi) {
    if (beats(ov, oi, best, at)) {
      best = ov;
      at = oi;
    }
  };
  auto fold_row = [&]() {
#define KRM_ARGMAX_DPP(CTRL)                                                                      \
  take(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, best),   \
                                                            CTRL, 0xf, 0xf, true)),              \
       (uint32_t)__builtin_amdgcn_update_dpp(0, (int)at, CTRL, 0xf, 0xf, true))
    KRM_ARGMAX_DPP(0xB1);
    KRM_ARGMAX_DPP(0x4E);
    KRM_ARGMAX_DPP(0x124);
    KRM_ARGMAX_DPP(0x128);
#undef KRM_ARGMAX_DPP
  };
  fold_row();
  for (int off = 16; off <= 32; off <<= 1)
    take(__shfl_xor(best, off, kWave), (uint32_t)__shfl_xor((int)at, off, kWave));
  if ((threadIdx.x & 63) == 0) {
    s_val[threadIdx.x >> 6] = best;
    s_idx[threadIdx.x >> 6] = at;
  }
  __syncthreads();
  if (threadIdx.x < kWave) {
    const int w = threadIdx.x & 15;
    best = s_val[w];
    at = s_idx[w];
    fold_row();
    if (threadIdx.x == 0) {
      // a row of -inf: every pair ties on the value and the smallest row index wins, which is
      // 0 as in argmax_kernel; no partial at all (count == 0) cannot happen (n >= 1)
      const int32_t tok = (int32_t)at;
      token[0] = tok;
      s_token = at;
      if (len_slot < history_len) history[len_slot] = tok;
      lengths[3] = len_slot + 1;
      uint32_t past = len_past;
      if (len_fault == 0u) {  // P advances by Q only when the step ran clean
        past += len_query;
        lengths[0] = past;
      }
      positions[0] = (int32_t)past;
    }
  }
  __syncthreads();
  const uint32_t pick = s_token;
  for (uint32_t col = threadIdx.x; col < hidden; col += kArgmaxThreads) {
    const float v = pick >= vocab ? NAN : ld<WT>(table, (size_t)pick * hidden + col);
    st<XT>(next_row, col, v);
  }
}

inline unsigned grid_for(size_t total) {
  size_t blocks = (total + kThreads - 1) / kThreads;
  if (blocks > 4096) blocks = 4096;
  return (unsigned)(blocks ? blocks : 1);
}

}  // namespace

#define KRM_IO_DISPATCH(io_dtype, CALL_F32, CALL_F16) \
  do {                                                \
    if ((io_dtype) == KRM_F32) {                      \
      CALL_F32;                                       \
    } else {                                          \
      CALL_F16;                                       \
    }                                                 \
  } while (0)

extern "C" {

int32_t krm_rms_norm(krm_ctx* ctx, krm_buf x, krm_buf weight_f32, krm_buf out, uint32_t rows,
                     uint32_t dim, float eps, int32_t io_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype), "krm_rms_norm: io_dtype %d", io_dtype);
  KRM_REQUIRE(ctx, dim >= 1 && std::isfinite(eps), "krm_rms_norm: dim %u / eps", dim);
  if (rows == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && weight_f32 && out, "krm_rms_norm: NULL buffer");
  KRM_IO_DISPATCH(io_dtype,
                  (rms_norm_kernel<float><<<dim3(rows), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const float>(x), ptr<const float>(weight_f32), ptr<float>(out), dim, eps)),
                  (rms_norm_kernel<__half><<<dim3(rows), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const __half>(x), ptr<const float>(weight_f32), ptr<__half>(out), dim,
                      eps)));
  return launched(ctx, "rms_norm_kernel");
}

int32_t krm_rms_norm_cast(krm_ctx* ctx, krm_buf x, krm_buf weight_f32, krm_buf out, uint32_t rows,
                          uint32_t dim, float eps, int32_t io_dtype, int32_t out_dtype) {
  if (out_dtype == io_dtype) return krm_rms_norm(ctx, x, weight_f32, out, rows, dim, eps, io_dtype);
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, io_dtype == KRM_F32 && out_dtype == KRM_F16,
              "krm_rms_norm_cast: io_dtype %d -> out_dtype %d (f32 -> fp16, or the same type)",
              io_dtype, out_dtype);
  KRM_REQUIRE(ctx, dim >= 1 && std::isfinite(eps), "krm_rms_norm_cast: dim %u / eps", dim);
  if (rows == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && weight_f32 && out, "krm_rms_norm_cast: NULL buffer");
  rms_norm_kernel<float, __half><<<dim3(rows), dim3(kThreads), 0, ctx->stream>>>(
      ptr<const float>(x), ptr<const float>(weight_f32), ptr<__half>(out), dim, eps);
  return launched(ctx, "rms_norm_kernel");
}

int32_t krm_rope_half(krm_ctx* ctx, krm_buf x, krm_buf positions_i32, krm_buf cos_table_f32,
                      krm_buf sin_table_f32, krm_buf out, uint32_t rows, uint32_t heads,
                      uint32_t head_dim, uint32_t table_rows, int32_t to_head_major,
                      int32_t io_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype), "krm_rope_half: io_dtype %d", io_dtype);
  KRM_REQUIRE(ctx, head_dim >= 2 && head_dim % 2 == 0, "krm_rope_half: head_dim %u is odd",
              head_dim);
  if (rows == 0 || heads == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && positions_i32 && cos_table_f32 && sin_table_f32 && out,
              "krm_rope_half: NULL buffer");
  KRM_REQUIRE(ctx, !(to_head_major && x == out && rows > 1 && heads > 1),
              "krm_rope_half: the transposing form cannot run in place");
  const size_t total = (size_t)rows * heads * head_dim;
  KRM_IO_DISPATCH(io_dtype,
                  (rope_kernel<float><<<dim3(grid_for(total)), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const float>(x), ptr<const int32_t>(positions_i32),
                      ptr<const float>(cos_table_f32), ptr<const float>(sin_table_f32),
                      ptr<float>(out), rows, heads, head_dim, table_rows, (uint32_t)to_head_major)),
                  (rope_kernel<__half><<<dim3(grid_for(total)), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const __half>(x), ptr<const int32_t>(positions_i32),
                      ptr<const float>(cos_table_f32), ptr<const float>(sin_table_f32),
                      ptr<__half>(out), rows, heads, head_dim, table_rows,
                      (uint32_t)to_head_major)));
  return launched(ctx, "rope_kernel");
}

int32_t krm_transpose_01(krm_ctx* ctx, krm_buf x, krm_buf out, uint32_t a, uint32_t b, uint32_t d,
                         int32_t io_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype), "krm_transpose_01: io_dtype %d", io_dtype);
  const size_t total = (size_t)a * b * d;
  if (total == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && out && x != out, "krm_transpose_01: NULL or aliased buffer");
  KRM_IO_DISPATCH(io_dtype,
                  (transpose_kernel<float><<<dim3(grid_for(total)), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const float>(x), ptr<float>(out), a, b, d)),
                  (transpose_kernel<__half><<<dim3(grid_for(total)), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const __half>(x), ptr<__half>(out), a, b, d)));
  return launched(ctx, "transpose_kernel");
}

int32_t krm_silu_mul(krm_ctx* ctx, krm_buf gate, krm_buf up, krm_buf out, uint64_t count,
                     int32_t io_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype), "krm_silu_mul: io_dtype %d", io_dtype);
  if (count == 0) return KRM_OK;
  KRM_REQUIRE(ctx, gate && up && out, "krm_silu_mul: NULL buffer");
  KRM_IO_DISPATCH(io_dtype,
                  (silu_mul_kernel<float><<<dim3(grid_for(count)), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const float>(gate), ptr<const float>(up), ptr<float>(out), count)),
                  (silu_mul_kernel<__half><<<dim3(grid_for(count)), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const __half>(gate), ptr<const __half>(up), ptr<__half>(out), count)));
  return launched(ctx, "silu_mul_kernel");
}

int32_t krm_add(krm_ctx* ctx, krm_buf a, krm_buf b, krm_buf out, uint64_t count,
                int32_t io_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype), "krm_add: io_dtype %d", io_dtype);
  if (count == 0) return KRM_OK;
  KRM_REQUIRE(ctx, a && b && out, "krm_add: NULL buffer");
  KRM_IO_DISPATCH(io_dtype,
                  (add_kernel<float><<<dim3(grid_for(count)), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const float>(a), ptr<const float>(b), ptr<float>(out), count)),
                  (add_kernel<__half><<<dim3(grid_for(count)), dim3(kThreads), 0, ctx->stream>>>(
                      ptr<const __half>(a), ptr<const __half>(b), ptr<__half>(out), count)));
  return launched(ctx, "add_kernel");
}

int32_t krm_embedding(krm_ctx* ctx, krm_buf table, krm_buf index_i32, krm_buf out, uint32_t rows,
                      uint32_t vocab, uint32_t hidden, int32_t table_dtype, int32_t out_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(table_dtype) && valid_dtype(out_dtype),
              "krm_embedding: table_dtype %d / out_dtype %d", table_dtype, out_dtype);
  KRM_REQUIRE(ctx, vocab >= 1 && hidden >= 1, "krm_embedding: vocab %u / hidden %u", vocab, hidden);
  if (rows == 0) return KRM_OK;
  KRM_REQUIRE(ctx, table && index_i32 && out, "krm_embedding: NULL buffer");
  const size_t total = (size_t)rows * hidden;
  const dim3 grid(grid_for(total)), block(kThreads);
  if (table_dtype == KRM_F16 && out_dtype == KRM_F16)
    embedding_kernel<__half, __half><<<grid, block, 0, ctx->stream>>>(
        ptr<const __half>(table), ptr<const int32_t>(index_i32), ptr<__half>(out), rows, vocab, hidden);
  else if (table_dtype == KRM_F16)
    embedding_kernel<__half, float><<<grid, block, 0, ctx->stream>>>(
        ptr<const __half>(table), ptr<const int32_t>(index_i32), ptr<float>(out), rows, vocab, hidden);
  else if (out_dtype == KRM_F16)
    embedding_kernel<float, __half><<<grid, block, 0, ctx->stream>>>(
        ptr<const float>(table), ptr<const int32_t>(index_i32), ptr<__half>(out), rows, vocab, hidden);
  else
    embedding_kernel<float, float><<<grid, block, 0, ctx->stream>>>(
        ptr<const float>(table), ptr<const int32_t>(index_i32), ptr<float>(out), rows, vocab, hidden);
  return launched(ctx, "embedding_kernel");
}

int32_t krm_argmax(krm_ctx* ctx, krm_buf x, krm_buf out_i32, uint32_t rows, uint32_t dim,
                   int32_t io_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype), "krm_argmax: io_dtype %d", io_dtype);
  KRM_REQUIRE(ctx, dim >= 1, "krm_argmax: the reduced dimension is empty");
  if (rows == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && out_i32, "krm_argmax: NULL buffer");
  KRM_IO_DISPATCH(io_dtype,
                  (argmax_kernel<float><<<dim3(rows), dim3(kArgmaxThreads), 0, ctx->stream>>>(
                      ptr<const float>(x), ptr<int32_t>(out_i32), dim)),
                  (argmax_kernel<__half><<<dim3(rows), dim3(kArgmaxThreads), 0, ctx->stream>>>(
                      ptr<const __half>(x), ptr<int32_t>(out_i32), dim)));
  return launched(ctx, "argmax_kernel");
}

int32_t krm_decode_tail(krm_ctx* ctx, krm_buf partials, uint32_t partial_count, krm_buf token_i32,
                        krm_buf lengths, krm_buf history_i32, uint32_t history_len,
                        krm_buf positions_i32, krm_buf table, uint32_t vocab, uint32_t hidden,
                        krm_buf next_row, int32_t table_dtype, int32_t out_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(table_dtype) && valid_dtype(out_dtype),
              "krm_decode_tail: table_dtype %d / out_dtype %d", table_dtype, out_dtype);
  KRM_REQUIRE(ctx, partial_count >= 1 && vocab >= 1 && hidden >= 1,
              "krm_decode_tail: partial_count %u / vocab %u / hidden %u", partial_count, vocab,
              hidden);
  KRM_REQUIRE(ctx, partials && token_i32 && lengths && history_i32 && positions_i32 && table &&
                       next_row,
              "krm_decode_tail: NULL buffer");
  KRM_REQUIRE(ctx, aligned(partials, 8) && aligned(token_i32, 4) && aligned(lengths, 4) &&
                       aligned(history_i32, 4) && aligned(positions_i32, 4) &&
                       aligned(table, dtype_bytes(table_dtype)) &&
                       aligned(next_row, dtype_bytes(out_dtype)),
              "krm_decode_tail: misaligned buffer");
#define KRM_TAIL(WT, XT)                                                                         \
  decode_tail_kernel<WT, XT><<<dim3(1), dim3(kArgmaxThreads), 0, ctx->stream>>>(                 \
      ptr<const uint2>(partials), partial_count, ptr<int32_t>(token_i32), ptr<uint32_t>(lengths), \
      ptr<int32_t>(history_i32), history_len, ptr<int32_t>(positions_i32), ptr<const WT>(table), \
      vocab, hidden, ptr<XT>(next_row))
  if (table_dtype == KRM_F16 && out_dtype == KRM_F16) KRM_TAIL(__half, __half);
  else if (table_dtype == KRM_F16) KRM_TAIL(__half, float);
  else if (out_dtype == KRM_F16) KRM_TAIL(float, __half);
  else KRM_TAIL(float, float);
#undef KRM_TAIL
  return launched(ctx, "decode_tail_kernel");
}

}  // extern "C"
