// int4 `linear` for M > 16 rows (prefill) on the gfx950 matrix cores.
//
// out[m, n] = sum_k x[m,k] * dequant(w)[n,k] + bias[n], same operands and layouts as the GEMV
// (packages/runtime/src/kernels/linear.ts:34-64, packages/runtime/src/kernels/gemm.ts:1187-1237).
// The reference computes this op in f32 and rejects f16 compute with int4 weights
// (packages/runtime/src/kernels/gemm.ts:1204-1209), so this kernel has no same-numerics
// counterpart there: activations are rounded to fp16 (exact when they already are fp16), each
// weight is dequantised to fp16 as fp16(u - 8) * fp16(scale) — one fp16 rounding of a value
// the reference holds exactly — and products are accumulated in f32 by
// v_mfma_f32_32x32x16_f16.  The caller opts in with KRM_COMPUTE_F16.
//
// Workgroup tile BM x BN (waves in a WM x WN grid, 64 x 64 outputs per wave = 2 x 2 MFMA
// tiles); K is walked 64 codes at a time through two LDS buffers:
//   A tile  x[BM rows][64]  fp16, each group of 8 stored as (x0,x4,x1,x5,x2,x6,x3,x7)
//   B tile  w[BN rows][64]  fp16 dequantised, the same order within each group of 8 — the
//           order the nibble trick produces (code i pairs with code i+4), so no shuffle is
//           spent on the weights; the k index inside an MFMA is a free permutation as long as
//           both operands use the same one.
// Rows are padded by 16 bytes so the 16-byte fragment reads of 32 consecutive rows spread over
// all LDS banks.  The next chunk's global loads are issued before the current chunk's MFMAs.
#include "krm_internal.h"

using namespace krm;

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kChunk = 64;             // codes of K per LDS stage
constexpr int kRowBytes = kChunk * 2 + 16;  // padded fp16 row

template <typename ST>
__device__ inline _Float16 scale_as_half(const ST* s, size_t i);
template <>
__device__ inline _Float16 scale_as_half<__half>(const __half* s, size_t i) {
  return __builtin_bit_cast(_Float16, s[i]);
}
template <>
__device__ inline _Float16 scale_as_half<float>(const float* s, size_t i) {
  return (_Float16)s[i];
}

// 8 codes of a word -> 8 fp16 values (u - 8) * scale, order (c0,c4,c1,c5,c2,c6,c3,c7).
__device__ inline uint4 dequant_word(uint32_t word, _Float16 scale) {
  const uint32_t magic = 0x64006400u;  // (1024, 1024)
  const half2_t off_lo = {(_Float16)1032.0f, (_Float16)1032.0f};
  const half2_t sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  const half2_t off_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
  const half2_t s2 = {scale, scale};
  const uint32_t upper = word >> 8;
  const half2_t q0 = (__builtin_bit_cast(half2_t, (word & 0x000F000Fu) | magic) - off_lo) * s2;
  const half2_t q1 =
      (__builtin_elementwise_fma(__builtin_bit_cast(half2_t, (word & 0x00F000F0u) | magic), sixteenth, off_hi)) * s2;
  const half2_t q2 = (__builtin_bit_cast(half2_t, (upper & 0x000F000Fu) | magic) - off_lo) * s2;
  const half2_t q3 =
      (__builtin_elementwise_fma(__builtin_bit_cast(half2_t, (upper & 0x00F000F0u) | magic), sixteenth, off_hi)) * s2;
  return make_uint4(__builtin_bit_cast(uint32_t, q0), __builtin_bit_cast(uint32_t, q1),
                    __builtin_bit_cast(uint32_t, q2), __builtin_bit_cast(uint32_t, q3));
}

// 8 consecutive activations -> fp16 in the order (x0,x4,x1,x5,x2,x6,x3,x7)
template <typename XT>
__device__ inline uint4 load_acts8(const XT* p, bool valid);
template <>
__device__ inline uint4 load_acts8<__half>(const __half* p, bool valid) {
  uint4 raw = *reinterpret_cast<const uint4*>(p);
  const uint32_t keep = valid ? 0xFFFFFFFFu : 0u;
  raw.x &= keep; raw.y &= keep; raw.z &= keep; raw.w &= keep;
  return make_uint4(__builtin_amdgcn_perm(raw.z, raw.x, 0x05040100u),
                    __builtin_amdgcn_perm(raw.z, raw.x, 0x07060302u),
                    __builtin_amdgcn_perm(raw.w, raw.y, 0x05040100u),
                    __builtin_amdgcn_perm(raw.w, raw.y, 0x07060302u));
}
template <>
__device__ inline uint4 load_acts8<float>(const float* p, bool valid) {
  const float4 a = reinterpret_cast<const float4*>(p)[0];
  const float4 b = reinterpret_cast<const float4*>(p)[1];
  const float z = valid ? 1.0f : 0.0f;
  auto pack = [&](float lo, float hi) {
    const half2_t h = {(_Float16)(lo * z), (_Float16)(hi * z)};  // round to nearest even
    return __builtin_bit_cast(uint32_t, h);
  };
  return make_uint4(pack(a.x, b.x), pack(a.y, b.y), pack(a.z, b.z), pack(a.w, b.w));
}

template <typename T>
__device__ inline float bias_f32(const T* p, size_t i);
template <>
__device__ inline float bias_f32<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ inline float bias_f32<__half>(const __half* p, size_t i) { return __half2float(p[i]); }
template <typename T>
__device__ inline void store_out(T* p, size_t i, float v);
template <>
__device__ inline void store_out<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ inline void store_out<__half>(__half* p, size_t i, float v) {
  p[i] = __float2half_rn(v);
}

template <typename XT, typename ST, int WM, int WN>
__global__ __launch_bounds__(WM * WN * 64) __attribute__((amdgpu_waves_per_eu(1, 2)))
void gemm_i4_f16_kernel(const XT* __restrict__ x, const uint32_t* __restrict__ w,
                        const ST* __restrict__ scales, const XT* __restrict__ bias,
                        XT* __restrict__ out, uint32_t m, uint32_t n, uint32_t k,
                        uint32_t group_shift, uint32_t m_blocks, uint32_t n_blocks,
                        uint32_t wide_rows) {
  constexpr int kThreads = WM * WN * 64;
  constexpr int BM = WM * 64, BN = WN * 64;
  constexpr int kAPieces = BM * (kChunk / 8);        // 16-byte pieces of the A tile
  constexpr int kAPer = kAPieces / kThreads;         // per thread
  constexpr int kBPieces = BN * (kChunk / 8);        // words of the B tile
  constexpr int kBPer = kBPieces / kThreads;         // words per thread (consecutive in a row)
  static_assert(kAPieces % kThreads == 0 && kBPieces % kThreads == 0, "tile / thread mismatch");
  static_assert(kBPer == 1 || kBPer == 2 || kBPer == 4 || kBPer == 8, "B words per thread");

  __shared__ __attribute__((aligned(16))) unsigned char lds_a[2][BM * kRowBytes];
  __shared__ __attribute__((aligned(16))) unsigned char lds_b[2][BN * kRowBytes];

  // Workgroups that share an x panel are placed on one XCD (ids are dealt round-robin over 8
  // XCDs), so that panel stays in that XCD's L2 while the weights stream through.
  uint32_t mb, nb;
  {
    const uint32_t id = blockIdx.x;
    if (8 % m_blocks == 0) {
      const uint32_t xcd = id & 7, slot = id >> 3, per = 8 / m_blocks;
      mb = xcd % m_blocks;
      nb = slot * per + xcd / m_blocks;
    } else {
      mb = id % m_blocks;
      nb = id / m_blocks;
    }
    if (nb >= n_blocks) return;
  }
  const uint32_t m0 = mb * BM, n0 = nb * BN;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WM, wn = wave / WM;

  const uint32_t words_per_row = k >> 3;
  const uint32_t groups_per_row = k >> group_shift;
  const uint32_t chunks = (k + kChunk - 1) / kChunk;

  // staging assignment
  uint32_t a_row[kAPer], a_pc[kAPer];
#pragma unroll
  for (int i = 0; i < kAPer; ++i) {
    const int p = tid + i * kThreads;
    a_row[i] = p / (kChunk / 8);
    a_pc[i] = p % (kChunk / 8);
  }
  const uint32_t b_row = (tid * kBPer) / (kChunk / 8);
  const uint32_t b_w0 = (tid * kBPer) % (kChunk / 8);
  const uint32_t b_grow = min(n0 + b_row, n - 1);  // rows past N re-read the last row, unused

  uint4 a_regs[kAPer];
  uint32_t b_regs[kBPer];
  _Float16 b_scale[kBPer];

  auto fetch = [&](uint32_t chunk) {
    const uint32_t k0 = chunk * kChunk;
#pragma unroll
    for (int i = 0; i < kAPer; ++i) {
      const uint32_t row = m0 + a_row[i], kk = k0 + a_pc[i] * 8;
      const bool valid = row < m && kk < k;
      const uint32_t rr = valid ? row : 0u, kc = valid ? kk : 0u;
      a_regs[i] = load_acts8<XT>(x + (size_t)rr * k + kc, valid);
    }
    // 16-byte weight loads when the rows are 16-byte aligned and the chunk lies inside K
    // (both conditions are uniform over the workgroup).
    const bool vec = kBPer >= 4 && wide_rows && k0 + kChunk <= k;
    if (vec) {
#pragma unroll
      for (int j = 0; j < kBPer; j += 4) {
        const uint4 v = *reinterpret_cast<const uint4*>(
            w + (size_t)b_grow * words_per_row + (k0 >> 3) + b_w0 + j);
        b_regs[j] = v.x;
        if (j + 1 < kBPer) b_regs[j + 1] = v.y;
        if (j + 2 < kBPer) b_regs[j + 2] = v.z;
        if (j + 3 < kBPer) b_regs[j + 3] = v.w;
      }
    }
#pragma unroll
    for (int j = 0; j < kBPer; ++j) {
      const uint32_t kk = k0 + (b_w0 + j) * 8;
      const uint32_t kc = kk < k ? kk : 0u;  // past the end of K: x is zero there, w is unused
      if (!vec) b_regs[j] = w[(size_t)b_grow * words_per_row + (kc >> 3)];
      b_scale[j] = scale_as_half<ST>(scales, (size_t)b_grow * groups_per_row + (kc >> group_shift));
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kAPer; ++i)
      *reinterpret_cast<uint4*>(&lds_a[buf][a_row[i] * kRowBytes + a_pc[i] * 16]) = a_regs[i];
#pragma unroll
    for (int j = 0; j < kBPer; ++j)
      *reinterpret_cast<uint4*>(&lds_b[buf][b_row * kRowBytes + (b_w0 + j) * 16]) =
          dequant_word(b_regs[j], b_scale[j]);
  };

  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  fetch(0);
  stage(0);
  __syncthreads();

  const int frag_row = lane & 31, frag_g = lane >> 5;
  for (uint32_t chunk = 0; chunk < chunks; ++chunk) {
    const int buf = chunk & 1;
    if (chunk + 1 < chunks) fetch(chunk + 1);
#pragma unroll
    for (int ks = 0; ks < kChunk / 16; ++ks) {
      half8_t af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = wm * 64 + i * 32 + frag_row;
        af[i] = *reinterpret_cast<const half8_t*>(
            &lds_a[buf][row * kRowBytes + (ks * 2 + frag_g) * 16]);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int row = wn * 64 + j * 32 + frag_row;
        bf[j] = *reinterpret_cast<const half8_t*>(
            &lds_b[buf][row * kRowBytes + (ks * 2 + frag_g) * 16]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (chunk + 1 < chunks) stage(buf ^ 1);
    __syncthreads();
  }

  // epilogue: lane holds column (lane % 32); register r holds row 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t col = n0 + wn * 64 + j * 32 + frag_row;
    if (col >= n) continue;
    const float add = bias ? bias_f32<XT>(bias, col) : 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const uint32_t row = m0 + wm * 64 + i * 32 + 8 * (r / 4) + 4 * frag_g + (r % 4);
        if (row < m) store_out<XT>(out, (size_t)row * n + col, acc[i][j][r] + add);
      }
    }
  }
}

template <typename XT, typename ST, int WM, int WN>
int32_t launch(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
               uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift) {
  constexpr int BM = WM * 64, BN = WN * 64;
  const uint32_t m_blocks = (m + BM - 1) / BM, n_blocks = (n + BN - 1) / BN;
  uint64_t total;
  if (8 % m_blocks == 0) {
    const uint32_t per = 8 / m_blocks;
    total = (uint64_t)((n_blocks + per - 1) / per) * 8;
  } else {
    total = (uint64_t)m_blocks * n_blocks;
  }
  if (total > 0x7fffffffull) return fail(ctx, KRM_ERR_VALIDATION, "linear: grid too large");
  gemm_i4_f16_kernel<XT, ST, WM, WN><<<dim3((unsigned)total), dim3(WM * WN * 64), 0, ctx->stream>>>(
      ptr<const XT>(x), ptr<const uint32_t>(w), ptr<const ST>(scales), ptr<const XT>(bias),
      ptr<XT>(out), m, n, k, group_shift, m_blocks, n_blocks,
      (k % 32 == 0 && aligned(w, 16)) ? 1u : 0u);
  return launched(ctx, "gemm_i4_f16_kernel");
}

template <typename XT, typename ST>
int32_t pick_tile(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                  uint32_t m, uint32_t n, uint32_t k, uint32_t group) {
  uint32_t group_shift = 0;
  while ((1u << group_shift) < group) ++group_shift;
  // 128 x 128 tiles unless that leaves compute units idle; then 128 x 64 or 64 x 64.
  const uint64_t cus = (uint64_t)ctx->num_cus;
  const uint64_t big = (uint64_t)((m + 127) / 128) * ((n + 127) / 128);
  const uint64_t mid = (uint64_t)((m + 127) / 128) * ((n + 63) / 64);
  if (m > 64 && big >= 2 * cus)
    return launch<XT, ST, 2, 2>(ctx, x, w, scales, bias, out, m, n, k, group_shift);
  if (m > 64 && mid >= cus)
    return launch<XT, ST, 2, 1>(ctx, x, w, scales, bias, out, m, n, k, group_shift);
  return launch<XT, ST, 1, 1>(ctx, x, w, scales, bias, out, m, n, k, group_shift);
}

}  // namespace

namespace krm {

int32_t linear_i4_gemm_f16(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                           krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                           int32_t io_dtype, int32_t scale_dtype) {
  if (io_dtype == KRM_F16) {
    if (scale_dtype == KRM_F16)
      return pick_tile<__half, __half>(ctx, x, w, scales, bias, out, m, n, k, group);
    return pick_tile<__half, float>(ctx, x, w, scales, bias, out, m, n, k, group);
  }
  if (scale_dtype == KRM_F16)
    return pick_tile<float, __half>(ctx, x, w, scales, bias, out, m, n, k, group);
  return pick_tile<float, float>(ctx, x, w, scales, bias, out, m, n, k, group);
}

}  // namespace krm
