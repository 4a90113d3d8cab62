// w4a8 `linear` for gfx950: per-token int8 activations x int4 group-quantised weights with
// integer dot products.
//
// Semantics follow the reference's opt-in integer-dot path for int4-resident weights
// (packages/runtime/src/kernels/quantize-rows.ts:89-146 for the activation quantiser,
// packages/runtime/src/kernels/linear-i8a8.ts:47-72,376-510 for the product, contract
// docs/decisions/0076-w4a8-linear-execution.md:40-60, CPU reference
// packages/runtime/src/reference/i8a8.ts:92-118,209-231):
//
//   xs[row]  = max(f32(amax(|x[row]|) * f32(1/127)), f32 tiny)      NaN in the row -> NaN
//   xq       = clamp(round-half-even(x / xs[row]), -127, +127)
//   accf     = 0;  for each group gi of the row, ascending:
//                acci = sum over the group of xq * wq               exact, int32
//                accf = fma(f32(acci), wscale[col, gi], accf)       one rounding per group
//   out      = fma(accf, xs[row], bias[col])
//
// Every floating-point operation is a correctly rounded IEEE operation in a fixed order, and
// everything inside a group is exact integer arithmetic, so the result does not depend on how
// a kernel tiles the problem: the kernels here differ in speed only and agree bit for bit with
// each other and with the CPU statement of the formula.
//
// The weight nibbles are stored u = q + 8.  u ^ 8 is q's 4-bit two's complement, and a
// two's-complement nibble in the upper half of a byte reads as the signed byte 16 * q; the
// integer dot products therefore run on bytes 16 * q (two ops per four codes, no sign
// extension) and the exact factor 16 is shifted out of the group sum before it is converted.
#include "krm_internal.h"

namespace {

using namespace krm;

typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));

constexpr float kF32Tiny = 1.1754943508222875e-38f;
constexpr uint32_t kMaxGroup = 2113664;      // int32 holds g * 127 * 8 (linear-i8a8.ts:124-132)
constexpr uint32_t kMaxGroupTimes16 = 131072;  // int32 holds g * 127 * 8 * 16

template <typename ST>
__device__ inline float scale_f32(const ST* s, size_t i);
template <>
__device__ inline float scale_f32<float>(const float* s, size_t i) { return s[i]; }
template <>
__device__ inline float scale_f32<__half>(const __half* s, size_t i) { return __half2float(s[i]); }

__device__ inline bool is_nan_bits(float v) {
  return (__float_as_uint(v) & 0x7fffffffu) > 0x7f800000u;
}

// ------------------------------------------------------------------------- quantize_rows
//
// One workgroup per row (grid-stride over rows): |x| maximum with NaN propagation, then the
// quotients.  Rows of up to 256 * 4 * kQuantCache elements stay in registers between the two
// (one trip to memory, all loads in flight together); longer rows are read twice.  x / s is the
// correctly rounded f32 division, so the codes equal the CPU formula's for every input, also
// next to a rounding tie.
constexpr int kQuantCache = 12;  // float4 per thread: rows of up to 12288 elements

// x / s must be the correctly rounded quotient only where it decides the code: t = x * (1 / s)
// (1 / s correctly rounded) lies within 2.3e-5 of it for |x / s| <= 127.5, so when t is further
// than 2^-14 from every half-integer both round to the same integer and the product serves;
// otherwise (and for a NaN) the lane divides.
__device__ inline uint32_t quantize4(const float4& v, float s, float inv_s) {
  const float f[4] = {v.x, v.y, v.z, v.w};
  float t[4];
  bool near[4], any_near = false;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    t[e] = f[e] * inv_s;
    near[e] = !(fabsf(__builtin_amdgcn_fractf(fabsf(t[e])) - 0.5f) > 0x1p-14f);
    any_near = any_near || near[e];
  }
  if (__builtin_amdgcn_ballot_w64(any_near) != 0) {  // wave-uniform and rare
    asm volatile("" ::: "memory");  // keeps the divisions inside the branch
#pragma unroll
    for (int e = 0; e < 4; ++e) t[e] = near[e] ? f[e] / s : t[e];
  }
  uint32_t packed = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float r = rintf(t[e]);
    r = is_nan_bits(r) ? 0.f : fminf(fmaxf(r, -127.f), 127.f);
    packed |= ((uint32_t)(int32_t)r & 0xffu) << (8 * e);
  }
  return packed;
}

__global__ __launch_bounds__(256) void quantize_rows_kernel(const float* __restrict__ x,
                                                            uint32_t* __restrict__ xq,
                                                            float* __restrict__ xs,
                                                            uint32_t rows, uint32_t dim) {
  __shared__ float s_max[4];
  __shared__ uint32_t s_nan[4];
  const uint32_t quads = dim >> 2;
  const bool cached = quads <= 256u * kQuantCache;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (uint32_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * dim);
    float4 cache[kQuantCache];
    float amax = 0.f;
    bool nan = false;
    auto fold = [&](const float4& v) {
      const float a[4] = {fabsf(v.x), fabsf(v.y), fabsf(v.z), fabsf(v.w)};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        nan = nan || is_nan_bits(a[e]);
        amax = fmaxf(amax, a[e]);  // ignores a NaN operand; the flag carries it
      }
    };
    if (cached) {
#pragma unroll
      for (int i = 0; i < kQuantCache; ++i) {
        if (256u * i >= quads) break;  // uniform: the row ends before this stride
        const uint32_t at = threadIdx.x + 256u * i;
        cache[i] = xr[at < quads ? at : 0u];  // past the row: its first quad again, not folded
      }
#pragma unroll
      for (int i = 0; i < kQuantCache; ++i)
        if (threadIdx.x + 256u * i < quads) fold(cache[i]);
    } else {
      for (uint32_t i = threadIdx.x; i < quads; i += 256) fold(xr[i]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const bool wave_nan = __any(nan);
    if (lane == 0) {
      s_max[wave] = amax;
      s_nan[wave] = wave_nan ? 1u : 0u;
    }
    __syncthreads();
    amax = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    const bool row_nan = (s_nan[0] | s_nan[1] | s_nan[2] | s_nan[3]) != 0u;
    float s = fmaxf(amax * (float)(1.0 / 127.0), kF32Tiny);
    if (row_nan) s = __uint_as_float(0x7fc00000u);
    if (threadIdx.x == 0) xs[row] = s;
    const float inv_s = 1.0f / s;
    uint32_t* qr = xq + (size_t)row * quads;
    if (cached) {
#pragma unroll
      for (int i = 0; i < kQuantCache; ++i) {
        const uint32_t at = threadIdx.x + 256u * i;
        if (at < quads) qr[at] = quantize4(cache[i], s, inv_s);
      }
    } else {
      for (uint32_t i = threadIdx.x; i < quads; i += 256) qr[i] = quantize4(xr[i], s, inv_s);
    }
    __syncthreads();  // s_max / s_nan are rewritten by the next row
  }
}

// ------------------------------------------------------------------- any shape (fallback)
//
// One wave per output column, one x row at a time; the lanes share the words of a group and
// add their exact partial sums.  Covers every group size the format allows; the kernels below
// take the shapes that matter for speed.
template <typename ST>
__global__ __launch_bounds__(256) void linear_w4a8_generic_kernel(
    const uint32_t* __restrict__ xq, const float* __restrict__ xs, const uint32_t* __restrict__ w,
    const ST* __restrict__ scales, const float* __restrict__ bias, float* __restrict__ out,
    uint32_t m, uint32_t n, uint32_t k, uint32_t group) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t col = blockIdx.x * 4 + wave;
  if (col >= n) return;
  const uint32_t words_per_group = group >> 3, groups = k / group;
  const uint32_t* wrow = w + (size_t)col * (k >> 3);
  for (uint32_t row = blockIdx.y; row < m; row += gridDim.y) {
    const uint32_t* xrow = xq + (size_t)row * (k >> 2);
    float accf = 0.f;
    for (uint32_t gi = 0; gi < groups; ++gi) {
      int32_t acci = 0;
      for (uint32_t j = lane; j < words_per_group; j += 64) {
        const uint32_t word = wrow[(size_t)gi * words_per_group + j];
        const uint32_t x0 = xrow[((size_t)gi * group >> 2) + 2 * j];
        const uint32_t x1 = xrow[((size_t)gi * group >> 2) + 2 * j + 1];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int32_t q = (int32_t)((word >> (4 * e)) & 15u) - 8;
          const int32_t xv = (int32_t)(int8_t)(((e < 4 ? x0 : x1) >> (8 * (e & 3))) & 0xffu);
          acci += q * xv;
        }
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) acci += __shfl_xor(acci, off);
      accf = fmaf((float)acci, scale_f32<ST>(scales, (size_t)col * groups + gi), accf);
    }
    if (lane == 0) out[(size_t)row * n + col] = fmaf(accf, xs[row], bias ? bias[col] : 0.f);
  }
}

// --------------------------------------------------------------- few rows of x (decode)
//
// Weight-streaming form for M <= 8 and 32 <= group <= 2048.  A wave owns two weight rows over
// the whole K and MB rows of x; a step is 64 lanes x 16 bytes = 2048 codes per weight row, a
// lane's 32 codes lie inside one group.  Per word: u ^ 8 once, the odd codes are the upper
// nibbles in place, the even codes one shift away; x's bytes are regrouped (even, odd) to
// match and two v_dot4_i32_i8 add eight products.  The lanes of a group add their sums
// (exact), the group totals and scales go through LDS to one lane per output, which runs the
// ascending fma chain.
//  FUSED: `xin` is the f32 activations themselves and the quantiser runs in the prologue: every
//  workgroup turns the whole block of x rows into int8 in LDS (the rows are needed whole by
//  every output; quantising them again per workgroup costs less than a launch of its own, and
//  it happens while the weights are on their way).  Same maximum, same scale, same correctly
//  rounded quotients as quantize_rows_kernel, so the result is the two-launch result bit for
//  bit.  The block's MB * K elements are held in registers between maximum and quotient, FUSE
//  float4 per thread (a compile-time count of unconditional loads: the waits for them can then
//  leave the weight requests behind them in flight): MB * K <= 256 * 4 * FUSE, FUSE <= 16.
constexpr int kFuseCache = 16;

template <typename ST, int MB, int FUSE>
__global__ __launch_bounds__(256) void linear_w4a8_rows_kernel(
    const void* __restrict__ xin, const float* __restrict__ xs, const uint32_t* __restrict__ w,
    const ST* __restrict__ scales, const float* __restrict__ bias, float* __restrict__ out,
    uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift) {
  constexpr int ROWS = 2;
  constexpr int kStep = 64 * 32;
  constexpr bool FUSED = FUSE > 0;
  __shared__ int32_t s_sum[4][ROWS * MB][64];
  __shared__ float s_ws[4][ROWS][64];
  __shared__ float s_max[4][MB];
  __shared__ uint32_t s_nan[4][MB];
  __shared__ float s_xs[MB];
  extern __shared__ __align__(16) uint32_t s_xq[];  // FUSED: MB rows of K int8
  const uint32_t* xq = static_cast<const uint32_t*>(xin);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t row0 = (blockIdx.x * 4 + wave) * ROWS;
  const uint32_t b0 = blockIdx.y * MB;
  const uint32_t span = 1u << (group_shift - 5);  // lanes per group
  const uint32_t per_step = 64u / span;           // groups per step
  const uint32_t groups = k >> group_shift;
  const uint32_t steps = (k + kStep - 1) / kStep;

  const uint32_t* wrow[ROWS];
  const ST* srow[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const uint32_t row = min(row0 + r, n - 1);  // rows past N re-read the last row, unused
    wrow[r] = w + (size_t)row * (k >> 3);
    srow[r] = scales + (size_t)row * groups;
  }
  const uint32_t* xrow[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) xrow[b] = xq + (size_t)min(b0 + b, m - 1) * (k >> 2);

  struct Step {
    uint4 w[ROWS];
    float s[ROWS];
    uint4 x[MB][2];
  };
  // requests only; lanes past the end of K re-read the row's start and are masked later
  auto fetch_x = [&](uint32_t step, Step& d) {
    const uint32_t k0 = step * kStep + lane * 32;
    const uint32_t kc = k0 < k ? k0 : 0u;
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const uint32_t* row = FUSED ? s_xq + (size_t)b * (k >> 2) : xrow[b];
      d.x[b][0] = *reinterpret_cast<const uint4*>(row + (kc >> 2));
      d.x[b][1] = *reinterpret_cast<const uint4*>(row + (kc >> 2) + 4);
    }
  };
  auto fetch_w = [&](uint32_t step, Step& d) {
    const uint32_t k0 = step * kStep + lane * 32;
    const uint32_t kc = k0 < k ? k0 : 0u;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      d.w[r] = *reinterpret_cast<const uint4*>(wrow[r] + (kc >> 3));
      d.s[r] = scale_f32<ST>(srow[r], kc >> group_shift);
    }
  };
  // activations first: they come from the cache, and loads return in order
  auto fetch = [&](uint32_t step, Step& d) {
    fetch_x(step, d);
    fetch_w(step, d);
  };

  const int chain_r = lane / MB, chain_b = lane % MB;  // the output a chain lane owns
  const bool chain = lane < ROWS * MB;
  float accf = 0.f;

  Step cur, nxt;
  if constexpr (FUSED) {
    // x first (it comes from the cache and returns first), then the first step's weights; the
    // quantiser below runs while those are on their way.
    const float* xf = static_cast<const float*>(xin) + (size_t)b0 * k;
    const uint32_t row_quads = k >> 2;
    const uint32_t live_rows = m - b0 < (uint32_t)MB ? m - b0 : (uint32_t)MB;
    const uint32_t quads = live_rows * row_quads;  // rows of the block lie back to back
    float4 cache[FUSED ? FUSE : 1];
#pragma unroll
    for (int i = 0; i < FUSE; ++i) {
      const uint32_t at = threadIdx.x + 256u * i;
      cache[i] = reinterpret_cast<const float4*>(xf)[at < quads ? at : 0u];  // no branch
    }
    fetch_w(0, cur);
    fetch_w(steps > 1 ? 1u : 0u, nxt);
    __builtin_amdgcn_sched_barrier(0);  // every request is out before the first x value is used
    float amax[MB];
    bool nan[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      amax[b] = 0.f;
      nan[b] = false;
    }
#pragma unroll
    for (int i = 0; i < FUSE; ++i) {
      const uint32_t at = threadIdx.x + 256u * i;
      const bool live = at < quads;
      const uint32_t row = MB == 1 ? 0u : at / row_quads;
      const float a[4] = {fabsf(cache[i].x), fabsf(cache[i].y), fabsf(cache[i].z),
                          fabsf(cache[i].w)};
      float top = 0.f;
      bool bad = false;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        bad = bad || is_nan_bits(a[e]);
        top = fmaxf(top, a[e]);  // ignores a NaN operand; the flag carries it
      }
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const bool mine = live && row == (uint32_t)b;
        amax[b] = mine ? fmaxf(amax[b], top) : amax[b];
        nan[b] = nan[b] || (mine && bad);
      }
    }
#pragma unroll
    for (int b = 0; b < MB; ++b) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) amax[b] = fmaxf(amax[b], __shfl_xor(amax[b], off));
      const bool wave_nan = __any(nan[b]);
      if (lane == 0) {
        s_max[wave][b] = amax[b];
        s_nan[wave][b] = wave_nan ? 1u : 0u;
      }
    }
    __syncthreads();
    float scale_of[MB], inverse_of[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const float top = fmaxf(fmaxf(s_max[0][b], s_max[1][b]), fmaxf(s_max[2][b], s_max[3][b]));
      const bool row_nan = (s_nan[0][b] | s_nan[1][b] | s_nan[2][b] | s_nan[3][b]) != 0u;
      float sc = fmaxf(top * (float)(1.0 / 127.0), kF32Tiny);
      if (row_nan) sc = __uint_as_float(0x7fc00000u);
      scale_of[b] = sc;
      inverse_of[b] = 1.0f / sc;
      if (threadIdx.x == 0) s_xs[b] = sc;
    }
#pragma unroll
    for (int i = 0; i < FUSE; ++i) {
      const uint32_t at = threadIdx.x + 256u * i;
      if (at < quads) {
        const uint32_t row = MB == 1 ? 0u : at / row_quads;
        float sc = scale_of[0], inv = inverse_of[0];
#pragma unroll
        for (int b = 1; b < MB; ++b) {
          sc = row == (uint32_t)b ? scale_of[b] : sc;
          inv = row == (uint32_t)b ? inverse_of[b] : inv;
        }
        s_xq[at] = quantize4(cache[i], sc, inv);
      }
    }
    // rows of the block past M: zeros (their outputs are not stored)
    for (uint32_t at = quads + threadIdx.x; at < (uint32_t)MB * row_quads; at += 256) s_xq[at] = 0u;
    __syncthreads();
    fetch_x(0, cur);
  } else {
    fetch(0, cur);
  }
  auto consume = [&](uint32_t step) {
    const bool active = step * kStep + lane * 32 < k;
    int32_t acc[ROWS][MB];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int b = 0; b < MB; ++b) acc[r][b] = 0;
    uint32_t hi[ROWS][4], lo[ROWS][4];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const uint32_t words[4] = {cur.w[r].x, cur.w[r].y, cur.w[r].z, cur.w[r].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t t = words[j] ^ 0x88888888u;
        hi[r][j] = t & 0xF0F0F0F0u;          // bytes 16 * q of codes 1, 3, 5, 7
        lo[r][j] = (t << 4) & 0xF0F0F0F0u;   // bytes 16 * q of codes 0, 2, 4, 6
      }
    }
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const uint32_t xw[8] = {cur.x[b][0].x, cur.x[b][0].y, cur.x[b][0].z, cur.x[b][0].w,
                              cur.x[b][1].x, cur.x[b][1].y, cur.x[b][1].z, cur.x[b][1].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t even = __builtin_amdgcn_perm(xw[2 * j + 1], xw[2 * j], 0x06040200u);
        const uint32_t odd = __builtin_amdgcn_perm(xw[2 * j + 1], xw[2 * j], 0x07050301u);
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
          acc[r][b] = __builtin_amdgcn_sdot4((int)lo[r][j], (int)even, acc[r][b], false);
          acc[r][b] = __builtin_amdgcn_sdot4((int)hi[r][j], (int)odd, acc[r][b], false);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        int32_t v = active ? acc[r][b] : 0;
        for (uint32_t off = 1; off < span; off <<= 1) v += __shfl_xor(v, (int)off);
        acc[r][b] = v;
      }
    if ((lane & (span - 1)) == 0) {
      const uint32_t slot = lane >> (group_shift - 5);
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        s_ws[wave][r][slot] = cur.s[r];
#pragma unroll
        for (int b = 0; b < MB; ++b) s_sum[wave][r * MB + b][slot] = acc[r][b];
      }
    }
    __syncthreads();
    if (chain) {
      const uint32_t first = step * per_step;
      const uint32_t count = groups - first < per_step ? groups - first : per_step;
      for (uint32_t j = 0; j < count; ++j)
        accf = fmaf((float)(s_sum[wave][lane][j] >> 4), s_ws[wave][chain_r][j], accf);
    }
    __syncthreads();
    cur = nxt;
  };
  uint32_t step = 0;
  if constexpr (FUSED) {  // the second step's weights were requested in front of the quantiser
    fetch_x(steps > 1 ? 1u : 0u, nxt);
    consume(0);
    step = 1;
  }
  for (; step < steps; ++step) {
    fetch(step + 1 < steps ? step + 1 : step, nxt);  // unconditional: no wait inside a branch
    consume(step);
  }
  if (chain) {
    const uint32_t row = row0 + chain_r, xb = b0 + chain_b;
    if (row < n && xb < m)
      out[(size_t)xb * n + row] = fmaf(accf, FUSED ? s_xs[chain_b] : xs[xb], bias ? bias[row] : 0.f);
  }
}

// ------------------------------------------------------------------ many rows (prefill)
//
// Matrix-core form for M > 8 and 64 <= group <= 131072: v_mfma_i32_32x32x32_i8 with A = xq
// (rows of the tile), B = the weight bytes 16 * q (columns), int32 accumulators.
//  * Lane (n = lane % 32, h = lane / 32) of a column tile holds 16 bytes = codes
//    64c + 32h .. + 31 of weight row n per 64-code chunk and expands words 2s, 2s + 1 into the
//    operand of the chunk's MFMA step s: (even codes of word 2s, odd codes of word 2s,
//    even codes of word 2s + 1, odd codes of word 2s + 1).
//  * xq's bytes are regrouped (even, odd) per 8 codes on the way into LDS, so that lane (m, h)
//    reads its 16 operand bytes at 64c + 32h + 16s in one piece and byte j of A meets byte j
//    of B.  LDS rows are padded by 16 bytes.
//  * The first MFMA of a group starts from a zero accumulator; after the group's last chunk
//    the int32 sums (16 x the group sums) are converted and fused into the f32 accumulators
//    with the lane's column scale / 16 — the same real product, hence the same rounded result;
//    where an f32 scale / 16 is not exact (a subnormal quotient) the sums are shifted instead.
//    The activation scale and the bias follow once, at the store.
//  * Every stage issues the same loads in the same order whatever K is (addresses past K are
//    clamped, chunks past K multiply zeros and are fused with a zero scale): a branch around a
//    load would make the compiler's wait counts assume the worst path.
// GSH = log2(group) for groups of 64, 128, 256 (group boundaries known at compile time);
// GSH = 0: any larger group (a whole number of stages).
// Workgroup ids are dealt so that the row blocks of a column block run on one XCD.
// (Weights loaded straight from global memory into the operand registers, without LDS, were
// measured 1.5 x slower: a lane's own 16 bytes of its own row make every quad of lanes touch
// four cache lines, and the vector cache's tag lookups become the bound.)
//
// Both operands go through LDS: eight waves, workgroup tile (64 * MT) x (128 * WN), wave
// (wm, wn) = 32 * MT rows x 32 * WN columns (WN = 1 when 256-column tiles would leave a
// quarter of the chip without work).  The packed weight
// bytes are staged as they are (coalesced 16-byte loads, 128 bytes of a row per stage) and
// expanded to the bytes 16 * q in registers after the LDS read, so LDS holds a quarter of what
// dequantised bytes would take; xq is staged with its bytes regrouped (even, odd) as above.
// The stage's group scales are staged too, already converted.  Two waves share a SIMD: one
// wave's group flush (VALU) runs under the other's MFMAs.
template <typename ST, int GSH, int MT, int WN>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void linear_w4a8_tile_kernel(
    const uint8_t* __restrict__ xq, const float* __restrict__ xs, const uint8_t* __restrict__ w,
    const ST* __restrict__ scales, const float* __restrict__ bias, float* __restrict__ out,
    uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift, uint32_t m_blocks,
    uint32_t n_blocks) {
  constexpr int BM = 2 * 32 * MT, BN = 4 * 32 * WN;  // two wave rows, four wave columns
  constexpr int kStage = 256;                 // codes per LDS stage
  constexpr int kRowA = kStage + 16;          // bytes per LDS row of xq
  constexpr int kRowB = kStage / 2 + 16;      // bytes per LDS row of packed weights
  constexpr int kChunksPerGroup = GSH ? (1 << (GSH - 6)) : 4;  // inside a stage
  constexpr int kScalesPerStage = GSH ? (kStage >> GSH) : 1;
  constexpr int kAUnits = BM * 16 / 512;      // 16-byte units of xq per thread and stage
  constexpr int kBUnits = BN * 8 / 512;       // and of packed weights
  __shared__ __align__(16) uint8_t s_a[2][BM * kRowA];
  __shared__ __align__(16) uint8_t s_b[2][BN * kRowB];
  __shared__ __align__(16) float s_s[2][BN][4];

  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
  const uint32_t mb = slot % m_blocks, nb = (slot / m_blocks) * 8u + xcd;
  if (nb >= n_blocks) return;  // the whole workgroup leaves before any barrier
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  const int frag_row = lane & 31, frag_h = lane >> 5;
  const uint32_t m0 = mb * BM, n0 = nb * BN;
  const uint32_t shift = GSH ? (uint32_t)GSH : group_shift;
  const uint32_t groups = k >> shift;
  const uint32_t chunks_total = k >> 6;
  const uint32_t stages = (k + kStage - 1) / kStage;
  const uint32_t stages_per_group = GSH ? 1u : 1u << (shift - 8);

  // staging roles: xq rows in 16 units of 16 bytes (rows tid / 16 + 32 i), weight rows in 8
  // (rows tid / 8 + 64 i), one scale row per thread; 32-bit offsets from the three bases
  const uint32_t arow0 = tid >> 4, aunit = (tid & 15u) * 16u;
  const uint32_t brow0 = tid >> 3, bunit = (tid & 7u) * 16u;
  const ST* ssrc = scales + (size_t)min(n0 + (uint32_t)(tid % BN), n - 1) * groups;
  struct Staged {
    uint4 a[kAUnits];
    uint4 b[kBUnits];
    ST s[kScalesPerStage];
  };
  // Requests only, clamped addresses: every stage issues the same loads in the same order.
  auto load_stage = [&](uint32_t stage, Staged& d) {
    const uint32_t a_at = stage * kStage + aunit, b_at = stage * (kStage / 2) + bunit;
    const uint32_t a_off = a_at < k ? a_at : 0u, b_off = b_at < (k >> 1) ? b_at : 0u;
#pragma unroll
    for (int i = 0; i < kAUnits; ++i)
      d.a[i] = *reinterpret_cast<const uint4*>(
          xq + (size_t)min(m0 + arow0 + 32u * i, m - 1) * k + a_off);
#pragma unroll
    for (int i = 0; i < kBUnits; ++i)
      d.b[i] = *reinterpret_cast<const uint4*>(
          w + (size_t)min(n0 + brow0 + 64u * i, n - 1) * (k >> 1) + b_off);
#pragma unroll
    for (int j = 0; j < kScalesPerStage; ++j) {
      const uint32_t code = stage * kStage + (j << (GSH ? GSH : 8));
      d.s[j] = ssrc[(code < k ? code : 0u) >> shift];
    }
  };
  // codes past the end of K are parked as zeros in xq: their products vanish whatever B holds
  auto park_stage = [&](uint32_t stage, int buf, const Staged& d) {
    const uint32_t keep = stage * kStage + aunit < k ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int i = 0; i < kAUnits; ++i) {
      uint4 v;
      v.x = __builtin_amdgcn_perm(d.a[i].y, d.a[i].x, 0x06040200u) & keep;
      v.y = __builtin_amdgcn_perm(d.a[i].y, d.a[i].x, 0x07050301u) & keep;
      v.z = __builtin_amdgcn_perm(d.a[i].w, d.a[i].z, 0x06040200u) & keep;
      v.w = __builtin_amdgcn_perm(d.a[i].w, d.a[i].z, 0x07050301u) & keep;
      *reinterpret_cast<uint4*>(&s_a[buf][(arow0 + 32u * i) * kRowA + aunit]) = v;
    }
#pragma unroll
    for (int i = 0; i < kBUnits; ++i)
      *reinterpret_cast<uint4*>(&s_b[buf][(brow0 + 64u * i) * kRowB + bunit]) = d.b[i];
    if (tid < BN) {
#pragma unroll
      for (int j = 0; j < kScalesPerStage; ++j) s_s[buf][tid][j] = scale_f32<ST>(&d.s[j], 0);
    }
  };

  v16i_t acc[MT][WN];
  float accf[MT][WN][16];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < WN; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[mt][nt][r] = 0;
        accf[mt][nt][r] = 0.f;
      }
  const v16i_t zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  Staged staged;
  load_stage(0, staged);
  park_stage(0, 0, staged);
  __syncthreads();

  const uint32_t a_base = (uint32_t)((wm * 32 * MT + frag_row) * kRowA + 32 * frag_h);
  const uint32_t b_base = (uint32_t)((wn * 32 * WN + frag_row) * kRowB + 16 * frag_h);
  auto run_stage = [&](uint32_t stage, int buf) {
    load_stage(stage + 1, staged);
    const uint32_t first_chunk = stage * 4u;
    const bool stage_opens = GSH ? true : (stage & (stages_per_group - 1)) == 0;
    const bool stage_closes = GSH ? true : ((stage + 1) & (stages_per_group - 1)) == 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const bool valid = first_chunk + c < chunks_total;
      const bool opens_static = GSH != 0 && (c % kChunksPerGroup) == 0;
      const bool closes = GSH ? ((c + 1) % kChunksPerGroup) == 0 : (stage_closes && c == 3);
      if (GSH == 0 && stage_opens && c == 0) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int nt = 0; nt < WN; ++nt) acc[mt][nt] = zero;
      }
      uint4 braw[WN];
#pragma unroll
      for (int nt = 0; nt < WN; ++nt)
        braw[nt] = *reinterpret_cast<const uint4*>(&s_b[buf][b_base + nt * 32 * kRowB + 32 * c]);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        v4i_t a[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          a[mt] = *reinterpret_cast<const v4i_t*>(
              &s_a[buf][a_base + mt * 32 * kRowA + 64 * c + 16 * s]);
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) {
          // (w ^ c) & m is one three-input bit operation; the shifted form folds the shift of
          // the constant: ((w ^ 0x88888888) << 4) & m == ((w << 4) ^ 0x80808080) & m
          const uint32_t w0 = s == 0 ? braw[nt].x : braw[nt].z;
          const uint32_t w1 = s == 0 ? braw[nt].y : braw[nt].w;
          v4i_t b;
          b[0] = (int)(((w0 << 4) ^ 0x80808080u) & 0xF0F0F0F0u);
          b[1] = (int)((w0 ^ 0x88888888u) & 0xF0F0F0F0u);
          b[2] = (int)(((w1 << 4) ^ 0x80808080u) & 0xF0F0F0F0u);
          b[3] = (int)((w1 ^ 0x88888888u) & 0xF0F0F0F0u);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                a[mt], b, (opens_static && s == 0) ? zero : acc[mt][nt], 0, 0, 0);
        }
      }
      if (closes) {
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) {
          const float ws =
              s_s[buf][wn * 32 * WN + nt * 32 + frag_row][GSH ? c / kChunksPerGroup : 0];
          // an fp16 scale / 16 is always exact in f32; an f32 scale below 2^-122 may not be
          const float ws16 = ws * 0.0625f;
          const bool exact = sizeof(ST) == 2 || __all(ws16 * 16.0f == ws);
          const float mult = valid ? (exact ? ws16 : ws) : 0.f;  // past K: accf + 0 * 0
          const int down = exact ? 0 : 4;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int32_t sum = sizeof(ST) == 2 ? acc[mt][nt][r] : acc[mt][nt][r] >> down;
              accf[mt][nt][r] = fmaf((float)sum, mult, accf[mt][nt][r]);
            }
        }
      }
    }
    park_stage(stage + 1, buf ^ 1, staged);
    __syncthreads();
  };
  for (uint32_t stage = 0; stage < stages; stage += 2) {
    run_stage(stage, 0);
    run_stage(stage + 1, 1);  // past the last stage: zeros, fused with a zero scale
  }

#pragma unroll
  for (int nt = 0; nt < WN; ++nt) {
    const uint32_t col = n0 + wn * 32 * WN + nt * 32 + frag_row;
    const float b = (bias && col < n) ? bias[col] : 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const uint32_t row = m0 + wm * 32 * MT + mt * 32 + 8 * (r / 4) + 4 * frag_h + (r % 4);
        if (row < m && col < n) out[(size_t)row * n + col] = fmaf(accf[mt][nt][r], xs[row], b);
      }
  }
}

// The same staging with a 128 x 256 workgroup tile, wave = 64 x 64, for groups of 64 or 128
// codes.  Four 32 x 32 tiles per wave would need 64 int32 and 64 f32 accumulators at once, more
// than two waves per SIMD leave room for, so the work is ordered by group: the group's weight
// words are expanded once (both column tiles, all MFMA steps of the group), then each row tile
// in turn runs its two MFMA chains over the group and is fused into its f32 accumulators — 32
// int32 accumulators live at a time, and the expansion is shared by the two row tiles.
template <typename ST, int GSH>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void linear_w4a8_tall_kernel(
    const uint8_t* __restrict__ xq, const float* __restrict__ xs, const uint8_t* __restrict__ w,
    const ST* __restrict__ scales, const float* __restrict__ bias, float* __restrict__ out,
    uint32_t m, uint32_t n, uint32_t k, uint32_t m_blocks, uint32_t n_blocks) {
  static_assert(GSH == 6 || GSH == 7, "groups of 64 or 128 codes");
  constexpr int MT = 2, WN = 2;
  constexpr int BM = 128, BN = 256;
  constexpr int kStage = 128;                          // codes per LDS stage
  constexpr int kRowA = kStage + 16, kRowB = kStage / 2 + 16;
  constexpr int kGroupsPerStage = kStage >> GSH;       // 2 or 1
  constexpr int kStepsPerGroup = 1 << (GSH - 5);       // MFMA steps of 32 codes: 2 or 4
  constexpr int kAUnits = BM * (kStage / 16) / 512;    // 16-byte units of xq per thread: 2
  constexpr int kBUnits = BN * (kStage / 32) / 512;    // and of packed weights: 2
  __shared__ __align__(16) uint8_t s_a[2][BM * kRowA];
  __shared__ __align__(16) uint8_t s_b[2][BN * kRowB];
  __shared__ __align__(16) float s_s[2][BN][2];

  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
  const uint32_t mb = slot % m_blocks, nb = (slot / m_blocks) * 8u + xcd;
  if (nb >= n_blocks) return;  // the whole workgroup leaves before any barrier
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  const int frag_row = lane & 31, frag_h = lane >> 5;
  const uint32_t m0 = mb * BM, n0 = nb * BN;
  const uint32_t groups = k >> GSH;
  const uint32_t chunks_total = k >> 6;
  const uint32_t stages = (k + kStage - 1) / kStage;

  // staging roles: xq rows in 8 units of 16 bytes (rows tid / 8 + 64 i), weight rows in 4
  // (rows tid / 4 + 128 i)
  const uint32_t arow0 = tid >> 3, aunit = (tid & 7u) * 16u;
  const uint32_t brow0 = tid >> 2, bunit = (tid & 3u) * 16u;
  const ST* ssrc = scales + (size_t)min(n0 + (uint32_t)(tid & 255), n - 1) * groups;

  struct Staged {
    uint4 a[kAUnits];
    uint4 b[kBUnits];
    ST s[kGroupsPerStage];
  };
  auto load_stage = [&](uint32_t stage, Staged& d) {
    const uint32_t a_at = stage * kStage + aunit, b_at = stage * (kStage / 2) + bunit;
    const uint32_t a_off = a_at < k ? a_at : 0u, b_off = b_at < (k >> 1) ? b_at : 0u;
#pragma unroll
    for (int i = 0; i < kAUnits; ++i)
      d.a[i] = *reinterpret_cast<const uint4*>(
          xq + (size_t)min(m0 + arow0 + 64u * i, m - 1) * k + a_off);
#pragma unroll
    for (int i = 0; i < kBUnits; ++i)
      d.b[i] = *reinterpret_cast<const uint4*>(
          w + (size_t)min(n0 + brow0 + 128u * i, n - 1) * (k >> 1) + b_off);
#pragma unroll
    for (int j = 0; j < kGroupsPerStage; ++j) {
      const uint32_t code = stage * kStage + (j << GSH);
      d.s[j] = ssrc[(code < k ? code : 0u) >> GSH];
    }
  };
  auto park_stage = [&](uint32_t stage, int buf, const Staged& d) {
    const uint32_t keep = stage * kStage + aunit < k ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int i = 0; i < kAUnits; ++i) {
      uint4 v;
      v.x = __builtin_amdgcn_perm(d.a[i].y, d.a[i].x, 0x06040200u) & keep;
      v.y = __builtin_amdgcn_perm(d.a[i].y, d.a[i].x, 0x07050301u) & keep;
      v.z = __builtin_amdgcn_perm(d.a[i].w, d.a[i].z, 0x06040200u) & keep;
      v.w = __builtin_amdgcn_perm(d.a[i].w, d.a[i].z, 0x07050301u) & keep;
      *reinterpret_cast<uint4*>(&s_a[buf][(arow0 + 64u * i) * kRowA + aunit]) = v;
    }
#pragma unroll
    for (int i = 0; i < kBUnits; ++i)
      *reinterpret_cast<uint4*>(&s_b[buf][(brow0 + 128u * i) * kRowB + bunit]) = d.b[i];
    if (tid < 256) {
#pragma unroll
      for (int j = 0; j < kGroupsPerStage; ++j) s_s[buf][tid][j] = scale_f32<ST>(&d.s[j], 0);
    }
  };

  float accf[MT][WN][16];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < WN; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) accf[mt][nt][r] = 0.f;
  const v16i_t zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  Staged staged;
  load_stage(0, staged);
  park_stage(0, 0, staged);
  __syncthreads();

  const uint32_t a_base = (uint32_t)((wm * 64 + frag_row) * kRowA + 32 * frag_h);
  const uint32_t b_base = (uint32_t)((wn * 64 + frag_row) * kRowB + 16 * frag_h);
  auto run_stage = [&](uint32_t stage, int buf) {
    load_stage(stage + 1, staged);
    __builtin_amdgcn_sched_barrier(0);  // the requests stay a stage ahead of their use
#pragma unroll
    for (int gi = 0; gi < kGroupsPerStage; ++gi) {
      // codes 0 .. (1 << GSH) - 1 of the group = MFMA steps 0 .. kStepsPerGroup - 1;
      // step st lies in chunk (gi << GSH) / 64 + st / 2, half st % 2
      const int first_chunk_in_stage = (gi << GSH) >> 6;
      const bool valid = stage * 2u + first_chunk_in_stage < chunks_total;
      v4i_t bexp[WN][kStepsPerGroup];
      float mult[WN];
#pragma unroll
      for (int nt = 0; nt < WN; ++nt) {
#pragma unroll
        for (int cc = 0; cc < kStepsPerGroup / 2; ++cc) {
          const uint4 braw = *reinterpret_cast<const uint4*>(
              &s_b[buf][b_base + nt * 32 * kRowB + 32 * (first_chunk_in_stage + cc)]);
          const uint32_t words[4] = {braw.x, braw.y, braw.z, braw.w};
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            v4i_t b;
            b[0] = (int)(((words[2 * s] << 4) ^ 0x80808080u) & 0xF0F0F0F0u);
            b[1] = (int)((words[2 * s] ^ 0x88888888u) & 0xF0F0F0F0u);
            b[2] = (int)(((words[2 * s + 1] << 4) ^ 0x80808080u) & 0xF0F0F0F0u);
            b[3] = (int)((words[2 * s + 1] ^ 0x88888888u) & 0xF0F0F0F0u);
            bexp[nt][2 * cc + s] = b;
          }
        }
        const float ws = s_s[buf][wn * 64 + nt * 32 + frag_row][gi];
        // an fp16 scale / 16 is exact in f32; an f32 scale may not be (subnormal quotient):
        // then the sums are shifted instead (below)
        mult[nt] = valid ? ws : 0.f;  // past K: accf + 0 * 0
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        v16i_t acc[WN];
#pragma unroll
        for (int st = 0; st < kStepsPerGroup; ++st) {
          const v4i_t a = *reinterpret_cast<const v4i_t*>(
              &s_a[buf][a_base + mt * 32 * kRowA + 64 * (first_chunk_in_stage + st / 2) +
                        16 * (st & 1)]);
#pragma unroll
          for (int nt = 0; nt < WN; ++nt)
            acc[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bexp[nt][st],
                                                            st == 0 ? zero : acc[nt], 0, 0, 0);
        }
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) {
          const float ws16 = mult[nt] * 0.0625f;
          const bool exact = sizeof(ST) == 2 || __all(ws16 * 16.0f == mult[nt]);
          const float factor = exact ? ws16 : mult[nt];
          const int down = exact ? 0 : 4;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int32_t sum = sizeof(ST) == 2 ? acc[nt][r] : acc[nt][r] >> down;
            accf[mt][nt][r] = fmaf((float)sum, factor, accf[mt][nt][r]);
          }
        }
      }
    }
    park_stage(stage + 1, buf ^ 1, staged);
    __syncthreads();
  };
  for (uint32_t stage = 0; stage < stages; ++stage) run_stage(stage, (int)(stage & 1u));

#pragma unroll
  for (int nt = 0; nt < WN; ++nt) {
    const uint32_t col = n0 + wn * 64 + nt * 32 + frag_row;
    const float b = (bias && col < n) ? bias[col] : 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const uint32_t row = m0 + wm * 64 + mt * 32 + 8 * (r / 4) + 4 * frag_h + (r % 4);
        if (row < m && col < n) out[(size_t)row * n + col] = fmaf(accf[mt][nt][r], xs[row], b);
      }
  }
}

template <typename ST>
int32_t launch_w4a8(krm_ctx* ctx, krm_buf xq, krm_buf xs, krm_buf w, krm_buf scales,
                    krm_buf bias, krm_buf out, uint32_t m, uint32_t n, uint32_t k,
                    uint32_t group) {
  const uint32_t* pxq = ptr<const uint32_t>(xq);
  const float* pxs = ptr<const float>(xs);
  const uint32_t* pw = ptr<const uint32_t>(w);
  const ST* ps = ptr<const ST>(scales);
  const float* pb = ptr<const float>(bias);
  float* po = ptr<float>(out);
  uint32_t shift = 0;
  while ((1u << shift) < group) ++shift;
  const bool rows_form = group >= 32 && group <= 2048 && m <= 8 && aligned(xq, 16) &&
                         aligned(w, 16);
  if (rows_form) {
    const dim3 grid((n + 7) / 8, m <= 1 ? 1 : m <= 2 ? 1 : (m + 3) / 4);
    if (m <= 1)
      hipLaunchKernelGGL((linear_w4a8_rows_kernel<ST, 1, 0>), grid, dim3(256), 0, ctx->stream, pxq,
                         pxs, pw, ps, pb, po, m, n, k, shift);
    else if (m <= 2)
      hipLaunchKernelGGL((linear_w4a8_rows_kernel<ST, 2, 0>), grid, dim3(256), 0, ctx->stream, pxq,
                         pxs, pw, ps, pb, po, m, n, k, shift);
    else
      hipLaunchKernelGGL((linear_w4a8_rows_kernel<ST, 4, 0>), grid, dim3(256), 0, ctx->stream, pxq,
                         pxs, pw, ps, pb, po, m, n, k, shift);
    return launched(ctx, "linear_w4a8_rows_kernel");
  }
  if (m > 8 && group >= 64 && group <= kMaxGroupTimes16 && aligned(xq, 16) && aligned(w, 16)) {
    const uint32_t n_blocks = (n + 255) / 256;
    // 128-row tiles for groups of 64 / 128 when they still cover most of the chip
    const uint32_t tall_blocks = (m + 127) / 128;
    if ((shift == 6 || shift == 7) &&
        (uint64_t)tall_blocks * n_blocks * 5 >= (uint64_t)ctx->num_cus * 3) {
      const uint64_t blocks = (uint64_t)((n_blocks + 7) / 8) * 8u * tall_blocks;
      if (blocks <= 0x7fffffffull) {
        if (shift == 6)
          hipLaunchKernelGGL((linear_w4a8_tall_kernel<ST, 6>), dim3((uint32_t)blocks), dim3(512),
                             0, ctx->stream, ptr<const uint8_t>(xq), pxs, ptr<const uint8_t>(w),
                             ps, pb, po, m, n, k, tall_blocks, n_blocks);
        else
          hipLaunchKernelGGL((linear_w4a8_tall_kernel<ST, 7>), dim3((uint32_t)blocks), dim3(512),
                             0, ctx->stream, ptr<const uint8_t>(xq), pxs, ptr<const uint8_t>(w),
                             ps, pb, po, m, n, k, tall_blocks, n_blocks);
        return launched(ctx, "linear_w4a8_tall_kernel");
      }
    }
    const uint32_t m_blocks = (m + 63) / 64;
    // 64 x 256 tiles, or 64 x 128 when those would leave a quarter of the chip without work
    const bool narrow = (uint64_t)m_blocks * n_blocks * 4 < (uint64_t)ctx->num_cus * 3;
    const uint32_t nb = narrow ? (n + 127) / 128 : n_blocks;
    const uint64_t blocks = (uint64_t)((nb + 7) / 8) * 8u * m_blocks;
    if (blocks <= 0x7fffffffull) {
#define KRM_W4A8_TILE(GSH, WN)                                                                 \
  hipLaunchKernelGGL((linear_w4a8_tile_kernel<ST, GSH, 1, WN>), dim3((uint32_t)blocks),        \
                     dim3(512), 0, ctx->stream, ptr<const uint8_t>(xq), pxs,                  \
                     ptr<const uint8_t>(w), ps, pb, po, m, n, k, shift, m_blocks, nb)
#define KRM_W4A8_TILE_G(GSH) \
  do { if (narrow) KRM_W4A8_TILE(GSH, 1); else KRM_W4A8_TILE(GSH, 2); } while (0)
      if (shift == 6) KRM_W4A8_TILE_G(6);
      else if (shift == 7) KRM_W4A8_TILE_G(7);
      else if (shift == 8) KRM_W4A8_TILE_G(8);
      else KRM_W4A8_TILE_G(0);
#undef KRM_W4A8_TILE_G
#undef KRM_W4A8_TILE
      return launched(ctx, "linear_w4a8_tile_kernel");
    }
  }
  const dim3 grid((n + 3) / 4, m < 65535u ? m : 65535u);
  hipLaunchKernelGGL((linear_w4a8_generic_kernel<ST>), grid, dim3(256), 0, ctx->stream, pxq, pxs,
                     pw, ps, pb, po, m, n, k, group);
  return launched(ctx, "linear_w4a8_generic_kernel");
}

// The quantiser inside the product's launch; false when the shape is not covered.
template <typename ST>
bool launch_w4a8_fused(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                       krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group) {
  uint32_t shift = 0;
  while ((1u << shift) < group) ++shift;
  const uint32_t block = m <= 1 ? 1u : m <= 2 ? 2u : 4u;
  if (!(group >= 32 && group <= 2048 && m <= 8 && aligned(x, 16) && aligned(w, 16) &&
        (uint64_t)block * k <= 256ull * 4 * kFuseCache))
    return false;
  const dim3 grid((n + 7) / 8, (m + block - 1) / block);
  const size_t lds = (size_t)block * k;
  const void* px = ptr<const void>(x);
  const uint32_t* pw = ptr<const uint32_t>(w);
  const ST* ps = ptr<const ST>(scales);
  const float* pb = ptr<const float>(bias);
  float* po = ptr<float>(out);
  const uint32_t per_thread = (uint32_t)(((uint64_t)block * k / 4 + 255) / 256);
#define KRM_W4A8_FUSED(MB, FUSE)                                                               \
  hipLaunchKernelGGL((linear_w4a8_rows_kernel<ST, MB, FUSE>), grid, dim3(256), lds,            \
                     ctx->stream, px, nullptr, pw, ps, pb, po, m, n, k, shift)
#define KRM_W4A8_FUSED_MB(MB)                      \
  do {                                             \
    if (per_thread <= 4) KRM_W4A8_FUSED(MB, 4);    \
    else if (per_thread <= 8) KRM_W4A8_FUSED(MB, 8); \
    else KRM_W4A8_FUSED(MB, 16);                   \
  } while (0)
  if (block == 1) KRM_W4A8_FUSED_MB(1);
  else if (block == 2) KRM_W4A8_FUSED_MB(2);
  else KRM_W4A8_FUSED_MB(4);
#undef KRM_W4A8_FUSED_MB
#undef KRM_W4A8_FUSED
  return true;
}

}  // namespace

extern "C" int32_t krm_quantize_rows(krm_ctx* ctx, krm_buf x, krm_buf xq, krm_buf xs,
                                     uint32_t rows, uint32_t dim) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, dim >= 1, "quantize_rows: dim must be positive (%u)", dim);
  KRM_REQUIRE(ctx, dim % 4 == 0, "quantize_rows: dim must be a multiple of 4 (%u)", dim);
  if (rows == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && xq && xs, "quantize_rows: null buffer");
  KRM_REQUIRE(ctx, aligned(x, 16) && aligned(xq, 4) && aligned(xs, 4),
              "quantize_rows: x needs 16-byte, xq and xs 4-byte alignment");
  const uint32_t blocks = rows < (1u << 16) ? rows : (1u << 16);
  hipLaunchKernelGGL(quantize_rows_kernel, dim3(blocks), dim3(256), 0, ctx->stream,
                     krm::ptr<const float>(x), krm::ptr<uint32_t>(xq), krm::ptr<float>(xs), rows,
                     dim);
  return krm::launched(ctx, "quantize_rows_kernel");
}

extern "C" int32_t krm_linear_w4a8(krm_ctx* ctx, krm_buf xq, krm_buf xs, krm_buf w,
                                   krm_buf scales, krm_buf bias, krm_buf out, uint32_t m,
                                   uint32_t n, uint32_t k, uint32_t group, int32_t scale_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, krm::valid_dtype(scale_dtype), "linear w4a8: unknown scale dtype %d",
              scale_dtype);
  KRM_REQUIRE(ctx, k > 0 && k % 4 == 0, "linear w4a8: k must be a positive multiple of 4 (%u)", k);
  KRM_REQUIRE(ctx, krm::is_pow2(group) && group >= 16,
              "linear w4a8: group_size %u is not a power of two >= 16", group);
  KRM_REQUIRE(ctx, k % group == 0, "linear w4a8: k=%u is not a multiple of group_size %u", k,
              group);
  KRM_REQUIRE(ctx, group <= kMaxGroup,
              "linear w4a8: group_size %u exceeds the int32 reduction limit %u", group, kMaxGroup);
  if (m == 0 || n == 0) return KRM_OK;
  KRM_REQUIRE(ctx, xq && xs && w && scales && out, "linear w4a8: null buffer");
  KRM_REQUIRE(ctx, krm::aligned(xq, 4) && krm::aligned(xs, 4) && krm::aligned(w, 4) &&
                       krm::aligned(out, 4) && krm::aligned(bias, 4) &&
                       krm::aligned(scales, krm::dtype_bytes(scale_dtype)),
              "linear w4a8: misaligned buffer");
  if (scale_dtype == KRM_F16)
    return launch_w4a8<__half>(ctx, xq, xs, w, scales, bias, out, m, n, k, group);
  return launch_w4a8<float>(ctx, xq, xs, w, scales, bias, out, m, n, k, group);
}

extern "C" int32_t krm_linear_w4a8_fused(krm_ctx* ctx, krm_buf x, krm_buf xq, krm_buf xs,
                                         krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                                         uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                                         int32_t scale_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, krm::valid_dtype(scale_dtype), "linear w4a8: unknown scale dtype %d",
              scale_dtype);
  KRM_REQUIRE(ctx, k > 0 && k % 4 == 0, "linear w4a8: k must be a positive multiple of 4 (%u)", k);
  KRM_REQUIRE(ctx, krm::is_pow2(group) && group >= 16,
              "linear w4a8: group_size %u is not a power of two >= 16", group);
  KRM_REQUIRE(ctx, k % group == 0, "linear w4a8: k=%u is not a multiple of group_size %u", k,
              group);
  KRM_REQUIRE(ctx, group <= kMaxGroup,
              "linear w4a8: group_size %u exceeds the int32 reduction limit %u", group, kMaxGroup);
  if (m == 0 || n == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && w && scales && out, "linear w4a8: null buffer");
  KRM_REQUIRE(ctx, krm::aligned(x, 16) && krm::aligned(w, 4) && krm::aligned(out, 4) &&
                       krm::aligned(bias, 4) &&
                       krm::aligned(scales, krm::dtype_bytes(scale_dtype)),
              "linear w4a8: misaligned buffer");
  const bool fused = scale_dtype == KRM_F16
                         ? launch_w4a8_fused<__half>(ctx, x, w, scales, bias, out, m, n, k, group)
                         : launch_w4a8_fused<float>(ctx, x, w, scales, bias, out, m, n, k, group);
  if (fused) return krm::launched(ctx, "linear_w4a8_rows_kernel");
  KRM_REQUIRE(ctx, xq && xs,
              "linear w4a8 (fused): this shape (m=%u, k=%u, group=%u) takes the two-launch form, "
              "which needs the xq and xs work buffers",
              m, k, group);
  KRM_TRY(krm_quantize_rows(ctx, x, xq, xs, m, k));
  return krm_linear_w4a8(ctx, xq, xs, w, scales, bias, out, m, n, k, group, scale_dtype);
}
