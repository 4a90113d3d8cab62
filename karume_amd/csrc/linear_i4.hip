// int4 group-quantised `linear` for gfx950: the dequant kernel (bit-exact gate) and the
// bandwidth-bound GEMV used for M <= 16 rows of activations.
//
// Semantics follow the reference's linear op with i4 weights
// (packages/runtime/src/kernels/linear.ts:34-64, body packages/runtime/src/kernels/gemm.ts:
// 1187-1237, dequant packages/runtime/src/kernels/weight-storage.ts:152-187): weights are
// packed [N, K] with K contiguous, 8 elements per little-endian u32 (element 8w+j at bits
// 4j), stored u = q + 8, one scale per `group` consecutive K elements of a row.
//
// The reference runs M = 1 through a 16x16-tile f32 GEMM with a strictly K-ascending
// accumulation.  Here a wave owns whole output rows instead: every lane streams 16 bytes
// (32 codes) of a row per step, accumulates sum((u-8)*x) for its 32 codes in f32, applies the
// group scale to that partial sum, and the 64 lane sums are added with a fixed DPP tree.  The
// reduction order therefore differs from the reference's (results agree within a stated
// tolerance, not bitwise) but depends on (K, group) only — never on M, N or the launch — so a
// row of x gives the same bits whether it is run alone or in a batch.
#include "krm_internal.h"

#include <cmath>

using namespace krm;

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// ------------------------------------------------------------------------------------ dequant

template <typename ST>
__device__ inline float load_scale(const ST* s, size_t i);
template <>
__device__ inline float load_scale<float>(const float* s, size_t i) { return s[i]; }
template <>
__device__ inline float load_scale<__half>(const __half* s, size_t i) {
  return __half2float(s[i]);
}

// Weights are read once per launch and not again before everything else a decode step touches
// has passed through the caches: they are requested non-temporally (`nt`:
// streamed through the L2, not kept in the memory-side cache), which leaves the Infinity Cache
// to what IS read again soon — activations, KV rows, lengths.  Measured on the 1.1B-shape
// decoder: 2020 -> 2144 tokens/s; the 128 MiB streaming GEMV 71 -> 74 % of the HBM peak.
// The scales stay ordinary loads: a line of them serves several lanes and rows, and streamed
// lines are dropped early (the streaming GEMV fell back to 70 % with them).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ inline uint4 stream_u128(const void* p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ inline uint32_t stream_u32(const uint32_t* p) { return __builtin_nontemporal_load(p); }


// One thread expands one u32 (8 codes).  f32(u - 8) * scale is a single rounded f32 multiply.
template <typename ST>
__global__ __launch_bounds__(256) void dequant_i4_kernel(const uint32_t* __restrict__ w,
                                                         const ST* __restrict__ scales,
                                                         float* __restrict__ out, size_t words,
                                                         size_t width, uint32_t group) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t groups = width / group;
  for (size_t wi = blockIdx.x * (size_t)blockDim.x + threadIdx.x; wi < words; wi += stride) {
    const uint32_t word = w[wi];
    const size_t i0 = wi * 8;
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const size_t i = i0 + j;
      const size_t row = i / width;
      const size_t g = (i - row * width) / group;
      const int code = (int)((word >> (4 * j)) & 0xFu) - 8;
      v[j] = __fmul_rn((float)code, load_scale<ST>(scales, row * groups + g));
    }
    float4* dst = reinterpret_cast<float4*>(out + i0);
    dst[0] = make_float4(v[0], v[1], v[2], v[3]);
    dst[1] = make_float4(v[4], v[5], v[6], v[7]);
  }
}

// ------------------------------------------------------------------------------------ GEMV

// Sums over the 64 lanes of a wave.  One fixed order of additions for every form, so a row's
// bits do not depend on how many rows its wave reduces: partner lane ^ 1, lane ^ 2 (quad
// permutes), then the quads of a 16-lane row (rotate by 4, by 8), the rows 16 apart (swizzle) and
// the halves 32 apart; the value of lane 0 (or of lane r for row r) is the result.
template <int CTRL>
__device__ inline float dpp_from(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// levels 3..6: every lane adds lanes at the same position mod 4
__device__ inline float wave_sum_tail(float v) {
  v += dpp_from<0x124>(v);  // row_ror:4
  v += dpp_from<0x128>(v);  // row_ror:8
  v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
  v += __shfl_xor(v, 32, kWave);
  return v;
}
__device__ inline float lane_value(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
// every lane returns the total
__device__ inline float wave_sum(float v) {
  v += dpp_from<0xB1>(v);  // quad_perm [1,0,3,2]
  v += dpp_from<0x4E>(v);  // quad_perm [2,3,0,1]
  v += dpp_from<0x124>(v);
  v += dpp_from<0x128>(v);
  // the last two levels through scalar registers: the same pairs as wave_sum_tail
  return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}
// Two and four sums at once: after the first level a lane keeps one of two values, after the
// second one of four, so the later levels run once.  Lane r ends with the total of value r.
__device__ inline float wave_sum2(float a, float b, int lane) {
  const bool odd = lane & 1;
  float p = (odd ? b : a) + dpp_from<0xB1>(odd ? a : b);
  p += dpp_from<0x4E>(p);
  return wave_sum_tail(p);
}
__device__ inline float wave_sum4(float a, float b, float c, float d, int lane) {
  const bool odd = lane & 1, high = lane & 2;
  const float p0 = (odd ? b : a) + dpp_from<0xB1>(odd ? a : b);  // even lanes: a, odd lanes: b
  const float p1 = (odd ? d : c) + dpp_from<0xB1>(odd ? c : d);  // even lanes: c, odd lanes: d
  const float q = (high ? p1 : p0) + dpp_from<0x4E>(high ? p0 : p1);
  return wave_sum_tail(q);
}

// Eight codes of one u32 as four fp16 pairs holding the exact integers (u - 8):
// pair i = (code i, code i+4).  1024 + u is built in the fp16 mantissa, then the offset is
// removed with one packed op; codes in the upper nibble of a byte arrive as 1024 + 16u.
// (a & mask) | bits in one VALU op: the compiler splits it in two when both constants are
// literals, because this ISA's three-operand encodings take no literal.
__device__ inline uint32_t and_or(uint32_t a, uint32_t mask, uint32_t bits) {
  uint32_t d;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask), "v"(bits));
  return d;
}

__device__ inline void codes_to_half2(uint32_t word, half2_t (&q)[4]) {
  const uint32_t magic = 0x64006400u;  // (1024.0, 1024.0)
  const half2_t off_lo = {(_Float16)1032.0f, (_Float16)1032.0f};
  const half2_t sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  const half2_t off_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
  const uint32_t upper = word >> 8;
  q[0] = __builtin_bit_cast(half2_t, and_or(word, 0x000F000Fu, magic)) - off_lo;
  q[1] = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, and_or(word, 0x00F000F0u, magic)),
                                   sixteenth, off_hi);
  q[2] = __builtin_bit_cast(half2_t, and_or(upper, 0x000F000Fu, magic)) - off_lo;
  q[3] = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, and_or(upper, 0x00F000F0u, magic)),
                                   sixteenth, off_hi);
}

// Eight consecutive fp16 activations (x0..x7 in four dwords) regrouped to match
// codes_to_half2: pair i = (x_i, x_{i+4}).
__device__ inline void pair_activations(const uint4& raw, half2_t (&p)[4]) {
  p[0] = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(raw.z, raw.x, 0x05040100u));
  p[1] = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(raw.z, raw.x, 0x07060302u));
  p[2] = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(raw.w, raw.y, 0x05040100u));
  p[3] = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(raw.w, raw.y, 0x07060302u));
}

template <typename XT>
struct Acts;  // per-lane activations of one x row for one step (VEC words = VEC*8 elements)

// fp16 activations: exact fp16 products, f32 accumulation through v_dot2_f32_f16.
template <>
struct Acts<__half> {
  template <int VEC>
  struct Regs {
    half2_t p[VEC][4];
  };
  // `g` (optional): rms_norm weights of the same 8*VEC positions; the lane then carries
  // fp16(x * g) and adds its x^2 to `squares`.
  // The loads of `load` alone (see Acts<float>::Raw).
  template <int VEC, bool NORM>
  struct Raw {
    uint4 x[VEC];
    float4 g[NORM ? VEC : 1][2];
  };
  template <int VEC, bool NORM>
  __device__ static inline void request(const __half* x, const float* g, Raw<VEC, NORM>& raw) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      raw.x[j] = reinterpret_cast<const uint4*>(x)[j];
      if constexpr (NORM) {
        raw.g[j][0] = reinterpret_cast<const float4*>(g)[2 * j];
        raw.g[j][1] = reinterpret_cast<const float4*>(g)[2 * j + 1];
      }
    }
  }
  template <int VEC, bool NORM>
  __device__ static inline void load(const __half* x, const float* g, bool active, Regs<VEC>& r,
                                     float& squares) {
    Raw<VEC, NORM> raw;
    request<VEC, NORM>(x, g, raw);
    finish<VEC, NORM>(raw, active, r, squares);
  }
  template <int VEC, bool NORM>
  __device__ static inline void finish(const Raw<VEC, NORM>& in, bool active, Regs<VEC>& r,
                                       float& squares) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      uint4 raw = in.x[j];
      if constexpr (NORM) {
        const uint32_t keep = active ? 0xFFFFFFFFu : 0u;  // x^2 of a lane past K must be 0
        raw.x &= keep; raw.y &= keep; raw.z &= keep; raw.w &= keep;
        const float4 ga = in.g[j][0];
        const float4 gb = in.g[j][1];
        const float gw[8] = {ga.x, ga.y, ga.z, ga.w, gb.x, gb.y, gb.z, gb.w};
        uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const half2_t h = __builtin_bit_cast(half2_t, words[i]);
          const float lo = (float)h.x, hi = (float)h.y;
          squares = fmaf(lo, lo, squares);
          squares = fmaf(hi, hi, squares);
          const half2_t scaled = {(_Float16)(lo * gw[2 * i]), (_Float16)(hi * gw[2 * i + 1])};
          words[i] = __builtin_bit_cast(uint32_t, scaled);
        }
        raw = make_uint4(words[0], words[1], words[2], words[3]);
      }
      pair_activations(raw, r.p[j]);
    }
  }
  // sum over the lane's VEC*8 codes of (u - 8) * x
  template <int VEC>
  __device__ static inline float dot(const uint32_t (&words)[VEC], const Regs<VEC>& r) {
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      half2_t q[4];
      codes_to_half2(words[j], q);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2(q[i], r.p[j][i], acc, false);
    }
    return acc;
  }
};

// f32 activations: f32 products.  The codes become exact fp16 integers (u - 8) as above and
// each one feeds a mixed-precision fma (fp16 * f32 + f32, the product is exact in f32).
template <>
struct Acts<float> {
  template <int VEC>
  struct Regs {
    float v[VEC][8];
  };
  // The loads of `load` alone (activations, then norm weights), so that a caller can put other
  // requests between them and their first use.
  template <int VEC, bool NORM>
  struct Raw {
    uint4 x[VEC][2];
    float4 g[NORM ? VEC : 1][2];
  };
  template <int VEC, bool NORM>
  __device__ static inline void request(const float* x, const float* g, Raw<VEC, NORM>& raw) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      raw.x[j][0] = reinterpret_cast<const uint4*>(x)[2 * j];
      raw.x[j][1] = reinterpret_cast<const uint4*>(x)[2 * j + 1];
      if constexpr (NORM) {
        raw.g[j][0] = reinterpret_cast<const float4*>(g)[2 * j];
        raw.g[j][1] = reinterpret_cast<const float4*>(g)[2 * j + 1];
      }
    }
  }
  template <int VEC, bool NORM>
  __device__ static inline void load(const float* x, const float* g, bool active, Regs<VEC>& r,
                                     float& squares) {
    Raw<VEC, NORM> raw;
    request<VEC, NORM>(x, g, raw);
    finish<VEC, NORM>(raw, active, r, squares);
  }
  template <int VEC, bool NORM>
  __device__ static inline void finish(const Raw<VEC, NORM>& raw, bool active, Regs<VEC>& r,
                                       float& squares) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const uint4 ua = raw.x[j][0], ub = raw.x[j][1];
      const uint32_t keep = (!NORM || active) ? 0xFFFFFFFFu : 0u;  // x^2 past K must be 0
      float4 a = make_float4(__uint_as_float(ua.x & keep), __uint_as_float(ua.y & keep),
                             __uint_as_float(ua.z & keep), __uint_as_float(ua.w & keep));
      float4 b = make_float4(__uint_as_float(ub.x & keep), __uint_as_float(ub.y & keep),
                             __uint_as_float(ub.z & keep), __uint_as_float(ub.w & keep));
      if constexpr (NORM) {
        const float4 ga = raw.g[j][0];
        const float4 gb = raw.g[j][1];
        squares = fmaf(a.x, a.x, squares); squares = fmaf(a.y, a.y, squares);
        squares = fmaf(a.z, a.z, squares); squares = fmaf(a.w, a.w, squares);
        squares = fmaf(b.x, b.x, squares); squares = fmaf(b.y, b.y, squares);
        squares = fmaf(b.z, b.z, squares); squares = fmaf(b.w, b.w, squares);
        a = make_float4(a.x * ga.x, a.y * ga.y, a.z * ga.z, a.w * ga.w);
        b = make_float4(b.x * gb.x, b.y * gb.y, b.z * gb.z, b.w * gb.w);
      }
      r.v[j][0] = a.x; r.v[j][1] = a.y; r.v[j][2] = a.z; r.v[j][3] = a.w;
      r.v[j][4] = b.x; r.v[j][5] = b.y; r.v[j][6] = b.z; r.v[j][7] = b.w;
    }
  }
  template <int VEC>
  __device__ static inline float dot(const uint32_t (&words)[VEC], const Regs<VEC>& r) {
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      half2_t q[4];  // pair i = codes (i, i + 4)
      codes_to_half2(words[j], q);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc = fmaf((float)q[i].x, r.v[j][i], acc);
        acc = fmaf((float)q[i].y, r.v[j][i + 4], acc);
      }
    }
    return acc;
  }
};

// ------------------------------------------------------------------ batched rows on MFMA
//
// 2 <= M <= 16 rows of fp16 activations: sixteen dot products per weight word on the VALU make
// the kernel above compute-bound (about 400 GB/s at M = 16).  Here the products run on
// v_mfma_f32_16x16x32_f16 and the VALU only dequantises: A = x (16 rows, rows past M repeat
// the last one and are dropped), B = W^T, where lane (n = lane % 16, g = lane / 16) holds eight
// codes of weight row n — one 32-bit word — as exact fp16 integers (u - 8), straight from the
// load, no LDS.  A workgroup owns 16 weight rows; its four waves split K in quarters and walk
// them in chunks of 256 codes.  Per chunk a lane loads the 16-byte pieces g and 4 + g of its
// row, so that the four lane groups of MFMA step s < 4 (word 4g + s) cover codes 0..127 of the
// chunk and steps 4..7 cover codes 128..255: each half lies inside one scale group (group >=
// 128), is accumulated on its own and multiplied by the f32 scale of the lane's row afterwards
// (the C layout keeps weight row n in lane % 16).  Products are exact, sums and scaling are
// f32: the same arithmetic class as the kernel above, in a different order.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

template <typename ST, int CHUNKS, int KW>
__global__ __launch_bounds__(KW * 64) void gemv_i4_mfma_kernel(
    const __half* __restrict__ x, const uint32_t* __restrict__ w, const ST* __restrict__ scales,
    const __half* __restrict__ bias, __half* __restrict__ out, uint32_t m, uint32_t n, uint32_t k,
    uint32_t group_shift) {
  constexpr int kChunk = 256;
  __shared__ float s_part[KW][4][kWave];  // [wave][register][lane]
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const uint32_t n0 = blockIdx.x * 16;
  const uint32_t wrow = min(n0 + r16, n - 1);  // rows past N re-read the last row, unused
  // This wave's share of K: an equal part with a compile-time chunk count, or (loop form) the
  // chunks of 256 codes dealt to the waves in order, the first k/256 % KW waves one more.
  uint32_t k_first, chunks;
  if constexpr (CHUNKS > 0) {
    k_first = wave * (k / KW);
    chunks = CHUNKS;
  } else {
    const uint32_t total = k / kChunk, base = total / KW, extra = total % KW;
    chunks = base + ((uint32_t)wave < extra ? 1u : 0u);
    k_first = (wave * base + ((uint32_t)wave < extra ? (uint32_t)wave : extra)) * kChunk;
    if (chunks == 0) k_first = 0;  // nothing to do: its (unused) requests stay inside the row
  }
  const uint32_t* wptr = w + (size_t)wrow * (k >> 3) + (k_first >> 3) + 4 * g;
  const ST* sptr = scales + (size_t)wrow * (k >> group_shift);

  struct Weights {
    uint4 words[2];   // pieces g and 4 + g of the row's 32 words
    float scale[2];   // scale of each half of the chunk for this lane's row
  };
  // Activations: lane (row r, group g) needs x[r][16-byte piece 4g + s] at step s — a gather
  // over 16 rows that the vector cache serves one row at a time.  So a wave first loads its
  // chunk of x coalesced (32 lanes x 16 bytes = one row's 512 bytes), pairs the values for
  // the nibble order and parks them in its own LDS strip, rows padded by 16 bytes so that
  // the gather is conflict-free there.  Only this wave touches the strip: no barrier.
  constexpr int kRowBytes = kChunk * 2 + 16;
  constexpr int kStripBytes = 16 * kRowBytes;
  __shared__ __attribute__((aligned(16))) unsigned char s_x[KW][CHUNKS == 1 ? 1 : 2][kStripBytes];
  struct Acts {
    uint4 piece[8];   // x pieces as loaded: rows 2j + lane / 32, piece lane % 32
  };
  auto fetch_w = [&](uint32_t chunk, Weights& c) {
    const uint32_t kc = chunk * kChunk;
    c.words[0] = *reinterpret_cast<const uint4*>(wptr + (kc >> 3));
    c.words[1] = *reinterpret_cast<const uint4*>(wptr + (kc >> 3) + 16);
    c.scale[0] = load_scale<ST>(sptr, (k_first + kc) >> group_shift);
    c.scale[1] = load_scale<ST>(sptr, (k_first + kc + 128) >> group_shift);
  };
  const int load_row = lane >> 5, load_piece = lane & 31;
  auto fetch_x = [&](uint32_t chunk, Acts& c) {
    const uint32_t kc = chunk * kChunk;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t row = min((uint32_t)(2 * j + load_row), m - 1);
      c.piece[j] =
          *reinterpret_cast<const uint4*>(x + (size_t)row * k + k_first + kc + 8 * load_piece);
    }
  };
  auto park_x = [&](const Acts& c, int strip) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      half2_t p[4];
      pair_activations(c.piece[j], p);
      const uint4 v = make_uint4(__builtin_bit_cast(uint32_t, p[0]), __builtin_bit_cast(uint32_t, p[1]),
                                 __builtin_bit_cast(uint32_t, p[2]), __builtin_bit_cast(uint32_t, p[3]));
      *reinterpret_cast<uint4*>(&s_x[wave][strip][(2 * j + load_row) * kRowBytes + 16 * load_piece]) = v;
    }
  };
  float4_t total = {0.f, 0.f, 0.f, 0.f};  // out[m = 4g + i][n = lane % 16] over this K quarter
  auto consume = [&](const Weights& c, int strip) {
    float4_t half_sum[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    half8_t a[8];
#pragma unroll
    for (int s = 0; s < 8; ++s)  // step s: word 4g + s (s < 4) or 16 + 4g + (s - 4)
      a[s] = *reinterpret_cast<const half8_t*>(
          &s_x[wave][strip][r16 * kRowBytes + 16 * ((s < 4 ? 4 * g + s : 16 + 4 * g + (s - 4)))]);
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const uint32_t word = s < 4 ? (&c.words[0].x)[s] : (&c.words[1].x)[s - 4];
      half2_t q[4];
      codes_to_half2(word, q);
      const half8_t b = {q[0].x, q[0].y, q[1].x, q[1].y, q[2].x, q[2].y, q[3].x, q[3].y};
      half_sum[s >> 2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[s], b, half_sum[s >> 2], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      total[i] = fmaf(half_sum[0][i], c.scale[0], total[i]);
      total[i] = fmaf(half_sum[1][i], c.scale[1], total[i]);
    }
  };
  if constexpr (CHUNKS > 0) {
    // The activations of the first two chunks are requested first: they come from the cache and
    // loads return in order, so they are parked while the wave's whole share of the weights
    // (requested next, the long trip) is still on its way.  Activations then run two chunks
    // ahead in registers and one ahead in LDS; fixed registers, no branches.
    Acts xa[2];
    fetch_x(0, xa[0]);
    if (CHUNKS > 1) fetch_x(1, xa[1]);
    Weights wq[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) fetch_w(c, wq[c]);
    __builtin_amdgcn_sched_barrier(0);
    park_x(xa[0], 0);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      if (c + 2 < CHUNKS) fetch_x(c + 2, xa[c & 1]);       // slot of the chunk parked last pass
      if (c + 1 < CHUNKS) park_x(xa[(c + 1) & 1], (c + 1) & 1);
      consume(wq[c], c & 1);
    }
  } else {
    // any chunk count: the next chunk's requests are out (unconditionally; the last pass asks
    // for its own chunk again) before this chunk is used
    Weights wq, wq_next;
    Acts xa, xa_next;
    fetch_x(0, xa);
    fetch_w(0, wq);
    for (uint32_t chunk = 0; chunk < chunks; ++chunk) {
      const uint32_t ahead = chunk + 1 < chunks ? chunk + 1 : chunk;
      fetch_x(ahead, xa_next);
      fetch_w(ahead, wq_next);
      park_x(xa, 0);
      consume(wq, 0);
      wq = wq_next;
      xa = xa_next;
    }
  }
  // the waves' shares of K, added in wave order
#pragma unroll
  for (int i = 0; i < 4; ++i) s_part[wave][i][lane] = total[i];
  __syncthreads();
  if (wave == 0) {
    const uint32_t col = n0 + r16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = s_part[0][i][lane];
#pragma unroll
      for (int q = 1; q < KW; ++q) v += s_part[q][i][lane];
      const uint32_t row = 4 * g + i;
      if (row < m && col < n) {
        if (bias) v += __half2float(bias[col]);
        out[(size_t)row * n + col] = __float2half_rn(v);
      }
    }
  }
}


template <typename T>
__device__ inline float to_f32(T v);
template <>
__device__ inline float to_f32<float>(float v) { return v; }
template <>
__device__ inline float to_f32<__half>(__half v) { return __half2float(v); }
template <typename T>
__device__ inline T from_f32(float v);
template <>
__device__ inline float from_f32<float>(float v) { return v; }
template <>
__device__ inline __half from_f32<__half>(float v) { return __float2half_rn(v); }

// Optional work fused around the dot products (all null / 0 = the plain linear op).
struct GemvFusion {
  const float* norm_weight;  // [K] rms_norm weight applied to x before the product
  float norm_eps;
  const void* residual;      // [M, N_out] added to the result (same element type as out)
  uint32_t pair_silu;        // rows (2i, 2i+1) = (gate_i, up_i): out[., i] = silu(gate) * up
  // Decode row of a fused [q; k; v] projection (positions != null; M = 1).  Rows (2i, 2i+1) of
  // the q and k sections hold dims (j, j + D/2) of one head, so the lane that finishes a pair
  // rotates it (half-split RoPE, two rounded products then the add, as rope_kernel does) and
  // writes it to its natural place in `out` ([H + 2*Hkv, D]); k pairs and the v rows (natural
  // order) are also appended to the state slots (same rule as state_append_kernel).
  const int32_t* positions;
  const float* cos_table;
  const float* sin_table;
  void* slot_k;
  void* slot_v;
  uint32_t* lengths;         // device {past, query, fault, ...} or null: `past` below
  uint32_t heads, kv_heads, depth, table_rows, capacity, window, past;
  uint32_t half_shift;       // log2(depth / 2) when that is a power of two, else 0xffffffff:
                             // the epilogue's index arithmetic is then shifts and masks instead
                             // of integer divisions (about 150 instructions behind the reductions)
  int32_t slot_f16;          // slot element type: 1 = fp16, 0 = f32
  // One row (M = 1), plain epilogue: every workgroup also writes the argmax of the outputs it
  // stored, {value bits, row index}, to argmax_partial[blockIdx.x] (a workgroup without a row:
  // {-inf, 0xffffffff}); the number of workgroups is reported through host_blocks.
  uint2* argmax_partial;
  uint32_t* host_blocks;     // host side only: where the launcher leaves its grid size
};

__device__ inline void slot_store(void* slot, int32_t is_f16, size_t i, float v) {
  if (is_f16)
    static_cast<__half*>(slot)[i] = __float2half_rn(v);
  else
    static_cast<float*>(slot)[i] = v;
}

// One wave = ROWS consecutive output rows over the whole K; a step covers 64 lanes x VEC
// words (VEC*8 codes per lane, all inside one scale group).
//  NSTEP > 0: K fits in NSTEP steps; every weight word, scale and (for MB == 1) activation of
//             the wave is requested before anything is consumed, so one memory round trip
//             covers the whole kernel.
//  NSTEP == 0: any K; the next step's weights, scales and activations are requested before
//             the current step is consumed.
// Both forms add the per-step partial sums in ascending step order, so they agree bitwise.
//  Shared activations (one row of f32 x, NSTEP > 0): every wave of the workgroup needs the
//  same x, which for f32 is four times the bytes of the two weight rows it meets; wave s
//  prepares step s once (norm weight applied) and parks it in LDS for the others, after all
//  weight requests are out.
template <typename XT, int MB, int NSTEP>
constexpr bool share_x_in_lds() {
  return MB == 1 && NSTEP > 0 && NSTEP <= 4;
}

// NORM and DECODE_ROW are compile-time so that the plain kernel carries neither their branches
// nor their registers (a run-time test at the top of the kernel cost the plain GEMV 8 %).
template <typename XT, typename ST, int MB, int ROWS, int VEC, int NSTEP, bool NORM, bool DECODE_ROW>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 4))) void gemv_i4_kernel(
    // Argument order: what the first addresses and the final store are made of comes first — the
    // leading 14 dwords of the arguments arrive in scalar registers with the wave
    // (kernel-argument preload), the rest through a load the kernel has to wait for.
    const XT* __restrict__ x, const uint32_t* __restrict__ w, const ST* __restrict__ scales,
    const float* __restrict__ norm_weight, XT* __restrict__ out, uint32_t n, uint32_t k,
    uint32_t group_shift, uint32_t m, const XT* __restrict__ bias, GemvFusion fuse) {
  constexpr int kLaneElems = VEC * 8;
  constexpr int kStepElems = kWave * kLaneElems;
  using Regs = typename Acts<XT>::template Regs<VEC>;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  constexpr bool XLDS = share_x_in_lds<XT, MB, NSTEP>();
  // Four waves a workgroup (the launch below).  A wave whose rows lie past N stays: it re-reads
  // the last row and stores nothing, so no branch stands between the kernel's entry and its
  // loads (an early exit made the pointer arguments wait for the row test).
  const uint32_t row0 = (blockIdx.x * 4u + wave) * ROWS;

  const uint32_t words_per_row = k >> 3;
  const uint32_t groups_per_row = k >> group_shift;

  const uint32_t* wrow[ROWS];
  const ST* srow[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const uint32_t row = min(row0 + r, n - 1);  // rows past N re-read the last row, unused
    wrow[r] = w + (size_t)row * words_per_row;
    srow[r] = scales + (size_t)row * groups_per_row;
  }

  float acc[ROWS][MB];
  float shared_squares = 0.f;  // XLDS: sum of x^2 over the whole row
  float squares[MB];  // sum of x^2 over the lane's share of K (fused rms_norm only)
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    squares[b] = 0.f;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r][b] = 0.f;
  }

  // Decode-row epilogue: the rotation's table entries and the run-time lengths of a recorded
  // step are requested early, so that they arrive with the weights instead of costing a round
  // trip of their own behind the reductions — but after the weight requests where the kernel
  // asks for those at once: the addresses of x and of the weights come from arguments that
  // arrive with the wave, these from arguments that have to be loaded first.
  float rope_cos[ROWS / 2 > 0 ? ROWS / 2 : 1][2], rope_sin[ROWS / 2 > 0 ? ROWS / 2 : 1][2];
  bool rope_in_table = false;
  uint32_t dev_past = 0, dev_query = 0;
  auto request_decode_row = [&]() {
    if constexpr (DECODE_ROW) {
      // The lengths and the position are asked for together and without a branch (a missing
      // lengths buffer reads x instead and is dropped): one wait for both, where a branch
      // around each made them two round trips in a row in front of the staging of x.
      const uint32_t* lengths_or_x =
          fuse.lengths ? fuse.lengths : reinterpret_cast<const uint32_t*>(x);
      const uint32_t word0 = lengths_or_x[0], word1 = lengths_or_x[1];
      const int32_t first_position = fuse.positions[0];
      dev_past = fuse.lengths ? word0 : 0u;
      dev_query = fuse.lengths ? word1 : 0u;
      const uint32_t half = fuse.depth >> 1;
      const uint32_t rope_pairs = (fuse.heads + fuse.kv_heads) * half;
      // (a table of one row is this step's row: no position to look it up by)
      const int32_t pos = fuse.table_rows == 1 ? 0 : first_position;
      rope_in_table = pos >= 0 && (uint32_t)pos < fuse.table_rows;
#pragma unroll
      for (int p = 0; p < ROWS / 2; ++p) {
        const uint32_t pair = (row0 >> 1) + p;
        const bool rotates = rope_in_table && pair < rope_pairs;
        const uint32_t j = fuse.half_shift != 0xffffffffu ? (pair & (half - 1u)) : pair % half;
        const size_t t = rotates ? (size_t)pos * fuse.depth + j : 0;
        rope_cos[p][0] = fuse.cos_table[t];
        rope_sin[p][0] = fuse.sin_table[t];
        rope_cos[p][1] = fuse.cos_table[rotates ? t + half : 0];
        rope_sin[p][1] = fuse.sin_table[rotates ? t + half : 0];
      }
    }
  };
  constexpr bool kRowAfterWeights = share_x_in_lds<XT, MB, NSTEP>() && VEC == 4;
  if constexpr (!kRowAfterWeights) request_decode_row();

  // Lanes past the end of K (last step of a K that is not a multiple of the step) read the
  // row's first words and activations instead and their partial sum is dropped, so every load
  // is unconditional and all of them can be in flight together.
  auto fetch = [&](uint32_t step, uint32_t (&dst_w)[ROWS][VEC], float (&dst_s)[ROWS]) {
    const uint32_t k0 = step * kStepElems + lane * kLaneElems;
    const bool active = k0 < k;
    const uint32_t kc = active ? k0 : 0u;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      if constexpr (VEC == 4) {
        const uint4 v = stream_u128(wrow[r] + (kc >> 3));
        dst_w[r][0] = v.x; dst_w[r][1] = v.y; dst_w[r][2] = v.z; dst_w[r][3] = v.w;
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) dst_w[r][j] = stream_u32(wrow[r] + (kc >> 3) + j);
      }
      dst_s[r] = load_scale<ST>(srow[r], kc >> group_shift);
    }
  };
  // `counted` = false: a repeated request whose values are not used (its x^2 must not be added)
  auto fetch_x = [&](uint32_t step, int b, Regs& regs, bool counted = true) {
    const uint32_t k0 = step * kStepElems + lane * kLaneElems;
    const uint32_t xrow = min((uint32_t)b, m - 1);  // rows past M re-read the last row, unused
    const uint32_t kc = k0 < k ? k0 : 0u;
    Acts<XT>::template load<VEC, NORM>(x + (size_t)xrow * k + kc, norm_weight + kc,
                                       k0 < k && counted, regs, squares[b]);
  };
  auto consume = [&](uint32_t step, const uint32_t (&cw)[ROWS][VEC], const float (&cs)[ROWS],
                     int b, const Regs& regs) {
    // bit mask, not a select: a select lets the compiler move the dot product behind a branch
    const uint32_t keep = step * kStepElems + lane * kLaneElems < k ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const float part = Acts<XT>::template dot<VEC>(cw[r], regs);
      acc[r][b] += __uint_as_float(__float_as_uint(part * cs[r]) & keep);
    }
  };

  if constexpr (NSTEP > 0) {
    uint32_t all_w[NSTEP][ROWS][VEC];
    float all_s[NSTEP][ROWS];
    if constexpr (XLDS) {
      // 16-byte units, unit u of lane l at [(step * kUnits + u) * 64 + l]: conflict-free
      constexpr int kUnits = sizeof(Regs) / 16;
      static_assert(sizeof(Regs) % 16 == 0, "activation registers are whole 16-byte units");
      __shared__ uint4 s_x[NSTEP * kUnits * kWave];
      __shared__ float s_squares[VEC == 4 ? 4 : NSTEP];
      if constexpr (VEC == 4) {
        // Every wave stages a quarter of each step (8 elements a lane) and asks for it before
        // its weights.  Loads return in order — also across the waves of a CU, whose requests
        // share one queue in the vector cache — so x lines asked for after any weight line
        // arrive behind it: with one staging wave the barrier below opened only when weights
        // had come back from HBM (1.2-3.9 us after the launch), and all waves then ran their
        // dot products at once.  With x first in every wave the barrier opens after a cache
        // round trip and each wave starts on its rows as soon as its own weights are there.
        using Quarter = typename Acts<XT>::template Raw<1, NORM>;
        Quarter raw_q[NSTEP];
#pragma unroll
        for (int step = 0; step < NSTEP; ++step) {
          const uint32_t q_k0 = (uint32_t)step * kStepElems + wave * 512 + lane * 8;
          const uint32_t q_kc = q_k0 < k ? q_k0 : 0u;
          Acts<XT>::template request<1, NORM>(x + q_kc, norm_weight + q_kc, raw_q[step]);
        }
#pragma unroll
        for (int step = 0; step < NSTEP; ++step) fetch(step, all_w[step], all_s[step]);
        request_decode_row();
#pragma unroll
        for (int step = 0; step < NSTEP; ++step) {
          const uint32_t q_k0 = (uint32_t)step * kStepElems + wave * 512 + lane * 8;
          typename Acts<XT>::template Regs<1> part;
          Acts<XT>::template finish<1, NORM>(raw_q[step], q_k0 < k, part, squares[0]);
          constexpr int kQuarterUnits = sizeof(part) / 16;  // 2 (f32) or 1 (fp16)
          uint4 units[kQuarterUnits];
          __builtin_memcpy(units, &part, sizeof(part));
          // elements wave * 512 + lane * 8 .. + 8 of the step are the units from
          // kQuarterUnits * (lane % 4) on of the consuming lane wave * 16 + lane / 4
#pragma unroll
          for (int j = 0; j < kQuarterUnits; ++j)
            s_x[(step * kUnits + (lane & 3) * kQuarterUnits + j) * kWave + wave * 16 + (lane >> 2)] =
                units[j];
        }
        if constexpr (NORM) {
          const float total = wave_sum(squares[0]);
          if (lane == 0) s_squares[wave] = total;
        }
        __syncthreads();
        if constexpr (NORM)
          shared_squares = ((s_squares[0] + s_squares[1]) + s_squares[2]) + s_squares[3];
      } else {
        // narrow steps (4-byte loads): wave s stages step s, its activations requested first
        typename Acts<XT>::template Raw<VEC, NORM> raw_x;
        const uint32_t x_k0 = (uint32_t)wave * kStepElems + lane * kLaneElems;
        const uint32_t x_kc = x_k0 < k ? x_k0 : 0u;
        if (wave < NSTEP)
          Acts<XT>::template request<VEC, NORM>(x + x_kc, norm_weight + x_kc, raw_x);
#pragma unroll
        for (int step = 0; step < NSTEP; ++step) fetch(step, all_w[step], all_s[step]);
        if (wave < NSTEP) {
          Regs regs;
          Acts<XT>::template finish<VEC, NORM>(raw_x, x_k0 < k, regs, squares[0]);
          uint4 units[kUnits];
          __builtin_memcpy(units, &regs, sizeof(Regs));
#pragma unroll
          for (int u = 0; u < kUnits; ++u) s_x[(wave * kUnits + u) * kWave + lane] = units[u];
          if constexpr (NORM) {
            const float total = wave_sum(squares[0]);
            if (lane == 0) s_squares[wave] = total;
          }
        }
        __syncthreads();
        if constexpr (NORM) {
          float total = 0.f;
#pragma unroll
          for (int step = 0; step < NSTEP; ++step) total += s_squares[step];
          shared_squares = total;
        }
      }
#pragma unroll
      for (int step = 0; step < NSTEP; ++step) {
        uint4 units[kUnits];
#pragma unroll
        for (int u = 0; u < kUnits; ++u) units[u] = s_x[(step * kUnits + u) * kWave + lane];
        Regs regs;
        __builtin_memcpy(&regs, units, sizeof(Regs));
        consume(step, all_w[step], all_s[step], 0, regs);
      }
    } else if constexpr (MB == 1) {
#pragma unroll
      for (int step = 0; step < NSTEP; ++step) fetch(step, all_w[step], all_s[step]);
      Regs regs[NSTEP];
#pragma unroll
      for (int step = 0; step < NSTEP; ++step) fetch_x(step, 0, regs[step]);
#pragma unroll
      for (int step = 0; step < NSTEP; ++step) consume(step, all_w[step], all_s[step], 0, regs[step]);
    } else {
#pragma unroll
      for (int step = 0; step < NSTEP; ++step) fetch(step, all_w[step], all_s[step]);
#pragma unroll
      for (int step = 0; step < NSTEP; ++step) {
#pragma unroll
        for (int b = 0; b < MB; ++b) {
          Regs regs;
          fetch_x(step, b, regs);
          consume(step, all_w[step], all_s[step], b, regs);
        }
      }
    }
  } else {
    const uint32_t steps = (k + kStepElems - 1) / kStepElems;
    uint32_t cur_w[ROWS][VEC], nxt_w[ROWS][VEC];
    float cur_s[ROWS], nxt_s[ROWS];
    Regs cur_x, nxt_x;  // MB == 1 only: activations travel with the weights
    if constexpr (MB == 1) fetch_x(0, 0, cur_x);
    fetch(0, cur_w, cur_s);
    for (uint32_t step = 0; step < steps; ++step) {
      // unconditional (the last pass asks for its own step again, a cache hit that is not
      // used): a branch around loads makes the compiler wait for everything inside it
      const uint32_t ahead = step + 1 < steps ? step + 1 : step;
      if constexpr (MB == 1) fetch_x(ahead, 0, nxt_x, step + 1 < steps);
      fetch(ahead, nxt_w, nxt_s);
      if constexpr (MB == 1) {
        consume(step, cur_w, cur_s, 0, cur_x);
        cur_x = nxt_x;
      } else {
#pragma unroll
        for (int b = 0; b < MB; ++b) {
          Regs regs;
          fetch_x(step, b, regs);
          consume(step, cur_w, cur_s, b, regs);
        }
      }
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) cur_w[r][j] = nxt_w[r][j];
        cur_s[r] = nxt_s[r];
      }
    }
  }

  // fused rms_norm: every wave has seen the whole row of x, so 1/sqrt(mean(x^2)+eps) is a
  // wave reduction; it scales the finished dot product (the norm weight already multiplied x).
  float inv[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b)
    // v_rsq_f32 (1 ulp) here, v_exp_f32 and v_rcp_f32 in the silu below: the IEEE sequences of
    // sqrt, division and expf were a third of this epilogue's instructions, issued by every wave
    // of the CU at the same moment (gate/up launch: 1.4 us between the last dot product and the
    // end); the stand-alone rms_norm and silu kernels keep the exact forms
    inv[b] = NORM ? __builtin_amdgcn_rsqf((XLDS ? shared_squares : wave_sum(squares[b])) / (float)k +
                                          fuse.norm_eps)
                  : 1.0f;
  const XT* residual = static_cast<const XT*>(fuse.residual);
  // the rows' totals, uniform (one row of x: two or four rows are reduced together)
  float total[ROWS][MB];
  if constexpr (MB == 1 && ROWS == 4) {
    const float t = wave_sum4(acc[0][0], acc[1][0], acc[2][0], acc[3][0], lane);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) total[r][0] = lane_value(t, r);
  } else if constexpr (MB == 1 && ROWS == 2) {
    const float t = wave_sum2(acc[0][0], acc[1][0], lane);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) total[r][0] = lane_value(t, r);
  } else {
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int b = 0; b < MB; ++b) total[r][b] = wave_sum(acc[r][b]);
  }
  if constexpr (ROWS % 2 == 0) {
    if (fuse.pair_silu) {
      // rows (2i, 2i+1) hold (gate_i, up_i): out[., i] = silu(gate) * up, n/2 outputs per row
      const uint32_t half_n = n >> 1;
#pragma unroll
      for (int p = 0; p < ROWS / 2; ++p) {
        const uint32_t row = row0 + 2 * p, col = row >> 1;
#pragma unroll
        for (int b = 0; b < MB; ++b) {
          float gate = total[2 * p][b] * inv[b];
          float up = total[2 * p + 1][b] * inv[b];
          if (lane == (p * MB + b) % kWave && row + 1 < n && (uint32_t)b < m) {
            if (bias) {
              gate += to_f32<XT>(bias[row]);
              up += to_f32<XT>(bias[row + 1]);
            }
            const float t = __builtin_amdgcn_exp2f(-fabsf(gate) * 1.4426950408889634f);
            const float r = __builtin_amdgcn_rcpf(1.0f + t);
            const float sig = gate < 0.f ? t * r : r;
            float value = __fmul_rn(__fmul_rn(gate, sig), up);
            if (residual) value += to_f32<XT>(residual[(size_t)b * half_n + col]);
            out[(size_t)b * half_n + col] = from_f32<XT>(value);
          }
        }
      }
      return;
    }
    if constexpr (DECODE_ROW) {
      const uint32_t half = fuse.depth >> 1;
      const uint32_t rope_pairs = (fuse.heads + fuse.kv_heads) * half;
      uint32_t past = fuse.past;
      bool append = true;
      if (fuse.lengths) {  // run-time lengths read on the device; same checks as the scalar form
        past = dev_past;
        append = dev_query == 1u && (uint64_t)past + 1 <= 0xffffffffull &&
                 (fuse.window != 0 || (uint64_t)past + 1 <= fuse.capacity);
        if (!append && row0 == 0 && lane == 0) fuse.lengths[2] = 1u;
      }
      const uint32_t prow = fuse.window ? past % fuse.window : past;
      const bool pow2 = fuse.half_shift != 0xffffffffu;
      const bool in_table = rope_in_table;
#pragma unroll
      for (int p = 0; p < ROWS / 2; ++p) {
        const uint32_t row = row0 + 2 * p, pair = row >> 1;
        float x0 = total[2 * p][0] * inv[0];
        float x1 = total[2 * p + 1][0] * inv[0];
        if (lane != p % kWave || row + 1 >= n) continue;
        if (bias) {
          x0 += to_f32<XT>(bias[row]);
          x1 += to_f32<XT>(bias[row + 1]);
        }
        // what a separate linear would have stored (rounded to the activation type)
        x0 = to_f32<XT>(from_f32<XT>(x0));
        x1 = to_f32<XT>(from_f32<XT>(x1));
        if (pair < rope_pairs) {
          const uint32_t head = pow2 ? pair >> fuse.half_shift : pair / half;
          const uint32_t j = pair - head * half;
          float o0 = NAN, o1 = NAN;  // a position outside the table is never a valid rotation
          if (in_table) {
            o0 = __fadd_rn(__fmul_rn(x0, rope_cos[p][0]), __fmul_rn(-x1, rope_sin[p][0]));
            o1 = __fadd_rn(__fmul_rn(x1, rope_cos[p][1]), __fmul_rn(x0, rope_sin[p][1]));
          }
          const size_t at = (size_t)head * fuse.depth + j;
          out[at] = from_f32<XT>(o0);
          out[at + half] = from_f32<XT>(o1);
          if (head >= fuse.heads && append) {
            const size_t dst = ((size_t)(head - fuse.heads) * fuse.capacity + prow) * fuse.depth + j;
            slot_store(fuse.slot_k, fuse.slot_f16, dst, to_f32<XT>(from_f32<XT>(o0)));
            slot_store(fuse.slot_k, fuse.slot_f16, dst + half, to_f32<XT>(from_f32<XT>(o1)));
          }
        } else {
          const uint32_t e = (pair - rope_pairs) * 2;  // element of the v section, natural order
          const size_t at = (size_t)(fuse.heads + fuse.kv_heads) * fuse.depth + e;
          out[at] = from_f32<XT>(x0);
          out[at + 1] = from_f32<XT>(x1);
          if (append) {
            const uint32_t plane = pow2 ? e >> (fuse.half_shift + 1u) : e / fuse.depth;
            const uint32_t d = e - plane * fuse.depth;
            const size_t dst = ((size_t)plane * fuse.capacity + prow) * fuse.depth + d;
            slot_store(fuse.slot_v, fuse.slot_f16, dst, x0);
            slot_store(fuse.slot_v, fuse.slot_f16, dst + 1, x1);
          }
        }
      }
      return;
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const float sum = total[r][b] * inv[b];
      const uint32_t row = row0 + r;
      if (lane == (r * MB + b) % kWave && row < n && (uint32_t)b < m) {
        float value = sum + (bias ? to_f32<XT>(bias[row]) : 0.f);
        if (residual) value += to_f32<XT>(residual[(size_t)b * n + row]);
        out[(size_t)b * n + row] = from_f32<XT>(value);
      }
    }
  }
  if constexpr (MB == 1) {
    if (fuse.argmax_partial) {  // uniform over the launch
      // the values as stored (the totals are uniform over the wave, so every lane can redo the
      // few additions), best of the wave's rows, then best of the workgroup's waves
      __shared__ float s_best[4];
      __shared__ uint32_t s_at[4];
      float best = -INFINITY;
      uint32_t at = 0xffffffffu;
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const uint32_t row = row0 + r;
        if (row < n) {
          float value = total[r][0] * inv[0] + (bias ? to_f32<XT>(bias[row]) : 0.f);
          if (residual) value += to_f32<XT>(residual[row]);
          value = to_f32<XT>(from_f32<XT>(value));
          if (argmax_beats(value, row, best, at)) {
            best = value;
            at = row;
          }
        }
      }
      if (lane == 0) {
        s_best[wave] = best;
        s_at[wave] = at;
      }
      __syncthreads();
      if (threadIdx.x == 0) {
#pragma unroll
        for (int q = 1; q < 4; ++q)
          if (argmax_beats(s_best[q], s_at[q], best, at)) {
            best = s_best[q];
            at = s_at[q];
          }
        fuse.argmax_partial[blockIdx.x] = make_uint2(__float_as_uint(best), at);
      }
    }
  }
}

template <typename XT, typename ST, int MB, int ROWS, int VEC, int NSTEP>
int32_t launch_gemv(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                    krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift,
                    const GemvFusion& fuse = GemvFusion{}) {
  const uint32_t rows_per_block = 4 * ROWS;
  const uint32_t blocks = (n + rows_per_block - 1) / rows_per_block;
  if (fuse.host_blocks) *fuse.host_blocks = blocks;
#define KRM_GEMV_LAUNCH(NORM, ROW)                                                              \
  gemv_i4_kernel<XT, ST, MB, ROWS, VEC, NSTEP, NORM, ROW>                                       \
      <<<dim3(blocks), dim3(256), 0, ctx->stream>>>(ptr<const XT>(x), ptr<const uint32_t>(w),  \
                                                    ptr<const ST>(scales), fuse.norm_weight,   \
                                                    ptr<XT>(out), n, k, group_shift, m,         \
                                                    ptr<const XT>(bias), fuse)
  if constexpr (MB == 1 && ROWS % 2 == 0) {
    if (fuse.positions) {
      if (fuse.norm_weight) KRM_GEMV_LAUNCH(true, true); else KRM_GEMV_LAUNCH(false, true);
      return launched(ctx, "gemv_i4_kernel");
    }
  }
  if (fuse.positions) return fail(ctx, KRM_ERR_VALIDATION, "decode row: one row, even row count");
  if (fuse.norm_weight) KRM_GEMV_LAUNCH(true, false); else KRM_GEMV_LAUNCH(false, false);
#undef KRM_GEMV_LAUNCH
  return launched(ctx, "gemv_i4_kernel");
}

template <typename XT, typename ST, int MB, int ROWS, int VEC>
int32_t pick_steps(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                   uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift,
                   const GemvFusion& fuse) {
  // Rows short enough to hold in registers are requested whole (VEC == 4: 2048 codes a step).
  if constexpr (VEC == 4 && MB == 1) {
    const uint32_t steps = (k + 2047) / 2048;
    if (steps == 1)
      return launch_gemv<XT, ST, MB, ROWS, VEC, 1>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
    if (steps == 2)
      return launch_gemv<XT, ST, MB, ROWS, VEC, 2>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
    if constexpr (ROWS <= 2)
      if (steps == 3)
        return launch_gemv<XT, ST, MB, ROWS, VEC, 3>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
  }
  return launch_gemv<XT, ST, MB, ROWS, VEC, 0>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
}

template <typename XT, typename ST, int MB, int VEC>
int32_t pick_rows(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                  uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift,
                  const GemvFusion& fuse) {
  // Rows per wave: two rows share one fetch of the activations; one row per wave keeps more
  // waves in flight when N is small.  The choice never changes a row's reduction order.
  const uint64_t cus = (uint64_t)ctx->num_cus;
  // f32 activations of one row in one or two steps (K <= 4096): every workgroup stages the row
  // once, so more rows a wave mean fewer of those.  With the rms_norm in front (the norm weight
  // is staged too) that pays early; measured at K = 2048, us per launch with 1 / 2 / 4 rows a
  // wave: N = 2048 2.53 / 2.42 / 2.86, 4096 3.03 / 2.95 / 3.22, 6144 4.35 / 3.52 / 4.04, 8192
  // 5.03 / 4.05 / 4.23, 11264 - / 5.01 / 4.93, 32000 14.2 / 10.3 / 9.0.  Without it one row a
  // wave stays ahead on few rows (N = 2048 with a residual: 2.57 against 2.80).
  if constexpr (MB == 1 && sizeof(XT) == 4 && VEC == 4)
    if (k <= 4096) {
      if ((uint64_t)n >= cus * (fuse.norm_weight ? 40 : 32))
        return pick_steps<XT, ST, MB, 4, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
      if (fuse.norm_weight && (uint64_t)n >= cus * 8)
        return pick_steps<XT, ST, MB, 2, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
    }
  // fp16 activations, many rows (the streaming case: every SIMD still gets 4 waves or more):
  // four rows a wave share the activations read from LDS and the per-wave bookkeeping, about a
  // sixth of the instructions of a launch that the vector ALU bounds (K = 4096, 1 / 2 / 4 rows a
  // wave: N = 4096 3.62 / 3.75 / 4.31, 8192 5.74 / 5.09 / 5.48, 16384 9.50 / 8.46 / 8.06 us;
  // eight rows a wave measured slower again: 24.8 against 23.8 us on 65536 rows)
  if constexpr (MB == 1 && sizeof(XT) == 2 && VEC == 4)
    if (k <= 4096 && (uint64_t)n >= cus * 4 * 4 * 4)
      return pick_steps<XT, ST, MB, 4, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
  // (one row of x shared through LDS: below 32 rows a CU one row a wave — twice the waves —
  // measured 1.5 % more decode tokens/s and 1 % on the 4096 x 4096 GEMV)
  const bool shared_x = MB == 1 && VEC == 4 && k <= 6144;  // compile-time step count, x in LDS
  if (fuse.pair_silu || fuse.positions || (uint64_t)n >= cus * 4 * (shared_x ? 8 : 2))
    return pick_steps<XT, ST, MB, 2, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
  return pick_steps<XT, ST, MB, 1, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
}

template <typename XT, typename ST, int VEC>
int32_t pick_batch(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                   uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift,
                   const GemvFusion& fuse) {
  if (m == 1) return pick_rows<XT, ST, 1, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
  if (m == 2) return pick_rows<XT, ST, 2, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
  if (m <= 4) return pick_rows<XT, ST, 4, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
  if (m <= 8) return pick_rows<XT, ST, 8, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
  return pick_rows<XT, ST, 16, VEC>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
}

template <typename XT, typename ST>
int32_t pick_vec(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                 uint32_t m, uint32_t n, uint32_t k, uint32_t group, const GemvFusion& fuse) {
  uint32_t group_shift = 0;
  while ((1u << group_shift) < group) ++group_shift;
  // 16-byte loads need 32 codes per lane inside one group and 16-byte aligned rows.
  const bool wide = (k % 32 == 0) && (group % 32 == 0) && aligned(w, 16);
  if (wide) return pick_batch<XT, ST, 4>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
  return pick_batch<XT, ST, 1>(ctx, x, w, scales, bias, out, m, n, k, group_shift, fuse);
}

}  // namespace

namespace krm {

// Rows M <= 16: the GEMV above.  Declared in gemm_i4.hip's dispatcher too.
static int32_t gemv_dispatch(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                             krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                             int32_t io_dtype, int32_t scale_dtype, const GemvFusion& fuse) {
  if (io_dtype == KRM_F16) {
    // batched fp16 rows on the matrix cores (plain op only)
    const bool plain = !fuse.norm_weight && !fuse.residual && !fuse.pair_silu && !fuse.positions;
    if (plain && m >= 2 && k % 256 == 0 && group >= 128 && aligned(w, 16) && aligned(x, 16) &&
        aligned(scales, 4)) {
      uint32_t group_shift = 0;
      while ((1u << group_shift) < group) ++group_shift;
      const uint32_t blocks = (n + 15) / 16;
#define KRM_MFMA_GEMV(ST, CH, KW)                                                              \
  gemv_i4_mfma_kernel<ST, CH, KW><<<dim3(blocks), dim3(KW * 64), 0, ctx->stream>>>(            \
      ptr<const __half>(x), ptr<const uint32_t>(w), ptr<const ST>(scales),                     \
      ptr<const __half>(bias), ptr<__half>(out), m, n, k, group_shift)
  // eight waves a workgroup (two per SIMD) when K gives each at least one chunk
#define KRM_MFMA_GEMV_BY_K(ST)                         \
  switch (k % 1024 ? 0u : k / 1024) {                  \
    case 1: KRM_MFMA_GEMV(ST, 1, 4); break;            \
    case 2: KRM_MFMA_GEMV(ST, 1, 8); break;            \
    case 4: KRM_MFMA_GEMV(ST, 2, 8); break;            \
    case 8: KRM_MFMA_GEMV(ST, 4, 8); break;            \
    default:                                           \
      if (k >= 2048) {                                 \
        KRM_MFMA_GEMV(ST, 0, 8);                       \
      } else {                                         \
        KRM_MFMA_GEMV(ST, 0, 4);                       \
      }                                                \
      break;                                           \
  }
      if (scale_dtype == KRM_F16) {
        KRM_MFMA_GEMV_BY_K(__half)
      } else {
        KRM_MFMA_GEMV_BY_K(float)
      }
#undef KRM_MFMA_GEMV_BY_K
#undef KRM_MFMA_GEMV
      return launched(ctx, "gemv_i4_mfma_kernel");
    }
    if (scale_dtype == KRM_F16)
      return pick_vec<__half, __half>(ctx, x, w, scales, bias, out, m, n, k, group, fuse);
    return pick_vec<__half, float>(ctx, x, w, scales, bias, out, m, n, k, group, fuse);
  }
  if (scale_dtype == KRM_F16)
    return pick_vec<float, __half>(ctx, x, w, scales, bias, out, m, n, k, group, fuse);
  return pick_vec<float, float>(ctx, x, w, scales, bias, out, m, n, k, group, fuse);
}

int32_t linear_i4_gemv(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                       krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                       int32_t io_dtype, int32_t scale_dtype) {
  return gemv_dispatch(ctx, x, w, scales, bias, out, m, n, k, group, io_dtype, scale_dtype,
                       GemvFusion{});
}

// MFMA GEMMs for M > 16 (gemm_i4.hip): exact integer weights (large shapes), fp16 weights.
int32_t linear_i4_gemm_exact(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                             krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                             int32_t io_dtype, int32_t scale_dtype, int32_t compute,
                             bool* handled);
int32_t linear_i4_gemm_rows(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                            krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                            int32_t io_dtype, int32_t scale_dtype, int32_t compute,
                            const RowsFusion& fuse, bool* handled, int32_t x_dtype);
int32_t linear_i4_gemm_f16(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                           krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                           int32_t io_dtype, int32_t scale_dtype);

}  // namespace krm

extern "C" {

int32_t krm_linear_i4(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                      krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                      int32_t io_dtype, int32_t scale_dtype, int32_t compute) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(scale_dtype),
              "krm_linear_i4: io_dtype %d / scale_dtype %d", io_dtype, scale_dtype);
  KRM_REQUIRE(ctx, compute == KRM_COMPUTE_F32 || compute == KRM_COMPUTE_F16,
              "krm_linear_i4: compute %d", compute);
  // Storage rules of the int4 format: group is a power of two >= 16 that divides K.
  KRM_REQUIRE(ctx, is_pow2(group) && group >= 16,
              "krm_linear_i4: group_size %u is not a power of two >= 16", group);
  KRM_REQUIRE(ctx, k >= 1 && k % group == 0,
              "krm_linear_i4: group_size %u does not divide k = %u", group, k);
  if (m == 0 || n == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && w && scales && out, "krm_linear_i4: NULL buffer");
  KRM_REQUIRE(ctx, aligned(x, 16) && aligned(out, dtype_bytes(io_dtype)) && aligned(w, 4) &&
                       aligned(scales, dtype_bytes(scale_dtype)) &&
                       aligned(bias, dtype_bytes(io_dtype)),
              "krm_linear_i4: x must be 16-byte aligned, w 4-byte aligned");
  if (m <= 16)
    return linear_i4_gemv(ctx, x, w, scales, bias, out, m, n, k, group, io_dtype, scale_dtype);
  bool handled = false;
  // Both MFMA forms compute the same arithmetic class.  The 32-row tiles win while their
  // workgroups make at most three rounds over the CUs (measured: 128 x 11264 x 2048 28.5 us
  // against 34.2 us, 512 x 2560 x 2048 29.2 against 33.9; 256 x 11264 x 2048 53.7 against 37.7).
  {
    uint64_t workgroups = (uint64_t)((m + 31) / 32) * ((n + 31) / 32);
    if (workgroups > (uint64_t)ctx->num_cus) workgroups = (workgroups + 1) / 2;
    if (workgroups <= 3ull * (uint64_t)ctx->num_cus) {
      KRM_TRY(linear_i4_gemm_rows(ctx, x, w, scales, bias, out, m, n, k, group, io_dtype,
                                  scale_dtype, compute, RowsFusion{}, &handled, io_dtype));
      if (handled) return KRM_OK;
    }
  }
  KRM_TRY(linear_i4_gemm_exact(ctx, x, w, scales, bias, out, m, n, k, group, io_dtype,
                               scale_dtype, compute, &handled));
  if (handled) return KRM_OK;
  KRM_TRY(linear_i4_gemm_rows(ctx, x, w, scales, bias, out, m, n, k, group, io_dtype, scale_dtype,
                              compute, RowsFusion{}, &handled, io_dtype));
  if (handled) return KRM_OK;
  if (compute == KRM_COMPUTE_F16)
    return linear_i4_gemm_f16(ctx, x, w, scales, bias, out, m, n, k, group, io_dtype,
                              scale_dtype);
  // f32 arithmetic for any M: the GEMV over blocks of 16 rows (weights re-read per block).
  const size_t eb = dtype_bytes(io_dtype);
  for (uint32_t r = 0; r < m; r += 16) {
    const uint32_t rows = m - r < 16 ? m - r : 16;
    KRM_TRY(linear_i4_gemv(ctx, x + (size_t)r * k * eb, w, scales, bias,
                           out + (size_t)r * n * eb, rows, n, k, group, io_dtype, scale_dtype));
  }
  return KRM_OK;
}

int32_t krm_probe_linear_series(krm_ctx* ctx, krm_buf x, const krm_buf* w_list,
                                const krm_buf* scales_list, uint32_t copies, krm_buf out,
                                uint32_t count, uint32_t m, uint32_t n, uint32_t k,
                                uint32_t group, int32_t io_dtype, int32_t scale_dtype) {
  KRM_TRY(enter(ctx));
  KRM_TRY(not_recording(ctx, "krm_probe_linear_series"));
  KRM_REQUIRE(ctx, w_list && scales_list && copies >= 1, "krm_probe_linear_series: no weights");
  KRM_REQUIRE(ctx, m >= 1 && m <= 16, "krm_probe_linear_series: m = %u (1..16)", m);
  for (uint32_t i = 0; i < count; ++i)
    KRM_TRY(krm_linear_i4(ctx, x, w_list[i % copies], scales_list[i % copies], 0, out, m, n, k,
                          group, io_dtype, scale_dtype, KRM_COMPUTE_F32));
  return KRM_OK;
}

int32_t krm_linear_i4_fused(krm_ctx* ctx, krm_buf x, krm_buf norm_weight_f32, float norm_eps,
                            krm_buf w, krm_buf scales, krm_buf bias, krm_buf residual,
                            krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                            int32_t io_dtype, int32_t scale_dtype, int32_t epilogue) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(scale_dtype),
              "krm_linear_i4_fused: io_dtype %d / scale_dtype %d", io_dtype, scale_dtype);
  KRM_REQUIRE(ctx, epilogue == KRM_EPILOGUE_NONE || epilogue == KRM_EPILOGUE_SILU_PAIRS,
              "krm_linear_i4_fused: epilogue %d", epilogue);
  KRM_REQUIRE(ctx, is_pow2(group) && group >= 16 && k >= 1 && k % group == 0,
              "krm_linear_i4_fused: group_size %u must be a power of two >= 16 dividing k = %u",
              group, k);
  KRM_REQUIRE(ctx, m >= 1 && m <= 16,
              "krm_linear_i4_fused: m = %u; the fused form covers 1..16 rows (use the separate ops "
              "for prefill chunks)", m);
  KRM_REQUIRE(ctx, epilogue != KRM_EPILOGUE_SILU_PAIRS || n % 2 == 0,
              "krm_linear_i4_fused: the gate/up epilogue needs an even n, got %u", n);
  KRM_REQUIRE(ctx, !norm_weight_f32 || std::isfinite(norm_eps), "krm_linear_i4_fused: eps");
  if (n == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && w && scales && out, "krm_linear_i4_fused: NULL buffer");
  KRM_REQUIRE(ctx, aligned(x, 16) && aligned(norm_weight_f32, 16) && aligned(w, 4) &&
                       aligned(out, dtype_bytes(io_dtype)) &&
                       aligned(residual, dtype_bytes(io_dtype)) &&
                       aligned(bias, dtype_bytes(io_dtype)) &&
                       aligned(scales, dtype_bytes(scale_dtype)),
              "krm_linear_i4_fused: x and norm weight must be 16-byte aligned, w 4-byte aligned");
  GemvFusion fuse{};
  fuse.norm_weight = ptr<const float>(norm_weight_f32);
  fuse.norm_eps = norm_eps;
  fuse.residual = ptr<const void>(residual);
  fuse.pair_silu = epilogue == KRM_EPILOGUE_SILU_PAIRS ? 1u : 0u;
  return gemv_dispatch(ctx, x, w, scales, bias, out, m, n, k, group, io_dtype, scale_dtype, fuse);
}

int32_t krm_decode_head(krm_ctx* ctx, krm_buf x, krm_buf norm_weight_f32, float norm_eps,
                        krm_buf w, krm_buf scales, krm_buf bias, krm_buf logits, krm_buf partials,
                        size_t partials_bytes, uint32_t* partial_count, uint32_t n, uint32_t k,
                        uint32_t group, int32_t io_dtype, int32_t scale_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(scale_dtype),
              "krm_decode_head: io_dtype %d / scale_dtype %d", io_dtype, scale_dtype);
  KRM_REQUIRE(ctx, is_pow2(group) && group >= 16 && k >= 1 && k % group == 0,
              "krm_decode_head: group_size %u must be a power of two >= 16 dividing k = %u", group,
              k);
  KRM_REQUIRE(ctx, n >= 1 && n <= 0x7fffffffu, "krm_decode_head: n = %u", n);
  KRM_REQUIRE(ctx, !norm_weight_f32 || std::isfinite(norm_eps), "krm_decode_head: eps");
  KRM_REQUIRE(ctx, partial_count != nullptr, "krm_decode_head: partial_count is NULL");
  KRM_REQUIRE(ctx, x && w && scales && logits && partials, "krm_decode_head: NULL buffer");
  KRM_REQUIRE(ctx, aligned(x, 16) && aligned(norm_weight_f32, 16) && aligned(w, 4) &&
                       aligned(logits, dtype_bytes(io_dtype)) &&
                       aligned(bias, dtype_bytes(io_dtype)) &&
                       aligned(scales, dtype_bytes(scale_dtype)) && aligned(partials, 8),
              "krm_decode_head: x and norm weight must be 16-byte aligned, w 4-byte, partials "
              "8-byte aligned");
  // at most one workgroup per four rows, whatever rows-per-wave the launch picks
  const size_t worst = ((size_t)n + 3) / 4 * sizeof(uint2);
  KRM_REQUIRE(ctx, partials_bytes >= worst,
              "krm_decode_head: partials of %zu bytes, %zu needed (8 bytes per 4 rows)",
              partials_bytes, worst);
  GemvFusion fuse{};
  fuse.norm_weight = ptr<const float>(norm_weight_f32);
  fuse.norm_eps = norm_eps;
  fuse.argmax_partial = ptr<uint2>(partials);
  uint32_t blocks = 0;
  fuse.host_blocks = &blocks;
  KRM_TRY(gemv_dispatch(ctx, x, w, scales, bias, logits, 1, n, k, group, io_dtype, scale_dtype,
                        fuse));
  *partial_count = blocks;
  return KRM_OK;
}

int32_t krm_linear_i4_rows(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                           krm_buf residual, krm_buf out, uint32_t m, uint32_t n, uint32_t k,
                           uint32_t group, int32_t io_dtype, int32_t scale_dtype, int32_t compute,
                           int32_t epilogue, int32_t x_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(scale_dtype),
              "krm_linear_i4_rows: io_dtype %d / scale_dtype %d", io_dtype, scale_dtype);
  KRM_REQUIRE(ctx, x_dtype == io_dtype ||
                       (x_dtype == KRM_F16 && io_dtype == KRM_F32 && compute == KRM_COMPUTE_F16),
              "krm_linear_i4_rows: x_dtype %d with io_dtype %d / compute %d (fp16 x beside f32 io "
              "needs KRM_COMPUTE_F16)", x_dtype, io_dtype, compute);
  KRM_REQUIRE(ctx, compute == KRM_COMPUTE_F32 || compute == KRM_COMPUTE_F16,
              "krm_linear_i4_rows: compute %d", compute);
  KRM_REQUIRE(ctx, epilogue == KRM_EPILOGUE_NONE || epilogue == KRM_EPILOGUE_SILU_PAIRS,
              "krm_linear_i4_rows: epilogue %d", epilogue);
  KRM_REQUIRE(ctx, is_pow2(group) && group >= 16 && k >= 1 && k % group == 0,
              "krm_linear_i4_rows: group_size %u must be a power of two >= 16 dividing k = %u",
              group, k);
  KRM_REQUIRE(ctx, epilogue != KRM_EPILOGUE_SILU_PAIRS || n % 2 == 0,
              "krm_linear_i4_rows: the gate/up epilogue needs an even n, got %u", n);
  if (m == 0 || n == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && w && scales && out, "krm_linear_i4_rows: NULL buffer");
  KRM_REQUIRE(ctx, aligned(out, dtype_bytes(io_dtype)) && aligned(residual, dtype_bytes(io_dtype)) &&
                       aligned(bias, dtype_bytes(io_dtype)) &&
                       aligned(scales, dtype_bytes(scale_dtype)),
              "krm_linear_i4_rows: misaligned buffer");
  RowsFusion fuse{};
  fuse.residual = ptr<const void>(residual);
  fuse.mode = epilogue == KRM_EPILOGUE_SILU_PAIRS ? 1 : 0;
  bool handled = false;
  KRM_TRY(linear_i4_gemm_rows(ctx, x, w, scales, bias, out, m, n, k, group, io_dtype, scale_dtype,
                              compute, fuse, &handled, x_dtype));
  if (handled) return KRM_OK;
  return fail(ctx, KRM_ERR_VALIDATION,
              "krm_linear_i4_rows: covers group_size >= 64, k %% 32 == 0, 16-byte aligned x and w, "
              "m * k and n * k / 2 below 2^32 and, in the f32 class, m <= 65536 (m %u, n %u, "
              "group %u, k %u); use krm_linear_i4 and the separate ops", m, n, group, k);
}

int32_t krm_prefill_qkv(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                        krm_buf positions_i32, krm_buf cos_table_f32, krm_buf sin_table_f32,
                        krm_buf q_out, krm_buf k_out, krm_buf v_out, uint32_t m, uint32_t heads,
                        uint32_t kv_heads, uint32_t depth, uint32_t k, uint32_t group,
                        uint32_t table_rows, int32_t io_dtype, int32_t scale_dtype,
                        int32_t compute, int32_t x_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(scale_dtype),
              "krm_prefill_qkv: io_dtype %d / scale_dtype %d", io_dtype, scale_dtype);
  KRM_REQUIRE(ctx, x_dtype == io_dtype ||
                       (x_dtype == KRM_F16 && io_dtype == KRM_F32 && compute == KRM_COMPUTE_F16),
              "krm_prefill_qkv: x_dtype %d with io_dtype %d / compute %d (fp16 x beside f32 io "
              "needs KRM_COMPUTE_F16)", x_dtype, io_dtype, compute);
  KRM_REQUIRE(ctx, compute == KRM_COMPUTE_F32 || compute == KRM_COMPUTE_F16,
              "krm_prefill_qkv: compute %d", compute);
  KRM_REQUIRE(ctx, is_pow2(group) && group >= 16 && k >= 1 && k % group == 0,
              "krm_prefill_qkv: group_size %u must be a power of two >= 16 dividing k = %u", group,
              k);
  KRM_REQUIRE(ctx, heads >= 1 && kv_heads >= 1 && depth >= 2 && depth % 2 == 0 && table_rows >= 1,
              "krm_prefill_qkv: H / Hkv / D / table rows (%u / %u / %u / %u)", heads, kv_heads,
              depth, table_rows);
  KRM_REQUIRE(ctx, ((uint64_t)heads + 2ull * kv_heads) * depth <= 0x7fffffffull,
              "krm_prefill_qkv: the row is too long");
  if (m == 0) return KRM_OK;
  KRM_REQUIRE(ctx, x && w && scales && positions_i32 && cos_table_f32 && sin_table_f32 && q_out &&
                       k_out && v_out,
              "krm_prefill_qkv: NULL buffer");
  KRM_REQUIRE(ctx, aligned(q_out, dtype_bytes(io_dtype)) && aligned(k_out, dtype_bytes(io_dtype)) &&
                       aligned(v_out, dtype_bytes(io_dtype)) &&
                       aligned(bias, dtype_bytes(io_dtype)) &&
                       aligned(scales, dtype_bytes(scale_dtype)) && aligned(positions_i32, 4) &&
                       aligned(cos_table_f32, 4) && aligned(sin_table_f32, 4),
              "krm_prefill_qkv: misaligned buffer");
  RowsFusion fuse{};
  fuse.mode = 2;
  fuse.positions = ptr<const int32_t>(positions_i32);
  fuse.cos_table = ptr<const float>(cos_table_f32);
  fuse.sin_table = ptr<const float>(sin_table_f32);
  fuse.q_out = ptr<void>(q_out);
  fuse.k_out = ptr<void>(k_out);
  fuse.v_out = ptr<void>(v_out);
  fuse.heads = heads;
  fuse.kv_heads = kv_heads;
  fuse.depth = depth;
  fuse.table_rows = table_rows;
  const uint32_t n = (heads + 2 * kv_heads) * depth;
  bool handled = false;
  KRM_TRY(linear_i4_gemm_rows(ctx, x, w, scales, bias, q_out, m, n, k, group, io_dtype, scale_dtype,
                              compute, fuse, &handled, x_dtype));
  if (handled) return KRM_OK;
  return fail(ctx, KRM_ERR_VALIDATION,
              "krm_prefill_qkv: covers group_size >= 64, k %% 32 == 0, 16-byte aligned x and w, "
              "m * k and n * k / 2 below 2^32 and, in the f32 class, m <= 65536 (m %u, group %u, "
              "k %u); use krm_linear_i4, krm_rope_half and krm_transpose_01", m, group, k);
}

int32_t krm_decode_qkv(krm_ctx* ctx, krm_buf x, krm_buf norm_weight_f32, float norm_eps,
                       krm_buf w, krm_buf scales, krm_buf bias, krm_buf positions_i32,
                       krm_buf cos_table_f32, krm_buf sin_table_f32, krm_buf out, krm_buf slot_k,
                       krm_buf slot_v, uint32_t heads, uint32_t kv_heads, uint32_t depth,
                       uint32_t k, uint32_t group, uint32_t table_rows, uint32_t capacity,
                       uint32_t window, uint32_t past, krm_buf lengths, int32_t io_dtype,
                       int32_t scale_dtype, int32_t kv_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(scale_dtype) && valid_dtype(kv_dtype),
              "krm_decode_qkv: io_dtype %d / scale_dtype %d / kv_dtype %d", io_dtype, scale_dtype,
              kv_dtype);
  KRM_REQUIRE(ctx, is_pow2(group) && group >= 16 && k >= 1 && k % group == 0,
              "krm_decode_qkv: group_size %u must be a power of two >= 16 dividing k = %u", group,
              k);
  KRM_REQUIRE(ctx, heads >= 1 && depth >= 2 && depth % 2 == 0 && capacity >= 1 && table_rows >= 1,
              "krm_decode_qkv: H / D / C / table rows (%u / %u / %u / %u)", heads, depth, capacity,
              table_rows);
  // kv_heads == 0: a layer that reads another layer's K / V projects and rotates q alone and
  // appends nothing (no slots)
  KRM_REQUIRE(ctx, kv_heads >= 1 || (!slot_k && !slot_v),
              "krm_decode_qkv: kv_heads = 0 (q only) takes no state slots");
  KRM_REQUIRE(ctx, ((uint64_t)heads + 2ull * kv_heads) * depth <= 0x7fffffffull,
              "krm_decode_qkv: the row is too long");
  KRM_REQUIRE(ctx, window <= capacity, "krm_decode_qkv: window %u exceeds capacity %u", window,
              capacity);
  KRM_REQUIRE(ctx, !norm_weight_f32 || std::isfinite(norm_eps), "krm_decode_qkv: eps");
  if (!lengths && window == 0 && (uint64_t)past + 1 > capacity)
    return fail(ctx, KRM_ERR_EXECUTION,
                "krm_decode_qkv: pastLength %u + queryLength 1 exceeds capacity %u", past, capacity);
  KRM_REQUIRE(ctx, x && w && scales && positions_i32 && cos_table_f32 && sin_table_f32 && out &&
                       (kv_heads == 0 || (slot_k && slot_v)),
              "krm_decode_qkv: NULL buffer");
  KRM_REQUIRE(ctx, aligned(x, 16) && aligned(norm_weight_f32, 16) && aligned(w, 4) &&
                       aligned(out, dtype_bytes(io_dtype)) && aligned(bias, dtype_bytes(io_dtype)) &&
                       aligned(scales, dtype_bytes(scale_dtype)) && aligned(positions_i32, 4) &&
                       aligned(cos_table_f32, 4) && aligned(sin_table_f32, 4) &&
                       aligned(slot_k, dtype_bytes(kv_dtype)) &&
                       aligned(slot_v, dtype_bytes(kv_dtype)) && aligned(lengths, 4),
              "krm_decode_qkv: misaligned buffer");
  GemvFusion fuse{};
  fuse.norm_weight = ptr<const float>(norm_weight_f32);
  fuse.norm_eps = norm_eps;
  fuse.positions = ptr<const int32_t>(positions_i32);
  fuse.cos_table = ptr<const float>(cos_table_f32);
  fuse.sin_table = ptr<const float>(sin_table_f32);
  fuse.slot_k = ptr<void>(slot_k);
  fuse.slot_v = ptr<void>(slot_v);
  fuse.lengths = ptr<uint32_t>(lengths);
  fuse.heads = heads;
  fuse.kv_heads = kv_heads;
  fuse.depth = depth;
  fuse.table_rows = table_rows;
  fuse.capacity = capacity;
  fuse.window = window;
  fuse.past = past;
  fuse.slot_f16 = kv_dtype == KRM_F16 ? 1 : 0;
  fuse.half_shift = 0xffffffffu;
  if (is_pow2(depth >> 1)) {
    fuse.half_shift = 0;
    while ((1u << fuse.half_shift) < (depth >> 1)) ++fuse.half_shift;
  }
  const uint32_t n = (heads + 2 * kv_heads) * depth;
  return gemv_dispatch(ctx, x, w, scales, bias, out, 1, n, k, group, io_dtype, scale_dtype, fuse);
}

int32_t krm_dequant_i4(krm_ctx* ctx, krm_buf w, krm_buf scales, krm_buf out_f32, uint64_t rows,
                       uint64_t width, uint32_t group, int32_t scale_dtype) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(scale_dtype), "krm_dequant_i4: scale_dtype %d", scale_dtype);
  KRM_REQUIRE(ctx, group >= 1 && width >= 1 && width % group == 0,
              "krm_dequant_i4: group_size %u does not divide the row length %llu", group,
              (unsigned long long)width);
  KRM_REQUIRE(ctx, (rows * width) % 8 == 0,
              "krm_dequant_i4: %llu x %llu codes is not a whole number of 32-bit words",
              (unsigned long long)rows, (unsigned long long)width);
  if (rows == 0) return KRM_OK;
  KRM_REQUIRE(ctx, w && scales && out_f32, "krm_dequant_i4: NULL buffer");
  KRM_REQUIRE(ctx, aligned(w, 4) && aligned(out_f32, 16) && aligned(scales, dtype_bytes(scale_dtype)),
              "krm_dequant_i4: w must be 4-byte and out 16-byte aligned");
  const size_t words = rows * width / 8;
  size_t blocks = (words + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  if (scale_dtype == KRM_F16)
    dequant_i4_kernel<__half><<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(
        ptr<const uint32_t>(w), ptr<const __half>(scales), ptr<float>(out_f32), words, width,
        group);
  else
    dequant_i4_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(
        ptr<const uint32_t>(w), ptr<const float>(scales), ptr<float>(out_f32), words, width,
        group);
  return launched(ctx, "dequant_i4_kernel");
}

}  // extern "C"
