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
// tiles, optionally KS wave groups that split each chunk's K and add their sums at the end);
// K is walked KC (64 or 128) codes at a time through LDS:
//   A tile  x[BM rows][KC]  fp16, each group of 8 stored as (x0,x4,x1,x5,x2,x6,x3,x7)
//   B tile  w[BN rows][KC]  fp16 dequantised, the same order within each group of 8 — the
//           order the nibble trick produces (code i pairs with code i+4), so no shuffle is
//           spent on the weights; the k index inside an MFMA is a free permutation as long as
//           both operands use the same one.
// Rows are padded by 16 bytes so the 16-byte fragment reads of 32 consecutive rows spread over
// all LDS banks.  Chunks travel memory -> registers (several in flight, no use of a loaded
// value before it is parked, so the waits are counted) -> LDS -> fragments.  Pipelined form:
// two LDS copies (distinct objects, so fragment reads may pass the parking writes), the
// dequantisation of chunk c + 1 interleaved with the MFMAs of chunk c, one barrier a chunk.
#include "krm_internal.h"

using namespace krm;

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// A K chunk of KC codes is staged per pass; rows are padded by 16 bytes so the 16-byte
// fragment reads of 32 consecutive rows spread over all LDS banks.
template <int KC>
struct ChunkGeometry {
  static constexpr int kRowBytes = KC * 2 + 16;
};

// A scale as it arrives from memory, kept in a whole 32-bit register until the chunk is parked
// (narrowing it on arrival would be an ALU op that has to wait for the load).
template <typename ST>
__device__ inline uint32_t scale_bits(const ST* s, size_t i);
template <>
__device__ inline uint32_t scale_bits<__half>(const __half* s, size_t i) {
  return reinterpret_cast<const uint16_t*>(s)[i];
}
template <>
__device__ inline uint32_t scale_bits<float>(const float* s, size_t i) {
  return reinterpret_cast<const uint32_t*>(s)[i];
}
template <typename ST>
__device__ inline float load_scale_f32(const ST* s, size_t i);
template <>
__device__ inline float load_scale_f32<__half>(const __half* s, size_t i) {
  return __half2float(s[i]);
}
template <>
__device__ inline float load_scale_f32<float>(const float* s, size_t i) { return s[i]; }
template <typename ST>
__device__ inline _Float16 scale_from_bits(uint32_t bits);
template <>
__device__ inline _Float16 scale_from_bits<__half>(uint32_t bits) {
  return __builtin_bit_cast(_Float16, (uint16_t)bits);
}
template <>
__device__ inline _Float16 scale_from_bits<float>(uint32_t bits) {
  return (_Float16)__uint_as_float(bits);
}

// (a & mask) | bits in one VALU op (the compiler emits two when both constants are literals).
__device__ inline uint32_t and_or(uint32_t a, uint32_t mask, uint32_t bits) {
  uint32_t d;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask), "v"(bits));
  return d;
}

// 8 codes of a word -> 8 fp16 values (u - 8) * scale, order (c0,c4,c1,c5,c2,c6,c3,c7).
__device__ inline uint4 dequant_word(uint32_t word, _Float16 scale) {
  const uint32_t magic = 0x64006400u;  // (1024, 1024)
  const half2_t off_lo = {(_Float16)1032.0f, (_Float16)1032.0f};
  const half2_t sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  const half2_t off_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
  const half2_t s2 = {scale, scale};
  const uint32_t upper = word >> 8;
  const half2_t q0 = (__builtin_bit_cast(half2_t, and_or(word, 0x000F000Fu, magic)) - off_lo) * s2;
  const half2_t q1 = (__builtin_elementwise_fma(
                         __builtin_bit_cast(half2_t, and_or(word, 0x00F000F0u, magic)), sixteenth,
                         off_hi)) * s2;
  const half2_t q2 = (__builtin_bit_cast(half2_t, and_or(upper, 0x000F000Fu, magic)) - off_lo) * s2;
  const half2_t q3 = (__builtin_elementwise_fma(
                         __builtin_bit_cast(half2_t, and_or(upper, 0x00F000F0u, magic)), sixteenth,
                         off_hi)) * s2;
  return make_uint4(__builtin_bit_cast(uint32_t, q0), __builtin_bit_cast(uint32_t, q1),
                    __builtin_bit_cast(uint32_t, q2), __builtin_bit_cast(uint32_t, q3));
}

// 8 consecutive activations as they arrive from memory; converted to fp16 in the order
// (x0,x4,x1,x5,x2,x6,x3,x7) only when they are parked in LDS, so the loads stay in flight.
template <typename XT>
struct Acts8;
template <>
struct Acts8<__half> {
  uint4 raw;
  __device__ inline void load(const __half* p) { raw = *reinterpret_cast<const uint4*>(p); }
  __device__ inline void keep(uint32_t bits) {
    raw.x &= bits; raw.y &= bits; raw.z &= bits; raw.w &= bits;
  }
  __device__ inline uint4 paired() const {
    return make_uint4(__builtin_amdgcn_perm(raw.z, raw.x, 0x05040100u),
                      __builtin_amdgcn_perm(raw.z, raw.x, 0x07060302u),
                      __builtin_amdgcn_perm(raw.w, raw.y, 0x05040100u),
                      __builtin_amdgcn_perm(raw.w, raw.y, 0x07060302u));
  }
};
template <>
struct Acts8<float> {
  uint4 a, b;  // raw bits of x0..x3, x4..x7
  __device__ inline void load(const float* p) {
    a = reinterpret_cast<const uint4*>(p)[0];
    b = reinterpret_cast<const uint4*>(p)[1];
  }
  __device__ inline void keep(uint32_t bits) {
    a.x &= bits; a.y &= bits; a.z &= bits; a.w &= bits;
    b.x &= bits; b.y &= bits; b.z &= bits; b.w &= bits;
  }
  __device__ inline uint4 paired() const {
    auto pack = [](uint32_t lo, uint32_t hi) {
      const half2_t h = {(_Float16)__uint_as_float(lo), (_Float16)__uint_as_float(hi)};  // RNE
      return __builtin_bit_cast(uint32_t, h);
    };
    return make_uint4(pack(a.x, b.x), pack(a.y, b.y), pack(a.z, b.z), pack(a.w, b.w));
  }
};

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

template <typename XT, typename ST, int WM, int WN, int KC, int KS, int DEPTH, bool PIPE, bool FAST>
__global__ __launch_bounds__(WM * WN * KS * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_i4_f16_kernel(const XT* __restrict__ x, const uint32_t* __restrict__ w,
                        const ST* __restrict__ scales, const XT* __restrict__ bias,
                        XT* __restrict__ out, uint32_t m, uint32_t n, uint32_t k,
                        uint32_t group_shift, uint32_t m_blocks, uint32_t n_blocks,
                        uint32_t wide_rows) {
  // KS wave groups share the tile and split every chunk's K between them (their sums are
  // added once at the end): more waves per output, so more work in flight per CU.
  constexpr int kThreads = WM * WN * KS * 64;
  constexpr int BM = WM * 64, BN = WN * 64;
  constexpr int kRowBytes = ChunkGeometry<KC>::kRowBytes;
  constexpr int kStepsPerGroup = KC / 16 / KS;
  static_assert(KC % (16 * KS) == 0, "the K split divides the chunk");
  constexpr int kRowPieces = KC / 8;                 // 16-byte pieces (or weight words) a row
  constexpr int kAPieces = BM * kRowPieces;          // 16-byte pieces of the A tile
  constexpr int kAPer = kAPieces / kThreads;         // per thread
  constexpr int kBPieces = BN * kRowPieces;          // words of the B tile
  constexpr int kBPer = kBPieces / kThreads;         // words per thread (consecutive in a row)
  static_assert(kAPieces % kThreads == 0 && kBPieces % kThreads == 0, "tile / thread mismatch");
  static_assert(kBPer == 1 || kBPer == 2 || kBPer == 4 || kBPer == 8 || kBPer == 16,
                "B words per thread");
  static_assert(kRowPieces % kBPer == 0, "a thread's weight words stay inside one row");

  // One LDS copy of the chunk; the NEXT chunk waits in registers (its loads are issued right
  // after this chunk is parked), and several workgroups share a CU, so a workgroup that sits
  // at a barrier or waits for memory leaves the matrix cores to the others.
  // PIPE: two LDS copies; while the matrix cores work on chunk c out of one copy, the same
  // wave parks chunk c + 1 in the other (the two instruction streams interleave), one barrier
  // per chunk.
  constexpr int kStageBytes = (BM + BN) * kRowBytes;
  constexpr int kStageValuPerMfma = (kAPer * 4 + kBPer * 13 + kStepsPerGroup * 4 - 1) / (kStepsPerGroup * 4);
  constexpr int kReduceBytes = KS > 1 ? WM * WN * (KS - 1) * 64 * 64 * 4 : 0;
  // two separate objects, so the compiler knows that parking into one copy cannot touch the
  // other and may move the fragment reads past those writes
  __shared__ __attribute__((aligned(16)))
  unsigned char lds[kStageBytes > kReduceBytes ? kStageBytes : kReduceBytes];
  __shared__ __attribute__((aligned(16))) unsigned char lds_other[PIPE ? kStageBytes : 16];
  constexpr int kOffB = BM * kRowBytes;

  // Workgroup ids are dealt round-robin over the 8 XCDs, each with its own L2.  The row panels
  // of one column block get consecutive slots of ONE XCD, so its weights cross the fabric once
  // and the other panels find them in that L2 (x, the smaller operand, is re-read instead).
  uint32_t mb, nb;
  {
    const uint32_t id = blockIdx.x;
    if (8 % m_blocks == 0) {
      const uint32_t xcd = id & 7, slot = id >> 3;
      mb = slot % m_blocks;
      nb = (slot / m_blocks) * 8 + xcd;
    } else {
      mb = id % m_blocks;
      nb = id / m_blocks;
    }
    if (nb >= n_blocks) return;
  }
  const uint32_t m0 = mb * BM, n0 = nb * BN;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WM, wn = (wave / WM) % WN, kg = wave / (WM * WN);

  const uint32_t words_per_row = k >> 3;
  const uint32_t groups_per_row = k >> group_shift;
  const uint32_t chunks = (k + KC - 1) / KC;

  // staging assignment: element offsets of the thread's pieces at chunk 0 (rows past M or N
  // re-read the last row; their products are never stored)
  uint32_t a_off[kAPer], a_lds[kAPer], a_k[kAPer];
#pragma unroll
  for (int i = 0; i < kAPer; ++i) {
    const int p = tid + i * kThreads;
    const uint32_t row = p / kRowPieces, pc = p % kRowPieces;
    a_off[i] = min(row, m - 1 - m0) * k + pc * 8;  // relative to the tile's first row
    a_k[i] = pc * 8;
    a_lds[i] = row * kRowBytes + pc * 16;
  }
  const uint32_t b_row = (tid * kBPer) / kRowPieces;
  const uint32_t b_w0 = (tid * kBPer) % kRowPieces;
  const uint32_t b_grow = min(n0 + b_row, n - 1);
  const uint32_t* b_src = w + (size_t)b_grow * words_per_row + b_w0;
  const size_t b_scale_row = (size_t)b_grow * groups_per_row;

  const XT* x_tile = x + (size_t)m0 * k;
  // A chunk's operands as they arrive from memory.  DEPTH of them are in flight: chunk c + DEPTH
  // is requested as soon as chunk c has been parked in LDS.
  struct Slot {
    Acts8<XT> a[kAPer];
    uint32_t b[kBPer];
    uint32_t scale[kBPer];  // raw bits, see scale_bits
  };
  // a thread's words are consecutive and aligned to their count, so they share one scale
  // whenever a group covers them all
  const bool one_scale = ((uint32_t)(kBPer * 8 - 1) >> group_shift) == 0;

  // FAST (16-byte aligned rows, one scale per thread, K a multiple of KC): a fetch is the same
  // straight run of loads for every chunk, so waits on an older chunk can be counted and the
  // younger requests stay in flight.  Any branch here would cost that.
  auto fetch = [&](uint32_t chunk, Slot& slot) {
    const uint32_t k0 = chunk * KC;
    if constexpr (FAST) {
#pragma unroll
      for (int i = 0; i < kAPer; ++i) slot.a[i].load(x_tile + a_off[i] + k0);
#pragma unroll
      for (int j = 0; j + 3 < kBPer; j += 4) {
        const uint4 v = *reinterpret_cast<const uint4*>(b_src + (k0 >> 3) + j);
        slot.b[j] = v.x; slot.b[j + 1] = v.y; slot.b[j + 2] = v.z; slot.b[j + 3] = v.w;
      }
      slot.scale[0] = scale_bits<ST>(scales, b_scale_row + ((k0 + b_w0 * 8) >> group_shift));
    } else if (k0 + KC <= k) {  // uniform: the whole chunk lies inside K
#pragma unroll
      for (int i = 0; i < kAPer; ++i) slot.a[i].load(x_tile + a_off[i] + k0);
      if (kBPer >= 4 && wide_rows) {
#pragma unroll
        for (int j = 0; j + 3 < kBPer; j += 4) {
          const uint4 v = *reinterpret_cast<const uint4*>(b_src + (k0 >> 3) + j);
          slot.b[j] = v.x; slot.b[j + 1] = v.y; slot.b[j + 2] = v.z; slot.b[j + 3] = v.w;
        }
      } else {
#pragma unroll
        for (int j = 0; j < kBPer; ++j) slot.b[j] = b_src[(k0 >> 3) + j];
      }
      if (one_scale) {  // only scale[0] is loaded (no copies: a copy would wait for the load)
        slot.scale[0] = scale_bits<ST>(scales, b_scale_row + ((k0 + b_w0 * 8) >> group_shift));
      } else {
#pragma unroll
        for (int j = 0; j < kBPer; ++j)
          slot.scale[j] =
              scale_bits<ST>(scales, b_scale_row + ((k0 + (b_w0 + j) * 8) >> group_shift));
      }
    } else {  // last chunk of a K that is not a multiple of KC: zero activations past K
#pragma unroll
      for (int i = 0; i < kAPer; ++i) {
        const bool inside = k0 + a_k[i] < k;
        slot.a[i].load(x_tile + a_off[i] + (inside ? k0 : 0u));
        slot.a[i].keep(inside ? 0xFFFFFFFFu : 0u);
      }
#pragma unroll
      for (int j = 0; j < kBPer; ++j) {
        const uint32_t kk = k0 + (b_w0 + j) * 8;
        const uint32_t kc = kk < k ? kk : 0u;  // x is zero there; any finite weight will do
        slot.b[j] = w[(size_t)b_grow * words_per_row + (kc >> 3)];
        slot.scale[j] = scale_bits<ST>(scales, b_scale_row + (kc >> group_shift));
      }
    }
  };
  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int frag_row = lane & 31, frag_g = lane >> 5;
  const int a_frag = (wm * 64 + frag_row) * kRowBytes + frag_g * 16 + kg * kStepsPerGroup * 32;
  const int b_frag =
      kOffB + (wn * 64 + frag_row) * kRowBytes + frag_g * 16 + kg * kStepsPerGroup * 32;

  // `ragged`: the chunk reaches past K and carries one scale per word
  auto stage = [&](const Slot& slot, bool ragged, int buf) {
#pragma unroll
    for (int i = 0; i < kAPer; ++i)
      *reinterpret_cast<uint4*>(&(buf ? lds_other : lds)[a_lds[i]]) = slot.a[i].paired();
#pragma unroll
    for (int j = 0; j < kBPer; ++j)
      *reinterpret_cast<uint4*>(&(buf ? lds_other : lds)[kOffB + b_row * kRowBytes + (b_w0 + j) * 16]) =
          dequant_word(slot.b[j], scale_from_bits<ST>(
                                      slot.scale[(FAST || (one_scale && !ragged)) ? 0 : j]));
  };
  // All fragments of the chunk are requested before the first matrix instruction, so only the
  // first one waits for LDS.
  auto compute = [&](int buf) {
    half8_t af[kStepsPerGroup][2], bf[kStepsPerGroup][2];
#pragma unroll
    for (int ks = 0; ks < kStepsPerGroup; ++ks) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
        af[ks][i] = *reinterpret_cast<const half8_t*>(
            &(buf ? lds_other : lds)[a_frag + i * 32 * kRowBytes + ks * 32]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        bf[ks][j] = *reinterpret_cast<const half8_t*>(
            &(buf ? lds_other : lds)[b_frag + j * 32 * kRowBytes + ks * 32]);
    }
#pragma unroll
    for (int ks = 0; ks < kStepsPerGroup; ++ks)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] =
              __builtin_amdgcn_mfma_f32_32x32x16_f16(af[ks][i], bf[ks][j], acc[i][j], 0, 0, 0);
  };
  if constexpr (PIPE) {
    // chunk c travels slot[c % DEPTH] -> LDS copy c % 2 (DEPTH is even); DEPTH - 1 chunks are
    // in flight behind the one being parked
    static_assert(DEPTH % 2 == 0, "the LDS copy of a slot is fixed");
    Slot slots[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if constexpr (FAST) {
        fetch(min((uint32_t)d, chunks - 1), slots[d]);
      } else {
        if ((uint32_t)d < chunks) fetch(d, slots[d]);
      }
    }
    stage(slots[0], KC > k, 0);
    if constexpr (FAST) {
      fetch(min((uint32_t)DEPTH, chunks - 1), slots[0]);
    } else {
      if ((uint32_t)DEPTH < chunks) fetch(DEPTH, slots[0]);
    }
    __syncthreads();
    // steady state: every body parks its successor; straight-line code so the staging and the
    // matrix instructions can be interleaved
    auto body = [&](uint32_t chunk, int d) {
      const int nd = (d + 1) % DEPTH;
      stage(slots[nd], (chunk + 1) * KC + KC > k, nd % 2);
      compute(d % 2);
      // one matrix instruction, then a share of the staging work, in turn
      constexpr int kMfmas = kStepsPerGroup * 4;
      constexpr int kLead = kMfmas >= 8 ? 8 : kMfmas;  // fragment reads ahead of the first MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, kLead, 0);
#pragma unroll
      for (int i = 0; i < kMfmas; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, kStageValuPerMfma, 0);
        if (i < kMfmas - kLead) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (i % 2) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      }
      if constexpr (FAST) {
        fetch(min(chunk + 1 + DEPTH, chunks - 1), slots[nd]);  // past the end: a harmless re-read
      } else {
        if (chunk + 1 + DEPTH < chunks) fetch(chunk + 1 + DEPTH, slots[nd]);
      }
      __syncthreads();
    };
    uint32_t chunk = 0;
    for (; chunk + DEPTH < chunks; chunk += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) body(chunk + d, d);
    }
    // the last 1..DEPTH chunks: the final one has no successor to park
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (chunk + d + 1 < chunks) {
        body(chunk + d, d);
      } else if (chunk + d < chunks) {
        compute(d % 2);
      }
    }
    __syncthreads();
  } else {
    Slot slots[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if constexpr (FAST) {
        fetch(min((uint32_t)d, chunks - 1), slots[d]);
      } else {
        if ((uint32_t)d < chunks) fetch(d, slots[d]);
      }
    }
    for (uint32_t base = 0; base < chunks; base += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {  // unrolled: every slot has fixed registers
        const uint32_t chunk = base + d;
        if (chunk >= chunks) break;
        stage(slots[d], chunk * KC + KC > k, 0);
        __syncthreads();
        if constexpr (FAST) {
          fetch(min(chunk + DEPTH, chunks - 1), slots[d]);  // past the end: a harmless re-read
        } else {
          if (chunk + DEPTH < chunks) fetch(chunk + DEPTH, slots[d]);
        }
        compute(0);
        __syncthreads();  // every wave is done with this chunk before the next one is parked
      }
    }
  }

  if constexpr (KS > 1) {
    // Sum of the K groups, group 0 + 1 + ... in that order; the tile's LDS is free again (the
    // loop ended on a barrier).  Word (r, lane) of a wave's 64 x 64 block: conflict-free.
    float* red = reinterpret_cast<float*>(lds);
    if (kg > 0) {
      float* dst = red + (size_t)(((kg - 1) * WN + wn) * WM + wm) * 64 * 64;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) dst[((i * 2 + j) * 16 + r) * 64 + lane] = acc[i][j][r];
    }
    __syncthreads();
    if (kg > 0) return;
#pragma unroll
    for (int g = 1; g < KS; ++g) {
      const float* src = red + (size_t)(((g - 1) * WN + wn) * WM + wm) * 64 * 64;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][j][r] += src[((i * 2 + j) * 16 + r) * 64 + lane];
    }
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

// ---------------------------------------------------------------- packed weights in LDS
//
// Eight waves, workgroup tile (64 * MT) x 256, wave (wm, wn) = 32 * MT rows x 64 columns, K in
// stages of 128 codes.  The weight bytes are staged as they are — coalesced 16-byte loads, a
// quarter of the LDS bytes the dequantised fp16 tile takes — and every wave dequantises the
// words of its own 64 columns after reading them back: lane (n = lane % 32, h = lane / 32)
// reads 16 bytes = codes 64c + 32h .. + 31 of column n per 64-code chunk, word j of which is
// the B operand of the chunk's MFMA step j (fp16(u - 8) * fp16(scale), order
// c0,c4,c1,c5,c2,c6,c3,c7); the A operand of that step is x[m][64c + 32h + 8j ..] in the
// same order, 16 bytes of the staged x row.  The same arithmetic as the kernel above, so the
// two agree up to the order of the f32 additions.  Two waves share a SIMD: one wave's
// dequantisation runs under the other's MFMAs.  Every stage issues the same loads whatever K
// is (clamped addresses; x past K is parked as zeros).
template <typename XT, typename ST, int MT>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_i4_f16_packed_kernel(const XT* __restrict__ x, const uint8_t* __restrict__ w,
                               const ST* __restrict__ scales, const XT* __restrict__ bias,
                               XT* __restrict__ out, uint32_t m, uint32_t n, uint32_t k,
                               uint32_t group_shift, uint32_t m_blocks, uint32_t n_blocks) {
  constexpr int WN = 2;
  constexpr int BM = 2 * 32 * MT, BN = 256;
  constexpr int kStage = 128;                 // codes per LDS stage
  constexpr int kRowA = kStage * 2 + 16;      // bytes per LDS row of fp16 x
  constexpr int kRowB = kStage / 2 + 16;      // bytes per LDS row of packed weights
  constexpr int kAUnits = BM * (kStage / 8) / 512;  // 8-element units of x per thread and stage
  __shared__ __align__(16) uint8_t s_a[2][BM * kRowA];
  __shared__ __align__(16) uint8_t s_b[2][BN * kRowB];
  __shared__ _Float16 s_s[2][BN][2];

  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
  const uint32_t mb = slot % m_blocks, nb = (slot / m_blocks) * 8u + xcd;
  if (nb >= n_blocks) return;  // the whole workgroup leaves before any barrier
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  const int frag_row = lane & 31, frag_h = lane >> 5;
  const uint32_t m0 = mb * BM, n0 = nb * BN;
  const uint32_t groups = k >> group_shift;
  const uint32_t stages = (k + kStage - 1) / kStage;

  // staging roles: x rows in 16 units of 8 elements (rows tid / 16 + 32 i), weight rows in 4
  // units of 16 bytes (rows tid / 4 + 128 i), one scale row per thread of the first four waves
  const uint32_t arow0 = tid >> 4, aunit = (tid & 15u) * 8u;      // element offset in the stage
  const uint32_t brow0 = tid >> 2, bunit = (tid & 3u) * 16u;      // byte offset in the stage
  const ST* ssrc = scales + (size_t)min(n0 + (uint32_t)(tid & 255), n - 1) * groups;

  struct Staged {
    Acts8<XT> a[kAUnits];
    uint4 b[2];
  };
  auto load_stage = [&](uint32_t stage, Staged& d) {
    const uint32_t a_at = stage * kStage + aunit, b_at = stage * (kStage / 2) + bunit;
    const uint32_t a_off = a_at < k ? a_at : 0u, b_off = b_at < (k >> 1) ? b_at : 0u;
#pragma unroll
    for (int i = 0; i < kAUnits; ++i)
      d.a[i].load(x + (size_t)min(m0 + arow0 + 32u * i, m - 1) * k + a_off);
#pragma unroll
    for (int i = 0; i < 2; ++i)
      d.b[i] = *reinterpret_cast<const uint4*>(
          w + (size_t)min(n0 + brow0 + 128u * i, n - 1) * (k >> 1) + b_off);
  };
  auto park_stage = [&](uint32_t stage, int buf, Staged& d) {
    const uint32_t keep = stage * kStage + aunit < k ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int i = 0; i < kAUnits; ++i) {
      uint4 v = d.a[i].paired();
      v.x &= keep; v.y &= keep; v.z &= keep; v.w &= keep;  // past K: zeros, whatever B holds
      *reinterpret_cast<uint4*>(&s_a[buf][(arow0 + 32u * i) * kRowA + aunit * 2u]) = v;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
      *reinterpret_cast<uint4*>(&s_b[buf][(brow0 + 128u * i) * kRowB + bunit]) = d.b[i];
    // The stage's (at most two) group scales of this thread's column, fetched here by the first
    // four waves.  (Requested a stage ahead like the tiles, or all at once into an LDS table,
    // measured 5-8 % slower: every lane's scale sits in another cache line.)
    if (tid < 256) {
      const uint32_t c0 = stage * kStage, c1 = stage * kStage + 64u;
      s_s[buf][tid][0] = scale_from_bits<ST>(scale_bits<ST>(ssrc, (c0 < k ? c0 : 0u) >> group_shift));
      s_s[buf][tid][1] = scale_from_bits<ST>(scale_bits<ST>(ssrc, (c1 < k ? c1 : 0u) >> group_shift));
    }
  };

  float16_t acc[MT][WN];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < WN; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.f;

  Staged staged;
  load_stage(0, staged);
  park_stage(0, 0, staged);
  __syncthreads();

  const uint32_t a_base = (uint32_t)((wm * 32 * MT + frag_row) * kRowA + 64 * frag_h);
  const uint32_t b_base = (uint32_t)((wn * 64 + frag_row) * kRowB + 16 * frag_h);
  auto run_stage = [&](uint32_t stage, int buf) {
    load_stage(stage + 1, staged);
    // the requests stay here, a whole stage ahead of their use (left alone, the scheduler
    // moves them down to the parking code, where their latency is in the open)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      uint4 braw[WN];
      _Float16 ws[WN];
#pragma unroll
      for (int nt = 0; nt < WN; ++nt) {
        braw[nt] = *reinterpret_cast<const uint4*>(&s_b[buf][b_base + nt * 32 * kRowB + 32 * c]);
        ws[nt] = s_s[buf][wn * 64 + nt * 32 + frag_row][c];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        half8_t a[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          a[mt] = *reinterpret_cast<const half8_t*>(
              &s_a[buf][a_base + mt * 32 * kRowA + 128 * c + 16 * j]);
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) {
          const uint32_t word = j == 0 ? braw[nt].x : j == 1 ? braw[nt].y : j == 2 ? braw[nt].z
                                                                                  : braw[nt].w;
          const half8_t b = __builtin_bit_cast(half8_t, dequant_word(word, ws[nt]));
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt], b, acc[mt][nt], 0, 0, 0);
        }
      }
    }
    park_stage(stage + 1, buf ^ 1, staged);
    __syncthreads();
  };
  for (uint32_t stage = 0; stage < stages; stage += 2) {
    run_stage(stage, 0);
    run_stage(stage + 1, 1);  // past the last stage: x is zeros
  }

#pragma unroll
  for (int nt = 0; nt < WN; ++nt) {
    const uint32_t col = n0 + wn * 64 + nt * 32 + frag_row;
    const float b = (bias && col < n) ? bias_f32<XT>(bias, col) : 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const uint32_t row = m0 + wm * 32 * MT + mt * 32 + 8 * (r / 4) + 4 * frag_h + (r % 4);
        if (row < m && col < n) store_out<XT>(out, (size_t)row * n + col, acc[mt][nt][r] + b);
      }
  }
}

// ------------------------------------------------ packed weights in LDS, K dealt by units
//
// The same 128 x 256 tile and stage loop as above, for outputs whose tiles do not fill the
// chip evenly (172 tiles on 256 CUs leave a third idle; 64 tiles three quarters).  The work is
// the list of (tile, stage) units, tiles in column-block-major order; it is cut into one
// contiguous range per workgroup (the grid is one workgroup per CU, ranges differ by at most
// one unit), so a tile is computed by up to a few workgroups, each over a slice of K.  A
// workgroup that computes a whole tile stores it.  Otherwise it writes its 128 x 256 f32
// partial (device-scope stores, each thread its own registers, 16 bytes at a time), waits for
// the stores, and takes a ticket on the tile's counter; the workgroup that arrives last adds
// the partials in ascending K order — its own from registers — so the bits do not depend on
// who arrives last.  No workgroup ever waits for another.
struct UnitDeal {
  uint32_t stages_per_tile;
  uint32_t units_lo, extra;  // workgroup v owns units_lo + (v < extra) units from deal_begin(v)
  float* partials;           // [2 * workgroups] slots of 128 x 256 floats
  uint32_t* tickets;         // one counter per tile, kTicketStride words apart, zero at rest
};
__host__ __device__ inline uint32_t deal_begin(const UnitDeal& d, uint32_t v) {
  return v * d.units_lo + (v < d.extra ? v : d.extra);
}
__device__ inline uint32_t deal_owner(const UnitDeal& d, uint32_t unit) {
  const uint32_t big = d.extra * (d.units_lo + 1u);
  return unit < big ? unit / (d.units_lo + 1u) : d.extra + (unit - big) / d.units_lo;
}
constexpr uint32_t kPartialFloats = 128u * 256u;

typedef float float4_t __attribute__((ext_vector_type(4)));
// 16 bytes written through to / read from memory that every XCD sees (device scope).
__device__ inline void publish4(float4_t* p, float4_t v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ inline float4_t observe4(const float4_t* p) {
  float4_t v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
  return v;
}
// The eight requests above have landed; the values pass through so that no use moves ahead.
__device__ inline void landed(float4_t (&p)[8]) {
  asm volatile("s_waitcnt vmcnt(0)"
               : "+v"(p[0]), "+v"(p[1]), "+v"(p[2]), "+v"(p[3]), "+v"(p[4]), "+v"(p[5]), "+v"(p[6]),
                 "+v"(p[7])::"memory");
}

// WM = 2 (the one in use): eight waves, wave = 64 x 64, two waves a SIMD, as above.  WM = 1: four
// waves, wave = 128 x 64, every weight word dequantised once for four MFMAs instead of twice for
// two — measured 101 us against 78 us on the 512 x 11008 x 4096 product: the single wave of a
// SIMD does not hide its own LDS reads and dequantisation under its MFMAs as compiled (and
// spills 31 registers).
template <typename XT, typename ST, int WM>
__global__ __launch_bounds__(WM * 256) __attribute__((amdgpu_waves_per_eu(WM, WM)))
void gemm_i4_f16_dealt_kernel(const XT* __restrict__ x, const uint8_t* __restrict__ w,
                              const ST* __restrict__ scales, const XT* __restrict__ bias,
                              XT* __restrict__ out, uint32_t m, uint32_t n, uint32_t k,
                              uint32_t group_shift, uint32_t m_blocks, UnitDeal deal) {
  constexpr int MT = 4 / WM, WN = 2;
  constexpr int T = WM * 256;  // threads
  constexpr int BM = WM * 32 * MT, BN = 256;
  static_assert(BM == 128, "the partial layout and the deal assume 128 x 256 tiles");
  constexpr int kStage = 128;
  constexpr int kRowA = kStage * 2 + 16;
  constexpr int kRowB = kStage / 2 + 16;
  constexpr int kAUnits = BM * (kStage / 8) / T;
  constexpr int kBUnits = BN * (kStage / 32) / T;
  __shared__ __align__(16) uint8_t s_a[2][BM * kRowA];
  __shared__ __align__(16) uint8_t s_b[2][BN * kRowB];
  __shared__ _Float16 s_s[2][BN][2];
  __shared__ uint32_t s_ticket;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  const int frag_row = lane & 31, frag_h = lane >> 5;
  const uint32_t groups = k >> group_shift;
  const uint32_t spt = deal.stages_per_tile;
  const uint32_t arow0 = tid >> 4, aunit = (tid & 15u) * 8u;
  const uint32_t brow0 = tid >> 2, bunit = (tid & 3u) * 16u;
  const uint32_t a_base = (uint32_t)((wm * 32 * MT + frag_row) * kRowA + 64 * frag_h);
  const uint32_t b_base = (uint32_t)((wn * 64 + frag_row) * kRowB + 16 * frag_h);

  // the workgroups of one XCD (ids equal mod 8) take neighbouring ranges: the row panels of a
  // column block then mostly share an L2
  uint32_t v = blockIdx.x;
  if ((gridDim.x & 7u) == 0) v = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const uint32_t my_begin = deal_begin(deal, v);
  uint32_t left = deal.units_lo + (v < deal.extra ? 1u : 0u);

  // The tiles of the range are taken last to first: a range usually ends with the first stages
  // of a tile and begins with the last stages of the one before, so every workgroup then walks
  // K upwards from (about) stage 0 and, at any moment, the chip reads few distinct K slices of
  // x, which stay in the L2s.
  while (left > 0) {
    const uint32_t range_end = my_begin + left;
    const uint32_t tile = (range_end - 1u) / spt;
    const uint32_t tile_first = tile * spt;
    const uint32_t s0 = my_begin > tile_first ? my_begin - tile_first : 0u;
    const uint32_t s1 = range_end - tile_first;
    const uint32_t nb = tile / m_blocks, mb = tile - nb * m_blocks;
    const uint32_t m0 = mb * BM, n0 = nb * BN;
    const ST* ssrc = scales + (size_t)min(n0 + (uint32_t)(tid & 255), n - 1) * groups;

    struct Staged {
      Acts8<XT> a[kAUnits];
      uint4 b[kBUnits];
    };
    auto load_stage = [&](uint32_t stage, Staged& d) {
      const uint32_t a_at = stage * kStage + aunit, b_at = stage * (kStage / 2) + bunit;
      const uint32_t a_off = a_at < k ? a_at : 0u, b_off = b_at < (k >> 1) ? b_at : 0u;
#pragma unroll
      for (int i = 0; i < kAUnits; ++i)
        d.a[i].load(x + (size_t)min(m0 + arow0 + (uint32_t)(T / 16) * i, m - 1) * k + a_off);
#pragma unroll
      for (int i = 0; i < kBUnits; ++i)
        d.b[i] = *reinterpret_cast<const uint4*>(
            w + (size_t)min(n0 + brow0 + (uint32_t)(T / 4) * i, n - 1) * (k >> 1) + b_off);
    };
    auto park_stage = [&](uint32_t stage, int buf, Staged& d) {
      const uint32_t keep = stage * kStage + aunit < k ? 0xFFFFFFFFu : 0u;
#pragma unroll
      for (int i = 0; i < kAUnits; ++i) {
        uint4 pv = d.a[i].paired();
        pv.x &= keep; pv.y &= keep; pv.z &= keep; pv.w &= keep;
        *reinterpret_cast<uint4*>(&s_a[buf][(arow0 + (uint32_t)(T / 16) * i) * kRowA + aunit * 2u]) = pv;
      }
#pragma unroll
      for (int i = 0; i < kBUnits; ++i)
        *reinterpret_cast<uint4*>(&s_b[buf][(brow0 + (uint32_t)(T / 4) * i) * kRowB + bunit]) = d.b[i];
      if (tid < 256) {
        const uint32_t c0 = stage * kStage, c1 = stage * kStage + 64u;
        s_s[buf][tid][0] = scale_from_bits<ST>(scale_bits<ST>(ssrc, (c0 < k ? c0 : 0u) >> group_shift));
        s_s[buf][tid][1] = scale_from_bits<ST>(scale_bits<ST>(ssrc, (c1 < k ? c1 : 0u) >> group_shift));
      }
    };

    float16_t acc[MT][WN];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < WN; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.f;

    Staged staged;
    load_stage(s0, staged);
    park_stage(s0, 0, staged);
    __syncthreads();

    auto run_stage = [&](uint32_t stage, int buf) {
      load_stage(stage + 1, staged);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        uint4 braw[WN];
        _Float16 ws[WN];
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) {
          braw[nt] = *reinterpret_cast<const uint4*>(&s_b[buf][b_base + nt * 32 * kRowB + 32 * c]);
          ws[nt] = s_s[buf][wn * 64 + nt * 32 + frag_row][c];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          half8_t a[MT];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            a[mt] = *reinterpret_cast<const half8_t*>(
                &s_a[buf][a_base + mt * 32 * kRowA + 128 * c + 16 * j]);
#pragma unroll
          for (int nt = 0; nt < WN; ++nt) {
            const uint32_t word = j == 0 ? braw[nt].x : j == 1 ? braw[nt].y : j == 2 ? braw[nt].z
                                                                                    : braw[nt].w;
            const half8_t b = __builtin_bit_cast(half8_t, dequant_word(word, ws[nt]));
            // the wave that feeds the matrix pipe goes first; the other one dequantises meanwhile
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt], b, acc[mt][nt], 0, 0, 0);
            __builtin_amdgcn_s_setprio(0);
          }
        }
      }
      park_stage(stage + 1, buf ^ 1, staged);
      __syncthreads();
    };
    for (uint32_t stage = s0; stage < s1; stage += 2) {
      run_stage(stage, 0);
      if (stage + 1 < s1) run_stage(stage + 1, 1);
    }

    auto store_block = [&](int mt, int nt, const float16_t& total) {
      const uint32_t col = n0 + wn * 64 + nt * 32 + frag_row;
      const float b = (bias && col < n) ? bias_f32<XT>(bias, col) : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const uint32_t row = m0 + wm * 32 * MT + mt * 32 + 8 * (r / 4) + 4 * frag_h + (r % 4);
        if (row < m && col < n) store_out<XT>(out, (size_t)row * n + col, total[r] + b);
      }
    };

    if (s0 == 0 && s1 == spt) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) store_block(mt, nt, acc[mt][nt]);
    } else {
      // Slot of workgroup u's partial of this tile: its second slot when its range began at or
      // before the tile's first unit, its first slot otherwise (a range holds at most one
      // partial of either kind).  16-byte piece c of thread t sits at [c * threads + t].
      const uint32_t tile_begin = tile * spt;
      auto slot_of = [&](uint32_t u) {
        return 2u * u + (deal_begin(deal, u) <= tile_begin ? 1u : 0u);
      };
      uint32_t* ticket = deal.tickets + (size_t)tile * kTicketStride;
      const uint32_t first = deal_owner(deal, tile_begin), last = deal_owner(deal, tile_begin + spt - 1u);
      // Every other partial already there (the usual case for the slice computed last: slices
      // that open a range finish early)?  Then this one need not be written at all.
      if (tid == 0)
        s_ticket = __hip_atomic_load(ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      bool merge = s_ticket == last - first;
      __syncthreads();  // s_ticket is written again below
      if (!merge) {
        float4_t* mine =
            reinterpret_cast<float4_t*>(deal.partials + (size_t)slot_of(v) * kPartialFloats);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int nt = 0; nt < WN; ++nt)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float4_t piece = {acc[mt][nt][4 * q], acc[mt][nt][4 * q + 1],
                                      acc[mt][nt][4 * q + 2], acc[mt][nt][4 * q + 3]};
              publish4(mine + (size_t)(((mt * WN + nt) * 4 + q) * T + tid), piece);
            }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's partial is in memory
        __syncthreads();
        if (tid == 0)
          s_ticket = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        merge = s_ticket == last - first;  // arrived last after all
      }
      if (merge) {  // every other partial of the tile is complete
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          float16_t total[WN];
          for (uint32_t u = first; u <= last; ++u) {
            float16_t part[WN];
#pragma unroll
            for (int nt = 0; nt < WN; ++nt) part[nt] = acc[mt][nt];
            if (u != v) {
              const float4_t* src =
                  reinterpret_cast<const float4_t*>(deal.partials + (size_t)slot_of(u) * kPartialFloats) +
                  (size_t)(mt * WN * 4 * T + tid);
              float4_t p[8];
#pragma unroll
              for (int i = 0; i < 8; ++i) p[i] = observe4(src + (size_t)i * T);
              landed(p);
#pragma unroll
              for (int nt = 0; nt < WN; ++nt)
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                  for (int i = 0; i < 4; ++i) part[nt][4 * q + i] = p[nt * 4 + q][i];
            }
#pragma unroll
            for (int nt = 0; nt < WN; ++nt) {
              if (u == first) {
                total[nt] = part[nt];
              } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) total[nt][r] += part[nt][r];
              }
            }
          }
#pragma unroll
          for (int nt = 0; nt < WN; ++nt) store_block(mt, nt, total[nt]);
        }
        if (tid == 0)
          __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    left -= s1 - s0;
  }
}

// ------------------------------------------------ exact integer operands, 64 x 512 tiles
//
// The weights enter the matrix cores as the exact integers (u - 8) in fp16 and the group scale
// multiplies the f32 sum of a group afterwards — the arithmetic of the GEMV, on MFMA.  Two
// activation forms:
//   kOperandF16  x is rounded to fp16 once (exact when it already is fp16): one MFMA a step;
//   kOperandSplit  f32 x is split as x * 2^e = hi + lo, both fp16, |x * 2^e - (hi + lo)| <=
//                2^-23 |x * 2^e| (e per row, chosen so that the row's largest magnitude lands in
//                [2^13, 2^14): no overflow, and small entries keep an absolute resolution of
//                2^-38 of the row's maximum): two MFMAs a step, products exact, f32 sums —
//                the class of the reference's default f32 `linear`, on the matrix cores.
// Tile 64 x 512, eight waves side by side (wave = 64 rows x 64 columns = 2 x 2 MFMA tiles), so
// every weight word is turned into integers exactly once per workgroup (in the 128 x 256 tile
// above the two waves of a column strip each do it).  Per MFMA step the wave holds the sums of
// the current scale group in `acc`; at a group's end total = fma(acc, scale[column], total)
// (the C layout keeps the column in lane % 32, so the scale is one value per lane and column
// tile).  Stages, LDS layout, the (tile, stage) deal over the CUs and the ordered merge of the
// partials are those of the kernel above.
constexpr int kOperandF16 = 0, kOperandSplit = 1;

// 8 codes of a word -> 8 fp16 integers (u - 8), order (c0,c4,c1,c5,c2,c6,c3,c7).
__device__ inline uint4 ints_word(uint32_t word) {
  const uint32_t magic = 0x64006400u;  // (1024, 1024)
  const half2_t off_lo = {(_Float16)1032.0f, (_Float16)1032.0f};
  const half2_t sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  const half2_t off_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
  const uint32_t upper = word >> 8;
  const half2_t q0 = __builtin_bit_cast(half2_t, and_or(word, 0x000F000Fu, magic)) - off_lo;
  const half2_t q1 = __builtin_elementwise_fma(
      __builtin_bit_cast(half2_t, and_or(word, 0x00F000F0u, magic)), sixteenth, off_hi);
  const half2_t q2 = __builtin_bit_cast(half2_t, and_or(upper, 0x000F000Fu, magic)) - off_lo;
  const half2_t q3 = __builtin_elementwise_fma(
      __builtin_bit_cast(half2_t, and_or(upper, 0x00F000F0u, magic)), sixteenth, off_hi);
  return make_uint4(__builtin_bit_cast(uint32_t, q0), __builtin_bit_cast(uint32_t, q1),
                    __builtin_bit_cast(uint32_t, q2), __builtin_bit_cast(uint32_t, q3));
}

// x * scale = hi + lo for eight f32 activations, both halves in the paired order.
__device__ inline void split_paired(const uint4& a, const uint4& b, float scale, uint4& hi,
                                    uint4& lo) {
  const float v[8] = {__uint_as_float(a.x), __uint_as_float(a.y), __uint_as_float(a.z),
                      __uint_as_float(a.w), __uint_as_float(b.x), __uint_as_float(b.y),
                      __uint_as_float(b.z), __uint_as_float(b.w)};
  _Float16 h[8], l[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float xs = v[i] * scale;             // exact: a power of two
    h[i] = (_Float16)xs;                       // round to nearest even
    l[i] = (_Float16)(xs - (float)h[i]);       // the difference is exact in f32
  }
  auto pack = [](_Float16 p, _Float16 q) {
    const half2_t t = {p, q};
    return __builtin_bit_cast(uint32_t, t);
  };
  hi = make_uint4(pack(h[0], h[4]), pack(h[1], h[5]), pack(h[2], h[6]), pack(h[3], h[7]));
  lo = make_uint4(pack(l[0], l[4]), pack(l[1], l[5]), pack(l[2], l[6]), pack(l[3], l[7]));
}

// Row scales of the split form: scale[2r] = 2^e with max|x[r, :]| * 2^e in [2^13, 2^14),
// scale[2r + 1] = 2^-e.  A row of zeros (or whose maximum is not finite) gets 1 / 1: what is
// not finite stays so through the product.
__global__ __launch_bounds__(256) void row_scale_kernel(const float* __restrict__ x,
                                                        float* __restrict__ row_scale, uint32_t k) {
  __shared__ uint32_t s_max[4];
  const float* row = x + (size_t)blockIdx.x * k;
  uint32_t top = 0;  // largest |x| as raw bits (monotonic for non-negative floats; NaN on top)
  const uint32_t pieces = k >> 2;
  for (uint32_t i = threadIdx.x; i < pieces; i += 256) {
    const uint4 v = reinterpret_cast<const uint4*>(row)[i];
    top = max(max(top, v.x & 0x7fffffffu), max(v.y & 0x7fffffffu, max(v.z & 0x7fffffffu, v.w & 0x7fffffffu)));
  }
  for (uint32_t i = (pieces << 2) + threadIdx.x; i < k; i += 256)
    top = max(top, __float_as_uint(row[i]) & 0x7fffffffu);
  for (int off = 32; off > 0; off >>= 1) top = max(top, (uint32_t)__shfl_xor((int)top, off, kWave));
  if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = top;
  __syncthreads();
  if (threadIdx.x == 0) {
    top = max(max(s_max[0], s_max[1]), max(s_max[2], s_max[3]));
    const uint32_t biased = top >> 23;  // exponent of the maximum
    uint32_t up = 127u, down = 127u;    // 2^0
    if (top != 0 && biased != 255u) {
      // e = 13 - (biased - 127), kept inside the normal range of both 2^e and 2^-e
      int e = 13 - ((int)biased - 127);
      e = e > 126 ? 126 : (e < -126 ? -126 : e);
      up = (uint32_t)(127 + e);
      down = (uint32_t)(127 - e);
    }
    row_scale[2 * (size_t)blockIdx.x] = __uint_as_float(up << 23);
    row_scale[2 * (size_t)blockIdx.x + 1] = __uint_as_float(down << 23);
  }
}

template <typename XT, typename ST, int OPERAND>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_i4_exact_kernel(const XT* __restrict__ x, const uint8_t* __restrict__ w,
                          const ST* __restrict__ scales, const XT* __restrict__ bias,
                          XT* __restrict__ out, uint32_t m, uint32_t n, uint32_t k,
                          uint32_t group_shift, uint32_t m_blocks, UnitDeal deal,
                          const float* __restrict__ row_scale) {
  constexpr int MT = 2, WN = 2, T = 512;
  constexpr int BM = 64, BN = 512;
  constexpr int NA = OPERAND == kOperandSplit ? 2 : 1;  // copies of the x tile (hi, lo)
  constexpr int kStage = 128;
  constexpr int kRowA = kStage * 2 + 16;
  constexpr int kRowB = kStage / 2 + 16;
  constexpr int kAUnits = BM * (kStage / 8) / T;   // 2
  constexpr int kBUnits = BN * (kStage / 32) / T;  // 4
  static_assert((size_t)BM * BN == kPartialFloats, "the partial slots hold one tile");
  static_assert(OPERAND == kOperandF16 || sizeof(XT) == 4, "only f32 activations are split");
  __shared__ __align__(16) uint8_t s_a[2][NA][BM * kRowA];
  __shared__ __align__(16) uint8_t s_b[2][BN * kRowB];
  __shared__ float s_s[2][BN][2];
  __shared__ float s_inv[BM];
  __shared__ uint32_t s_ticket;

  const int tid = threadIdx.x, lane = tid & 63, wn = tid >> 6;
  const int frag_row = lane & 31, frag_h = lane >> 5;
  const uint32_t groups = k >> group_shift;
  const bool half_stage_groups = group_shift == 6;  // 64 codes a group: two groups a stage
  const uint32_t spt = deal.stages_per_tile;
  const uint32_t arow0 = tid >> 4, aunit = (tid & 15u) * 8u;
  const uint32_t brow0 = tid >> 2, bunit = (tid & 3u) * 16u;
  const uint32_t a_base = (uint32_t)(frag_row * kRowA + 64 * frag_h);
  const uint32_t b_base = (uint32_t)((wn * 64 + frag_row) * kRowB + 16 * frag_h);

  uint32_t v = blockIdx.x;
  if ((gridDim.x & 7u) == 0) v = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const uint32_t my_begin = deal_begin(deal, v);
  uint32_t left = deal.units_lo + (v < deal.extra ? 1u : 0u);

  while (left > 0) {
    const uint32_t range_end = my_begin + left;
    const uint32_t tile = (range_end - 1u) / spt;
    const uint32_t tile_first = tile * spt;
    const uint32_t s0 = my_begin > tile_first ? my_begin - tile_first : 0u;
    const uint32_t s1 = range_end - tile_first;
    const uint32_t nb = tile / m_blocks, mb = tile - nb * m_blocks;
    const uint32_t m0 = mb * BM, n0 = nb * BN;
    const ST* ssrc = scales + (size_t)min(n0 + (uint32_t)tid, n - 1) * groups;

    float rs[kAUnits];  // 2^e of the rows this thread stages
#pragma unroll
    for (int i = 0; i < kAUnits; ++i) rs[i] = 1.0f;
    if constexpr (OPERAND == kOperandSplit) {
#pragma unroll
      for (int i = 0; i < kAUnits; ++i)
        rs[i] = row_scale[2 * (size_t)min(m0 + arow0 + 32u * i, m - 1)];
      if (tid < BM) s_inv[tid] = row_scale[2 * (size_t)min(m0 + (uint32_t)tid, m - 1) + 1];
    }

    struct Staged {
      Acts8<XT> a[kAUnits];
      uint4 b[kBUnits];
    };
    auto load_stage = [&](uint32_t stage, Staged& d) {
      const uint32_t a_at = stage * kStage + aunit, b_at = stage * (kStage / 2) + bunit;
      const uint32_t a_off = a_at < k ? a_at : 0u, b_off = b_at < (k >> 1) ? b_at : 0u;
#pragma unroll
      for (int i = 0; i < kAUnits; ++i)
        d.a[i].load(x + (size_t)min(m0 + arow0 + 32u * i, m - 1) * k + a_off);
#pragma unroll
      for (int i = 0; i < kBUnits; ++i)
        d.b[i] = *reinterpret_cast<const uint4*>(
            w + (size_t)min(n0 + brow0 + 128u * i, n - 1) * (k >> 1) + b_off);
    };
    auto park_stage = [&](uint32_t stage, int buf, Staged& d) {
      const uint32_t keep = stage * kStage + aunit < k ? 0xFFFFFFFFu : 0u;
#pragma unroll
      for (int i = 0; i < kAUnits; ++i) {
        const uint32_t at = (arow0 + 32u * i) * kRowA + aunit * 2u;
        if constexpr (OPERAND == kOperandSplit) {
          uint4 hi, lo;
          split_paired(d.a[i].a, d.a[i].b, rs[i], hi, lo);
          hi.x &= keep; hi.y &= keep; hi.z &= keep; hi.w &= keep;  // past K: zeros
          lo.x &= keep; lo.y &= keep; lo.z &= keep; lo.w &= keep;
          *reinterpret_cast<uint4*>(&s_a[buf][0][at]) = hi;
          *reinterpret_cast<uint4*>(&s_a[buf][NA - 1][at]) = lo;
        } else {
          uint4 pv = d.a[i].paired();
          pv.x &= keep; pv.y &= keep; pv.z &= keep; pv.w &= keep;
          *reinterpret_cast<uint4*>(&s_a[buf][0][at]) = pv;
        }
      }
#pragma unroll
      for (int i = 0; i < kBUnits; ++i)
        *reinterpret_cast<uint4*>(&s_b[buf][(brow0 + 128u * i) * kRowB + bunit]) = d.b[i];
      const uint32_t c0 = stage * kStage, c1 = stage * kStage + 64u;
      s_s[buf][tid][0] = load_scale_f32<ST>(ssrc, (c0 < k ? c0 : 0u) >> group_shift);
      s_s[buf][tid][1] = load_scale_f32<ST>(ssrc, (c1 < k ? c1 : 0u) >> group_shift);
    };

    float16_t total[MT][WN], acc[MT][WN];
    float16_t zero16;
#pragma unroll
    for (int r = 0; r < 16; ++r) zero16[r] = 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < WN; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) total[mt][nt][r] = acc[mt][nt][r] = 0.f;

    Staged staged;
    load_stage(s0, staged);
    park_stage(s0, 0, staged);
    __syncthreads();

    auto run_stage = [&](uint32_t stage, int buf) {
      load_stage(stage + 1, staged);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        uint4 braw[WN];
        float ws[WN];
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) {
          braw[nt] = *reinterpret_cast<const uint4*>(&s_b[buf][b_base + nt * 32 * kRowB + 32 * c]);
          ws[nt] = s_s[buf][wn * 64 + nt * 32 + frag_row][c];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          half8_t a[NA][MT];
#pragma unroll
          for (int copy = 0; copy < NA; ++copy)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              a[copy][mt] = *reinterpret_cast<const half8_t*>(
                  &s_a[buf][copy][a_base + mt * 32 * kRowA + 128 * c + 16 * j]);
#pragma unroll
          for (int nt = 0; nt < WN; ++nt) {
            const uint32_t word = j == 0 ? braw[nt].x : j == 1 ? braw[nt].y : j == 2 ? braw[nt].z
                                                                                    : braw[nt].w;
            const half8_t b = __builtin_bit_cast(half8_t, ints_word(word));
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
              for (int copy = 0; copy < NA; ++copy) {
                // the first product of a scale group starts from zero (an inline constant of
                // the instruction: the sums are not cleared by VALU moves)
                const bool opens = copy == 0 && j == 0 && (c == 0 || half_stage_groups);
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                    a[copy][mt], b, opens ? zero16 : acc[mt][nt], 0, 0, 0);
              }
            }
            __builtin_amdgcn_s_setprio(0);
          }
        }
        if (c == 1 || half_stage_groups) {  // the scale group ends here
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < WN; ++nt)
#pragma unroll
              for (int r = 0; r < 16; ++r)
                total[mt][nt][r] = fmaf(acc[mt][nt][r], ws[nt], total[mt][nt][r]);
        }
      }
      park_stage(stage + 1, buf ^ 1, staged);
      __syncthreads();
    };
    for (uint32_t stage = s0; stage < s1; stage += 2) {
      run_stage(stage, 0);
      if (stage + 1 < s1) run_stage(stage + 1, 1);
    }

    auto store_block = [&](int mt, int nt, const float16_t& sum) {
      const uint32_t col = n0 + wn * 64 + nt * 32 + frag_row;
      const float b = (bias && col < n) ? bias_f32<XT>(bias, col) : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const uint32_t local = mt * 32 + 8 * (r / 4) + 4 * frag_h + (r % 4);
        const uint32_t row = m0 + local;
        float value = sum[r];
        if constexpr (OPERAND == kOperandSplit) value *= s_inv[local];  // exact: a power of two
        if (row < m && col < n) store_out<XT>(out, (size_t)row * n + col, value + b);
      }
    };

    if (s0 == 0 && s1 == spt) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < WN; ++nt) store_block(mt, nt, total[mt][nt]);
    } else {
      const uint32_t tile_begin = tile * spt;
      auto slot_of = [&](uint32_t u) {
        return 2u * u + (deal_begin(deal, u) <= tile_begin ? 1u : 0u);
      };
      uint32_t* ticket = deal.tickets + (size_t)tile * kTicketStride;
      const uint32_t first = deal_owner(deal, tile_begin), last = deal_owner(deal, tile_begin + spt - 1u);
      if (tid == 0)
        s_ticket = __hip_atomic_load(ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      bool merge = s_ticket == last - first;
      __syncthreads();
      if (!merge) {
        float4_t* mine =
            reinterpret_cast<float4_t*>(deal.partials + (size_t)slot_of(v) * kPartialFloats);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int nt = 0; nt < WN; ++nt)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float4_t piece = {total[mt][nt][4 * q], total[mt][nt][4 * q + 1],
                                      total[mt][nt][4 * q + 2], total[mt][nt][4 * q + 3]};
              publish4(mine + (size_t)(((mt * WN + nt) * 4 + q) * T + tid), piece);
            }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0)
          s_ticket = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        merge = s_ticket == last - first;
      }
      if (merge) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          float16_t sum[WN];
          for (uint32_t u = first; u <= last; ++u) {
            float16_t part[WN];
#pragma unroll
            for (int nt = 0; nt < WN; ++nt) part[nt] = total[mt][nt];
            if (u != v) {
              const float4_t* src =
                  reinterpret_cast<const float4_t*>(deal.partials + (size_t)slot_of(u) * kPartialFloats) +
                  (size_t)(mt * WN * 4 * T + tid);
              float4_t p[8];
#pragma unroll
              for (int i = 0; i < 8; ++i) p[i] = observe4(src + (size_t)i * T);
              landed(p);
#pragma unroll
              for (int nt = 0; nt < WN; ++nt)
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                  for (int i = 0; i < 4; ++i) part[nt][4 * q + i] = p[nt * 4 + q][i];
            }
#pragma unroll
            for (int nt = 0; nt < WN; ++nt) {
              if (u == first) {
                sum[nt] = part[nt];
              } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) sum[nt][r] += part[nt][r];
              }
            }
          }
#pragma unroll
          for (int nt = 0; nt < WN; ++nt) store_block(mt, nt, sum[nt]);
        }
        if (tid == 0)
          __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    __syncthreads();  // s_inv and the LDS tiles are rewritten by the next tile of the range
    left -= s1 - s0;
  }
}

// The deal of the 64 x 512 tiles: one workgroup per CU, every workgroup at least two stages.
bool plan_exact_deal(krm_ctx* ctx, uint32_t m, uint32_t n, uint32_t k, uint32_t& grid,
                     UnitDeal& deal) {
  const uint64_t cus = (uint64_t)ctx->num_cus;
  const uint64_t tiles = (uint64_t)((m + 63) / 64) * ((n + 511) / 512);
  const uint32_t spt = (k + 127) / 128;
  const uint64_t units = tiles * spt;
  if (tiles > kTicketSlots || units > 0x7fffffffull || units < 2 * cus) return false;
  if (tiles * 8 < cus) return false;  // a tile shared by more than eight workgroups
  if (!ctx->gemm_partials) return false;
  grid = (uint32_t)cus;
  deal.stages_per_tile = spt;
  deal.units_lo = (uint32_t)(units / cus);
  deal.extra = (uint32_t)(units % cus);
  deal.partials = ctx->gemm_partials;
  deal.tickets = ctx->tickets;
  return true;
}

// Workgroups, units and scratch of a dealt launch; false when the shape is not worth it.
bool plan_deal(krm_ctx* ctx, uint32_t m, uint32_t n, uint32_t k, uint32_t& grid, UnitDeal& deal) {
  const uint64_t cus = (uint64_t)ctx->num_cus;
  const uint64_t tiles = (uint64_t)((m + 127) / 128) * ((n + 255) / 256);
  const uint32_t spt = (k + 127) / 128;
  const uint64_t units = tiles * spt;
  // at least four stages to a workgroup: with less, a tile is the sum of so many short slices
  // that writing and merging the partials costs more than the idle CUs did (128 x 11264 x 2048:
  // 2.75 stages each, 36.8 us against 30.9 us for one workgroup per 128 x 64 tile)
  if (tiles > kTicketSlots || units > 0x7fffffffull || units < 4 * cus) return false;
  // whole rounds of tiles already use the chip well
  const uint64_t rounds = (tiles + cus - 1) / cus;
  if (tiles * 10 >= rounds * cus * 9) return false;
  // a tile shared by many workgroups costs more in partials than the idle CUs did
  if (tiles * 6 < cus) return false;
  if (!ctx->gemm_partials) return false;
  grid = (uint32_t)cus;
  deal.stages_per_tile = spt;
  deal.units_lo = (uint32_t)(units / cus);
  deal.extra = (uint32_t)(units % cus);
  deal.partials = ctx->gemm_partials;
  deal.tickets = ctx->tickets;
  return true;
}

template <typename XT, typename ST, int WM>
int32_t launch_dealt(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                     uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift, uint32_t grid,
                     const UnitDeal& deal) {
  KRM_TRY(needs_serial_scratch(ctx, "the unit-dealt GEMM"));
  gemm_i4_f16_dealt_kernel<XT, ST, WM><<<dim3(grid), dim3(WM * 256), 0, ctx->stream>>>(
      ptr<const XT>(x), ptr<const uint8_t>(w), ptr<const ST>(scales), ptr<const XT>(bias),
      ptr<XT>(out), m, n, k, group_shift, (m + 127) / 128, deal);
  return launched(ctx, "gemm_i4_f16_dealt_kernel");
}

template <typename XT, typename ST, int MT>
int32_t launch_packed(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                      krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift) {
  const uint32_t m_blocks = (m + 64 * MT - 1) / (64 * MT), n_blocks = (n + 255) / 256;
  const uint64_t total = (uint64_t)((n_blocks + 7) / 8) * 8 * m_blocks;
  if (total > 0x7fffffffull) return fail(ctx, KRM_ERR_VALIDATION, "linear: grid too large");
  gemm_i4_f16_packed_kernel<XT, ST, MT><<<dim3((unsigned)total), dim3(512), 0, ctx->stream>>>(
      ptr<const XT>(x), ptr<const uint8_t>(w), ptr<const ST>(scales), ptr<const XT>(bias),
      ptr<XT>(out), m, n, k, group_shift, m_blocks, n_blocks);
  return launched(ctx, "gemm_i4_f16_packed_kernel");
}

template <typename XT, typename ST, int WM, int WN, int KC, int KS, int DEPTH, bool PIPE = false>
int32_t launch(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
               uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift) {
  constexpr int BM = WM * 64, BN = WN * 64;
  const uint32_t m_blocks = (m + BM - 1) / BM, n_blocks = (n + BN - 1) / BN;
  uint64_t total;
  if (8 % m_blocks == 0) {
    total = (uint64_t)((n_blocks + 7) / 8) * 8 * m_blocks;
  } else {
    total = (uint64_t)m_blocks * n_blocks;
  }
  if (total > 0x7fffffffull) return fail(ctx, KRM_ERR_VALIDATION, "linear: grid too large");
  constexpr int kWordsPerThread = BN * (KC / 8) / (WM * WN * KS * 64);
  const uint32_t wide = (k % 32 == 0 && aligned(w, 16)) ? 1u : 0u;
  const bool fast = wide && kWordsPerThread >= 4 && k % KC == 0 &&
                    (((uint32_t)(kWordsPerThread * 8 - 1) >> group_shift) == 0);
  if (fast)
    gemm_i4_f16_kernel<XT, ST, WM, WN, KC, KS, DEPTH, PIPE, true>
        <<<dim3((unsigned)total), dim3(WM * WN * KS * 64), 0, ctx->stream>>>(
            ptr<const XT>(x), ptr<const uint32_t>(w), ptr<const ST>(scales), ptr<const XT>(bias),
            ptr<XT>(out), m, n, k, group_shift, m_blocks, n_blocks, wide);
  else
    gemm_i4_f16_kernel<XT, ST, WM, WN, KC, KS, DEPTH, PIPE, false>
        <<<dim3((unsigned)total), dim3(WM * WN * KS * 64), 0, ctx->stream>>>(
            ptr<const XT>(x), ptr<const uint32_t>(w), ptr<const ST>(scales), ptr<const XT>(bias),
            ptr<XT>(out), m, n, k, group_shift, m_blocks, n_blocks, wide);
  return launched(ctx, "gemm_i4_f16_kernel");
}

template <typename XT, typename ST>
int32_t pick_tile(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                  uint32_t m, uint32_t n, uint32_t k, uint32_t group) {
  uint32_t group_shift = 0;
  while ((1u << group_shift) < group) ++group_shift;
  // 128 x 64 tiles (two waves, chunks of 64 codes, two chunks in flight) when they fill the
  // chip at least twice over.  Otherwise four wave groups split every 128-code chunk of K
  // between them on a 64 x 64 tile: four times the waves for the same outputs.
  // Enough 128 x 128 tiles for every CU: four waves a tile, chunks of 64 codes, pipelined with
  // four chunks in flight.  Fewer (a narrow output with a long K, or few rows): 128 x 64 tiles
  // whose two wave groups split every 128-code chunk of K, or 64 x 64 tiles with four groups.
  const uint64_t cus = (uint64_t)ctx->num_cus;
  // 128 x 256 tiles with the packed weights in LDS.  Dealt by (tile, stage) units over all CUs
  // when whole rounds of tiles would leave part of the chip idle (512 x 11008 x 4096: 69 us
  // against 77 us for one workgroup per tile; 512 x 4096 x 11008: 75 us against 93 us for the
  // K-splitting form below); one workgroup per tile when the tiles cover most of the chip; with
  // fewer tiles the forms below, which split K inside a workgroup.
  const uint64_t packed_tiles = (uint64_t)((m + 127) / 128) * ((n + 255) / 256);
  const bool packed_ok = m > 64 && group >= 64 && k % 8 == 0 && aligned(w, 16) && aligned(x, 16);
  if (packed_ok) {
    uint32_t grid = 0;
    UnitDeal deal{};
    if (plan_deal(ctx, m, n, k, grid, deal))
      return launch_dealt<XT, ST, 2>(ctx, x, w, scales, bias, out, m, n, k, group_shift, grid, deal);
  }
  if (packed_ok && packed_tiles * 5 >= cus * 3)
    return launch_packed<XT, ST, 2>(ctx, x, w, scales, bias, out, m, n, k, group_shift);
  const uint64_t tiles = (uint64_t)((m + 127) / 128) * ((n + 127) / 128);
  if (m > 64 && tiles >= cus)
    return launch<XT, ST, 2, 2, 64, 1, 4, true>(ctx, x, w, scales, bias, out, m, n, k, group_shift);
  // Few tiles and a K of several chunks: 64 x 64 tiles whose four wave groups split every
  // 128-code chunk, two LDS copies and two chunks in flight (measured on 128-row products:
  // N = 2048, K = 2048 21.5 us against 28.3 us for the 128 x 64 form below and 25.7 us for the
  // same tiles with one copy; N = 2048, K = 5632 37 us against 58 us).
  const uint64_t tiles_128x64 = (uint64_t)((m + 127) / 128) * ((n + 63) / 64);
  if (k >= 512 && (m <= 64 || tiles_128x64 * 2 < cus))
    return launch<XT, ST, 1, 1, 128, 4, 2, true>(ctx, x, w, scales, bias, out, m, n, k, group_shift);
  if (m > 64 && k >= 256)
    return launch<XT, ST, 2, 1, 128, 2, 2, true>(ctx, x, w, scales, bias, out, m, n, k, group_shift);
  return launch<XT, ST, 1, 1, 64, 1, 1>(ctx, x, w, scales, bias, out, m, n, k, group_shift);
}

// ------------------------------------------------ exact integer operands, few rows
//
// The same arithmetic for products too small for the 64 x 512 deal (a prefill chunk of a few
// hundred rows): tile 32 x 32 (or 32 x 64) per workgroup, and the eight waves of a workgroup
// split K between them instead of the columns, so (M / 32) (N / 32) workgroups each walk K / 8
// per wave.  Such a product is bound by what a CU's vector memory path takes per workgroup,
// which counts cache lines per load: every load here covers whole rows, 16 bytes a lane.
// A wave's slice is walked 128 codes at a time:
//   x     32 rows x 128 codes, turned into fp16 (or hi + lo) and parked in the wave's own LDS
//         area in natural order; no other wave reads it, so the K loop has no barrier;
//   w     32 (64) rows x 64 bytes, parked as they are; a lane reads the word of its column and
//         MFMA step back, turns it into integers and puts them in natural order (four byte
//         permutes a word);
//   two chunks are in flight: a K of 2048 is requested whole before anything is used.
// At the end the eight waves' sums meet in LDS and are added in wave order; the epilogue (bias,
// residual, gate/up pairs, RoPE of a fused [q; k; v] projection) works on column pairs there.
template <typename XT>
__device__ inline float round_io(float v);
template <>
__device__ inline float round_io<float>(float v) { return v; }
template <>
__device__ inline float round_io<__half>(float v) { return __half2float(__float2half_rn(v)); }

// Columns (col, col + 1) of output row `row`, summed: bias, then what the call asked for.
template <typename XT>
__device__ inline void finish_pair(float v0, float v1, uint32_t row, uint32_t col, uint32_t m,
                                   uint32_t n, const XT* __restrict__ bias, XT* __restrict__ out,
                                   const RowsFusion& fuse) {
  const XT* residual = static_cast<const XT*>(fuse.residual);
  const bool two = col + 1 < n;
  if (bias) {
    v0 += bias_f32<XT>(bias, col);
    if (two) v1 += bias_f32<XT>(bias, col + 1);
  }
  if (fuse.mode == 1) {
    // (gate, up) -> silu(gate) * up, the roundings of the decode row's epilogue
    const float t = __builtin_amdgcn_exp2f(-fabsf(v0) * 1.4426950408889634f);
    const float r = __builtin_amdgcn_rcpf(1.0f + t);
    const float sig = v0 < 0.f ? t * r : r;
    float value = __fmul_rn(__fmul_rn(v0, sig), v1);
    const size_t at = (size_t)row * (n >> 1) + (col >> 1);
    if (residual) value += bias_f32<XT>(residual, at);
    store_out<XT>(out, at, value);
  } else if (fuse.mode == 2) {
    // what a separate linear would have stored, then the rotation of krm_rope_half
    const float x0 = round_io<XT>(v0), x1 = round_io<XT>(v1);
    const uint32_t half = fuse.depth >> 1, pair = col >> 1;
    const uint32_t rope_pairs = (fuse.heads + fuse.kv_heads) * half;
    if (pair < rope_pairs) {
      const uint32_t head = pair / half, j = pair - head * half;
      const int32_t pos = fuse.positions[row];
      float o0 = NAN, o1 = NAN;  // a position outside the table is never a valid rotation
      if (pos >= 0 && (uint32_t)pos < fuse.table_rows) {
        const size_t t = (size_t)pos * fuse.depth + j;
        o0 = __fadd_rn(__fmul_rn(x0, fuse.cos_table[t]), __fmul_rn(-x1, fuse.sin_table[t]));
        o1 = __fadd_rn(__fmul_rn(x1, fuse.cos_table[t + half]),
                       __fmul_rn(x0, fuse.sin_table[t + half]));
      }
      XT* dst = head < fuse.heads
                    ? static_cast<XT*>(fuse.q_out) + ((size_t)head * m + row) * fuse.depth
                    : static_cast<XT*>(fuse.k_out) +
                          ((size_t)(head - fuse.heads) * m + row) * fuse.depth;
      store_out<XT>(dst, j, o0);
      store_out<XT>(dst, j + half, o1);
    } else {
      const uint32_t e = (pair - rope_pairs) * 2u;  // the v section keeps its natural order
      const uint32_t plane = e / fuse.depth, d = e - plane * fuse.depth;
      XT* dst = static_cast<XT*>(fuse.v_out) + ((size_t)plane * m + row) * fuse.depth;
      store_out<XT>(dst, d, x0);
      store_out<XT>(dst, d + 1, x1);
    }
  } else {
    const size_t at = (size_t)row * n + col;
    if (residual) {
      v0 += bias_f32<XT>(residual, at);
      if (two) v1 += bias_f32<XT>(residual, at + 1);
    }
    store_out<XT>(out, at, v0);
    if (two) store_out<XT>(out, at + 1, v1);
  }
}

// 8 codes of a word -> 8 fp16 integers (u - 8) in their natural order c0..c7.
__device__ inline uint4 ints_word_natural(uint32_t word) {
  const uint4 q = ints_word(word);  // (c0,c4), (c1,c5), (c2,c6), (c3,c7)
  return make_uint4(__builtin_amdgcn_perm(q.y, q.x, 0x05040100u),   // (c0, c1)
                    __builtin_amdgcn_perm(q.w, q.z, 0x05040100u),   // (c2, c3)
                    __builtin_amdgcn_perm(q.y, q.x, 0x07060302u),   // (c4, c5)
                    __builtin_amdgcn_perm(q.w, q.z, 0x07060302u));  // (c6, c7)
}

// One row piece of x as it arrives (16 bytes: 4 f32 or 8 fp16) and as it is parked (fp16, natural
// order; the split form parks hi and lo).
template <typename XT, int OPERAND>
struct RowPiece;
template <int OPERAND>
struct RowPiece<float, OPERAND> {
  static constexpr int kCodes = 4;
  uint4 raw;
  __device__ inline void park(uint8_t* hi_at, uint8_t* lo_at, float scale, uint32_t keep) const {
    const float v[4] = {__uint_as_float(raw.x), __uint_as_float(raw.y), __uint_as_float(raw.z),
                        __uint_as_float(raw.w)};
    _Float16 h[4], l[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (OPERAND == kOperandSplit) {
        const float xs = v[i] * scale;        // exact: a power of two
        h[i] = (_Float16)xs;                  // round to nearest even
        l[i] = (_Float16)(xs - (float)h[i]);  // the difference is exact in f32
      } else {
        h[i] = (_Float16)v[i];
      }
    }
    auto pack = [](_Float16 p, _Float16 q) {
      const half2_t t = {p, q};
      return __builtin_bit_cast(uint32_t, t);
    };
    *reinterpret_cast<uint2*>(hi_at) = make_uint2(pack(h[0], h[1]) & keep, pack(h[2], h[3]) & keep);
    if constexpr (OPERAND == kOperandSplit)
      *reinterpret_cast<uint2*>(lo_at) =
          make_uint2(pack(l[0], l[1]) & keep, pack(l[2], l[3]) & keep);
  }
};
template <int OPERAND>
struct RowPiece<__half, OPERAND> {
  static constexpr int kCodes = 8;
  uint4 raw;
  __device__ inline void park(uint8_t* hi_at, uint8_t*, float, uint32_t keep) const {
    *reinterpret_cast<uint4*>(hi_at) =
        make_uint4(raw.x & keep, raw.y & keep, raw.z & keep, raw.w & keep);
  }
};

// XT: element type of x; OT: element type of bias, residual and out (the call's io type).  They
// differ only for fp16 x with f32 io: an fp16 copy of the activations written by the producing
// kernel, the same values the f32 activations are rounded to under KRM_COMPUTE_F16.
template <typename XT, typename OT, typename ST, int OPERAND, int WN>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_i4_rows_kernel(const XT* __restrict__ x, const uint8_t* __restrict__ w,
                         const ST* __restrict__ scales, const OT* __restrict__ bias,
                         OT* __restrict__ out, uint32_t m, uint32_t n, uint32_t k,
                         uint32_t group_shift, uint32_t m_blocks, uint32_t tiles,
                         const float* __restrict__ row_scale, RowsFusion fuse) {
  constexpr int BM = 32, BN = 32 * WN, kWaves = 8;
  constexpr int NA = OPERAND == kOperandSplit ? 2 : 1;
  constexpr int kChunk = 128;
  // The split form with 64-column tiles parks the x rows of a chunk in two parts of 64 codes
  // (hi and lo planes of 128 codes for eight waves would not fit the LDS next to 64 weight
  // rows); every other form parks the chunk at once.
  constexpr int kParts = (OPERAND == kOperandSplit && WN == 2) ? 2 : 1;
  constexpr int kPartCodes = kChunk / kParts;
  constexpr int kRowA = kPartCodes * 2 + 16;      // bytes of a parked x row
  constexpr int kPlane = BM * kRowA;
  constexpr int kRowB = kChunk / 2 + 16;          // bytes of a parked weight row
  constexpr int kWords = BN * kRowB;
  constexpr int kSumBytes = BM * BN * 4;
  constexpr int kStageBytes = NA * kPlane + kWords;
  constexpr int kWaveBytes = kStageBytes > kSumBytes ? kStageBytes : kSumBytes;
  constexpr int kPieceCodes = RowPiece<XT, OPERAND>::kCodes;
  constexpr int kLanesPerRow = kPartCodes / kPieceCodes;      // 32 (f32), 16 (fp16, f32 in parts)
  constexpr int kRowsPerLoad = 64 / kLanesPerRow;             // 2 or 4
  constexpr int kPartLoads = BM / kRowsPerLoad;               // loads of one part: 16 or 8
  constexpr int kActLoads = kPartLoads * kParts;
  static_assert(kWaves * kWaveBytes + 1024 <= 160 * 1024, "the waves' areas fit the LDS");
  constexpr int kWordLoads = BN / 16;                         // 16 rows x 4 pieces a load
  static_assert(OPERAND == kOperandF16 || sizeof(XT) == 4, "only f32 activations are split");
  __shared__ __align__(16) uint8_t s_wave[kWaves][kWaveBytes];
  __shared__ float s_inv[BM], s_up[BM];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frag_row = lane & 31, frag_h = lane >> 5;
  const uint32_t groups = k >> group_shift;
  const bool half_groups = group_shift == 6;  // 64 codes a group: two groups a chunk
  // blockIdx & 7 is the XCD: each XCD takes a contiguous range of tiles, the row tiles of a
  // column tile next to each other, so the weights of a column tile come from memory once
  const uint32_t per_xcd = (tiles + 7u) >> 3;
  const uint32_t tile = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
  if (tile >= tiles) return;
  const uint32_t nb = tile / m_blocks, mb = tile - nb * m_blocks;
  const uint32_t m0 = mb * BM, n0 = nb * BN;
  const uint32_t chunks = (k + kChunk - 1) / kChunk;
  const uint32_t c_begin = (uint32_t)wave * chunks / kWaves;
  const uint32_t c_end = ((uint32_t)wave + 1u) * chunks / kWaves;
  uint8_t* mine = s_wave[wave];
  uint8_t* my_words = mine + NA * kPlane;

  // staging: whole rows, 16 bytes a lane (coalesced), kRowsPerLoad rows a load
  const uint32_t a_piece = lane % kLanesPerRow, a_row = lane / kLanesPerRow;
  const uint32_t b_piece = lane & 3u, b_row = lane >> 2;
  // (element offsets in 32 bits — the launcher checks that x and w are that small — and the
  // row scales in LDS: the registers are wanted for two chunks in flight)
  const uint32_t x_row0 = m0 + a_row;
  if constexpr (OPERAND == kOperandSplit) {
    if (tid < BM) {
      const size_t row = min(m0 + (uint32_t)tid, m - 1);
      s_up[tid] = row_scale[2 * row];
      s_inv[tid] = row_scale[2 * row + 1];
    }
    __syncthreads();
  }
  uint32_t wrow[kWordLoads];
#pragma unroll
  for (int i = 0; i < kWordLoads; ++i) wrow[i] = min(n0 + 16u * i + b_row, n - 1) * (k >> 1);
  const ST* srow[WN];
#pragma unroll
  for (int nt = 0; nt < WN; ++nt)
    srow[nt] = scales + (size_t)min(n0 + 32u * nt + (uint32_t)frag_row, n - 1) * groups;

  struct Staged {
    RowPiece<XT, OPERAND> a[kActLoads];
    uint4 b[kWordLoads];
    float ws[WN][2];  // the scales of the chunk's first and second 64 codes
  };
  auto load_chunk = [&](uint32_t c, Staged& d) {
#pragma unroll
    for (int part = 0; part < kParts; ++part) {
      const uint32_t at = c * kChunk + part * kPartCodes + a_piece * kPieceCodes;
      const uint32_t off = at < k ? at : 0u;
#pragma unroll
      for (int i = 0; i < kPartLoads; ++i)
        d.a[part * kPartLoads + i].raw = *reinterpret_cast<const uint4*>(
            x + ((size_t)(min(x_row0 + (uint32_t)(kRowsPerLoad * i), m - 1) * k) + off));
    }
    const uint32_t bat = c * (kChunk / 2) + b_piece * 16u;
    const uint32_t boff = bat < (k >> 1) ? bat : 0u;
#pragma unroll
    for (int i = 0; i < kWordLoads; ++i)
      d.b[i] = *reinterpret_cast<const uint4*>(w + ((size_t)wrow[i] + boff));
    const uint32_t c0 = c * kChunk < k ? c * kChunk : 0u;
    const uint32_t c1 = c * kChunk + 64u < k ? c * kChunk + 64u : c0;
#pragma unroll
    for (int nt = 0; nt < WN; ++nt) {
      d.ws[nt][0] = load_scale_f32<ST>(srow[nt], c0 >> group_shift);
      d.ws[nt][1] = load_scale_f32<ST>(srow[nt], c1 >> group_shift);
    }
  };
  auto park_rows = [&](uint32_t c, const Staged& d, int part) {
    const uint32_t keep =  // past K: zeros
        c * kChunk + part * kPartCodes + a_piece * kPieceCodes < k ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int i = 0; i < kPartLoads; ++i) {
      const uint32_t at = (kRowsPerLoad * i + a_row) * kRowA + a_piece * (kPieceCodes * 2);
      float up = 1.0f;
      if constexpr (OPERAND == kOperandSplit) up = s_up[kRowsPerLoad * i + a_row];
      d.a[part * kPartLoads + i].park(mine + at, mine + kPlane + at, up, keep);
    }
  };
  auto park_chunk = [&](uint32_t c, const Staged& d) {
    park_rows(c, d, 0);
#pragma unroll
    for (int i = 0; i < kWordLoads; ++i)
      *reinterpret_cast<uint4*>(my_words + (16 * i + b_row) * kRowB + b_piece * 16u) = d.b[i];
  };
  // The parked rows are written and read by the same wave only: what orders them is the LDS
  // queue of the wave, and the compiler is told not to move accesses across this point.
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  float16_t total[WN], acc[WN];
#pragma unroll
  for (int nt = 0; nt < WN; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) total[nt][r] = acc[nt][r] = 0.f;
  auto flush = [&](const float (&ws)[WN][2], int which) {
#pragma unroll
    for (int nt = 0; nt < WN; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        total[nt][r] = fmaf(acc[nt][r], ws[nt][which], total[nt][r]);
        acc[nt][r] = 0.f;
      }
  };

  // kDepth chunks in flight (two where the registers allow: a K of 2048 is then requested whole
  // before anything is used)
  constexpr int kDepth = (sizeof(XT) == 2 || (WN == 1 && OPERAND == kOperandF16)) ? 2 : 1;
  Staged staged[kDepth];
#pragma unroll
  for (int d = 0; d < kDepth; ++d)
    if (c_begin + d < c_end) load_chunk(c_begin + d, staged[d]);
  auto run_chunk = [&](uint32_t c, int cur) {
    park_chunk(c, staged[cur]);
    float ws[WN][2];
#pragma unroll
    for (int nt = 0; nt < WN; ++nt) {
      ws[nt][0] = staged[cur].ws[nt][0];
      ws[nt][1] = staged[cur].ws[nt][1];
    }
    if constexpr (kParts == 1) {
      if (c + kDepth < c_end) load_chunk(c + kDepth, staged[cur]);
    }
    wave_sync();
#pragma unroll
    for (int j = 0; j < 8; ++j) {  // step j: codes 16 j + 8 h .. + 7 of the chunk
      if constexpr (kParts == 2) {
        if (j == 4) {  // the second 64 codes of the x rows take the first ones' place
          wave_sync();
          park_rows(c, staged[cur], 1);
          if (c + kDepth < c_end) load_chunk(c + kDepth, staged[cur]);
          wave_sync();
        }
      }
      half8_t a[NA];
#pragma unroll
      for (int copy = 0; copy < NA; ++copy)
        a[copy] = *reinterpret_cast<const half8_t*>(mine + copy * kPlane + frag_row * kRowA +
                                                    32 * (j % (8 / kParts)) + 16 * frag_h);
#pragma unroll
      for (int nt = 0; nt < WN; ++nt) {
        const uint32_t word = *reinterpret_cast<const uint32_t*>(
            my_words + (32 * nt + frag_row) * kRowB + 8 * j + 4 * frag_h);
        const half8_t b = __builtin_bit_cast(half8_t, ints_word_natural(word));
#pragma unroll
        for (int copy = 0; copy < NA; ++copy)
          acc[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[copy], b, acc[nt], 0, 0, 0);
      }
      if (j == 3 && half_groups) flush(ws, 0);
    }
    wave_sync();
    // the scale group ends with this chunk, or the wave's slice does
    if (half_groups || (((c + 1) * kChunk) & ((1u << group_shift) - 1u)) == 0u || c + 1 == c_end)
      flush(ws, 1);
  };
  for (uint32_t c = c_begin; c < c_end; c += kDepth) {
    run_chunk(c, 0);
    if constexpr (kDepth == 2) {
      if (c + 1 < c_end) run_chunk(c + 1, 1);
    }
  }

  // the wave's sums, [row][column] in its own area
  float* sums = reinterpret_cast<float*>(mine);
#pragma unroll
  for (int nt = 0; nt < WN; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int local = 8 * (r / 4) + 4 * frag_h + (r % 4);
      sums[local * BN + nt * 32 + frag_row] = total[nt][r];
    }
  __syncthreads();

  constexpr int kPairs = BM * BN / 2;
#pragma unroll
  for (int i = 0; i < kPairs / 512; ++i) {
    const int p = tid + 512 * i;
    const int local = p / (BN / 2), cp = p - local * (BN / 2);
    const uint32_t row = m0 + local, col = n0 + 2u * cp;
    float v0 = 0.f, v1 = 0.f;
#pragma unroll
    for (int wv = 0; wv < kWaves; ++wv) {  // wave order: a fixed sum
      const float2 part =
          *reinterpret_cast<const float2*>(s_wave[wv] + (size_t)(local * BN + 2 * cp) * 4);
      v0 += part.x;
      v1 += part.y;
    }
    if (row >= m || col >= n) continue;
    if constexpr (OPERAND == kOperandSplit) {  // exact: a power of two
      v0 *= s_inv[local];
      v1 *= s_inv[local];
    }
    finish_pair<OT>(v0, v1, row, col, m, n, bias, out, fuse);
  }
}

template <typename XT, typename OT, typename ST, int OPERAND, int WN>
int32_t launch_rows(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                    uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift,
                    const RowsFusion& fuse) {
  if constexpr (OPERAND == kOperandSplit) {
    KRM_TRY(needs_serial_scratch(ctx, "the f32-class few-row GEMM"));
    row_scale_kernel<<<dim3(m), dim3(256), 0, ctx->stream>>>(ptr<const float>(x), ctx->row_scales, k);
    KRM_TRY(launched(ctx, "row_scale_kernel"));
  }
  const uint32_t m_blocks = (m + 31) / 32, n_blocks = (n + 32 * WN - 1) / (32 * WN);
  const uint32_t tiles = m_blocks * n_blocks;
  gemm_i4_rows_kernel<XT, OT, ST, OPERAND, WN>
      <<<dim3(((tiles + 7) / 8) * 8), dim3(512), 0, ctx->stream>>>(
          ptr<const XT>(x), ptr<const uint8_t>(w), ptr<const ST>(scales), ptr<const OT>(bias),
          ptr<OT>(out), m, n, k, group_shift, m_blocks, tiles, ctx->row_scales, fuse);
  return launched(ctx, "gemm_i4_rows_kernel");
}

template <typename XT, typename ST, int OPERAND>
int32_t launch_exact(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias, krm_buf out,
                     uint32_t m, uint32_t n, uint32_t k, uint32_t group_shift, uint32_t grid,
                     const UnitDeal& deal) {
  KRM_TRY(needs_serial_scratch(ctx, "the unit-dealt GEMM"));
  if constexpr (OPERAND == kOperandSplit) {
    row_scale_kernel<<<dim3(m), dim3(256), 0, ctx->stream>>>(ptr<const float>(x), ctx->row_scales, k);
    KRM_TRY(launched(ctx, "row_scale_kernel"));
  }
  gemm_i4_exact_kernel<XT, ST, OPERAND><<<dim3(grid), dim3(512), 0, ctx->stream>>>(
      ptr<const XT>(x), ptr<const uint8_t>(w), ptr<const ST>(scales), ptr<const XT>(bias),
      ptr<XT>(out), m, n, k, group_shift, (m + 63) / 64, deal, ctx->row_scales);
  return launched(ctx, "gemm_i4_exact_kernel");
}

}  // namespace

namespace krm {

// The exact-integer-operand GEMM for shapes whose (tile, stage) units cover the chip; sets
// *handled = false (and launches nothing) for every other shape.
int32_t linear_i4_gemm_exact(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                             krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                             int32_t io_dtype, int32_t scale_dtype, int32_t compute,
                             bool* handled) {
  *handled = false;
  const bool split = compute == KRM_COMPUTE_F32 && io_dtype == KRM_F32;
  if (group < 64 || k % 32 != 0 || !aligned(w, 16) || !aligned(x, 16)) return KRM_OK;
  if (split && (m > kMaxSplitRows || !ctx->row_scales)) return KRM_OK;
  uint32_t grid = 0;
  UnitDeal deal{};
  if (!plan_exact_deal(ctx, m, n, k, grid, deal)) return KRM_OK;
  uint32_t group_shift = 0;
  while ((1u << group_shift) < group) ++group_shift;
  *handled = true;
#define KRM_EXACT(XT, ST, OP) \
  return launch_exact<XT, ST, OP>(ctx, x, w, scales, bias, out, m, n, k, group_shift, grid, deal)
  if (io_dtype == KRM_F16) {
    if (scale_dtype == KRM_F16) KRM_EXACT(__half, __half, kOperandF16);
    KRM_EXACT(__half, float, kOperandF16);
  }
  if (split) {
    if (scale_dtype == KRM_F16) KRM_EXACT(float, __half, kOperandSplit);
    KRM_EXACT(float, float, kOperandSplit);
  }
  if (scale_dtype == KRM_F16) KRM_EXACT(float, __half, kOperandF16);
  KRM_EXACT(float, float, kOperandF16);
#undef KRM_EXACT
}

// The few-row form of the same arithmetic, with its epilogues; any shape with a group of at
// least 64 codes, K a multiple of 32 and 16-byte aligned rows.  *handled = false (nothing
// launched) otherwise.
int32_t linear_i4_gemm_rows(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                            krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                            int32_t io_dtype, int32_t scale_dtype, int32_t compute,
                            const RowsFusion& fuse, bool* handled, int32_t x_dtype) {
  *handled = false;
  const bool half_x = x_dtype == KRM_F16 && io_dtype == KRM_F32;  // fp16 x, f32 bias / out
  if (x_dtype != io_dtype && !(half_x && compute == KRM_COMPUTE_F16)) return KRM_OK;
  const bool split = compute == KRM_COMPUTE_F32 && io_dtype == KRM_F32;
  if (group < 64 || k % 32 != 0 || !aligned(w, 16) || !aligned(x, 16)) return KRM_OK;
  if (split && (m > kMaxSplitRows || !ctx->row_scales)) return KRM_OK;
  const uint64_t m_blocks = (m + 31) / 32;
  if (m_blocks * ((n + 31) / 32) > 0x7fffffffull) return KRM_OK;
  if ((uint64_t)m * k > 0xffffffffull || (uint64_t)n * (k >> 1) > 0xffffffffull) return KRM_OK;
  uint32_t group_shift = 0;
  while ((1u << group_shift) < group) ++group_shift;
  *handled = true;
  // 64 columns a workgroup once 32 would need more than one round of workgroups: fewer reads of
  // x for the same weights
  const bool wide = m_blocks * ((n + 31) / 32) > (uint64_t)ctx->num_cus;
#define KRM_ROWS(XT, OT, ST, OP)                                                                  \
  return wide ? launch_rows<XT, OT, ST, OP, 2>(ctx, x, w, scales, bias, out, m, n, k, group_shift, \
                                               fuse)                                              \
              : launch_rows<XT, OT, ST, OP, 1>(ctx, x, w, scales, bias, out, m, n, k, group_shift, \
                                               fuse)
  if (io_dtype == KRM_F16) {
    if (scale_dtype == KRM_F16) KRM_ROWS(__half, __half, __half, kOperandF16);
    KRM_ROWS(__half, __half, float, kOperandF16);
  }
  if (half_x) {
    if (scale_dtype == KRM_F16) KRM_ROWS(__half, float, __half, kOperandF16);
    KRM_ROWS(__half, float, float, kOperandF16);
  }
  if (split) {
    if (scale_dtype == KRM_F16) KRM_ROWS(float, float, __half, kOperandSplit);
    KRM_ROWS(float, float, float, kOperandSplit);
  }
  if (scale_dtype == KRM_F16) KRM_ROWS(float, float, __half, kOperandF16);
  KRM_ROWS(float, float, float, kOperandF16);
#undef KRM_ROWS
}

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
