// states-form attention over the KV state slots for gfx950.
//
// Contract (packages/runtime/src/kernels/state-attention.ts:1-113, docs/ir-v1.md:296-351):
// logical columns [0, P+Q); column c < P is read from the slot at physical row c (or c % W for
// a sliding window), column c >= P from this step's ins row c - P; output row r attends to
// c <= P + r and, with a window, P + r - c < W; kv plane = floor((b*H + h) / r); rows >= Q
// are written as exact 0; the half-scale multiplies q and k.
//
// The reference materialises S, reduces row statistics and multiplies by V in three
// dispatches.  Here one launch streams K and V once with an online softmax:
//  * decode (Q = 1, M = 1): split-K.  A workgroup owns one KV head and one range of past
//    columns, loads that range's K and V with 16-byte coalesced loads, scores all r query
//    heads of the KV head against it (the KV bytes are read once, not r times), and writes
//    (max, sum, weighted V) partials that a second small kernel merges in split order.
//    The column partition depends only on the number of past columns, the head dim and the
//    slot dtype, so a sequence gives the same bits alone or inside a ragged batch.
//  * everything else (prefill chunks, pad rows, head dims the fast path does not cover):
//    a generic kernel, one workgroup per (plane, row).
#include "krm_internal.h"

#include <cmath>

using namespace krm;

namespace {

constexpr int kThreads = 256;
constexpr int kDecodeIter = 8;  // K/V rows each lane group walks per split

template <typename T>
__device__ inline float ld_f32(const T* p, size_t i);
template <>
__device__ inline float ld_f32<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ inline float ld_f32<__half>(const __half* p, size_t i) { return __half2float(p[i]); }
template <typename T>
__device__ inline void st_f32(T* p, size_t i, float v);
template <>
__device__ inline void st_f32<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ inline void st_f32<__half>(__half* p, size_t i, float v) { p[i] = __float2half_rn(v); }

// first logical column a row with causal limit `limit` may see (0 for a full context)
__host__ __device__ inline uint64_t window_low(uint32_t window, uint64_t limit) {
  return (window && limit + 1 > window) ? limit + 1 - window : 0;
}

// ------------------------------------------------------------------------------ generic

struct GenericArgs {
  uint32_t heads, kv_heads, chunk_rows, depth, capacity, window, past, query;
  float scale;
  uint32_t* lengths;  // device {past, query, fault} overriding past / query when not null
};

// Run-time lengths read on the device (the reference carries them in a uniform buffer the
// generation context rewrites every run, packages/runtime/src/kernels/state-attention.ts:
// 190-193).  The host checks of the scalar form are repeated here; a violation raises the
// fault word instead of touching memory.
__device__ inline bool device_lengths(uint32_t* lengths, uint32_t chunk_rows, uint32_t capacity,
                                      uint32_t window, uint32_t& past, uint32_t& query) {
  if (!lengths) return true;
  past = lengths[0];
  query = lengths[1];
  const bool ok = query >= 1 && query <= chunk_rows &&
                  (uint64_t)past + query <= 0xffffffffull &&
                  (window != 0 || (uint64_t)past + query <= capacity);
  if (!ok && threadIdx.x == 0) lengths[2] = 1u;
  return ok;
}

// One workgroup per (plane z = b*H + h, row).  Columns are walked 256 at a time: a thread
// scores one column (serial dot over D), the block folds the chunk into the running
// (max, sum), then threads switch to one output dim each and add the chunk's P*V.
template <typename XT, typename ST>
__global__ __launch_bounds__(kThreads) void attention_generic_kernel(
    const XT* __restrict__ q, const XT* __restrict__ ins_k, const XT* __restrict__ ins_v,
    const ST* __restrict__ slot_k, const ST* __restrict__ slot_v, XT* __restrict__ out,
    GenericArgs a) {
  __shared__ float s_q[1024];
  __shared__ float s_p[kThreads];
  __shared__ float s_red[kThreads / kWave];
  __shared__ float s_bcast;

  const uint32_t z = blockIdx.x;
  const uint32_t row = blockIdx.y;
  const uint32_t tid = threadIdx.x;
  const uint32_t D = a.depth;
  const size_t q_base = ((size_t)z * a.chunk_rows + row) * D;
  if (!device_lengths(a.lengths, a.chunk_rows, a.capacity, a.window, a.past, a.query)) return;

  if (row >= a.query) {  // pad row: exact zeros, nothing is read
    for (uint32_t d = tid; d < D; d += kThreads) st_f32<XT>(out, q_base + d, 0.0f);
    return;
  }
  const uint32_t kv_plane = z / (a.heads / a.kv_heads);
  const uint64_t limit = (uint64_t)a.past + row;
  const uint64_t lo = window_low(a.window, limit);
  const uint64_t count = limit - lo + 1;  // >= 1: the row always sees its own column

  for (uint32_t d = tid; d < D; d += kThreads) s_q[d] = ld_f32<XT>(q, q_base + d) * a.scale;
  __syncthreads();

  float run_max = -INFINITY, run_sum = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};  // output dims tid, tid+256, ... (D <= 1024)

  for (uint64_t c0 = 0; c0 < count; c0 += kThreads) {
    const uint64_t col = lo + c0 + tid;
    const bool valid = c0 + tid < count;
    float score = -INFINITY;
    if (valid) {
      float dot = 0.f;
      if (col < a.past) {
        // (a slot column is below `past`, a u32: the ring row is a 32-bit modulo)
        const uint32_t prow = a.window ? (uint32_t)col % a.window : (uint32_t)col;
        const ST* kp = slot_k + ((size_t)kv_plane * a.capacity + prow) * D;
        for (uint32_t d = 0; d < D; ++d) dot = fmaf(s_q[d], ld_f32<ST>(kp, d) * a.scale, dot);
      } else {
        const XT* kp = ins_k + ((size_t)kv_plane * a.chunk_rows + (col - a.past)) * D;
        for (uint32_t d = 0; d < D; ++d) dot = fmaf(s_q[d], ld_f32<XT>(kp, d) * a.scale, dot);
      }
      score = dot;
    }
    // chunk max
    float m = score;
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, kWave));
    if ((tid & (kWave - 1)) == 0) s_red[tid >> 6] = m;
    __syncthreads();
    if (tid == 0) {
      float t = s_red[0];
      for (int i = 1; i < kThreads / kWave; ++i) t = fmaxf(t, s_red[i]);
      s_bcast = fmaxf(t, run_max);
    }
    __syncthreads();
    const float new_max = s_bcast;  // finite: every chunk holds at least one valid column
    const float alpha = expf(run_max - new_max);  // exp(-inf) = 0 on the first chunk
    const float p = valid ? expf(score - new_max) : 0.f;
    s_p[tid] = p;
    float s = p;
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, kWave);
    __syncthreads();  // s_p complete; s_red free to reuse
    if ((tid & (kWave - 1)) == 0) s_red[tid >> 6] = s;
    __syncthreads();
    float chunk_sum = 0.f;
    for (int i = 0; i < kThreads / kWave; ++i) chunk_sum += s_red[i];
    run_sum = run_sum * alpha + chunk_sum;
    run_max = new_max;

    const uint32_t ncols = (uint32_t)((count - c0) < kThreads ? (count - c0) : kThreads);
#pragma unroll
    for (int slot = 0; slot < 4; ++slot) {
      const uint32_t d = tid + slot * kThreads;
      if (d >= D) break;
      float sum = 0.f;
      for (uint32_t c = 0; c < ncols; ++c) {
        const uint64_t vc = lo + c0 + c;
        float v;
        if (vc < a.past) {
          const uint32_t prow = a.window ? (uint32_t)vc % a.window : (uint32_t)vc;
          v = ld_f32<ST>(slot_v, ((size_t)kv_plane * a.capacity + prow) * D + d);
        } else {
          v = ld_f32<XT>(ins_v, ((size_t)kv_plane * a.chunk_rows + (vc - a.past)) * D + d);
        }
        sum = fmaf(s_p[c], v, sum);
      }
      acc[slot] = acc[slot] * alpha + sum;
    }
    __syncthreads();  // before s_p / s_red are overwritten
  }
  const float inv = 1.0f / run_sum;  // run_sum >= 1: the max column contributes exp(0)
#pragma unroll
  for (int slot = 0; slot < 4; ++slot) {
    const uint32_t d = tid + slot * kThreads;
    if (d < D) st_f32<XT>(out, q_base + d, acc[slot] * inv);
  }
}

// ------------------------------------------------------------------- chunks of rows, MFMA
//
// A chunk of M > 1 rows with D = 64 or 128 (a prefill step): workgroup = (plane z, 16 query
// rows), WAVES waves; the key columns the 16 rows can see are walked in blocks of 32 and wave w
// takes blocks w, w + WAVES, ...  All arithmetic is f32 (v_mfma_f32_16x16x4_f32: f32 products,
// f32 sums), the operand roundings are the generic kernel's: q * scale and k * scale are
// rounded before the product.  With g = lane / 16:
//   S^T = K Q^T    two tiles of 16 keys; A = the K tile (row = key, lane group g walks dims
//                  g D/4 ..), B = Q^T (column = query row): a lane ends up with the scores of
//                  ONE query row (lane % 16) against keys 16 t + 4 g + i (t < 2, i < 4), so the
//                  running maximum and sum of the online softmax are per lane, plus an
//                  exchange between the four lane groups;
//   O^T += V^T P^T the scores a lane holds are exactly a B operand if MFMA step (t, i) is
//                  given the keys 16 t + 4 g + i, so the probabilities never move; V^T is the A
//                  operand, read from the parked V block with the same key per step.  The
//                  result again has the query row in lane % 16 (dims 16 dt + 4 g + 0..3).
// K and V blocks are parked in the wave's own LDS area (coalesced 16-byte loads; a block may
// straddle the state slot and this step's rows).  The waves' (max, sum, O) are merged in LDS
// at the end; rows >= query are written as +0.  Sixteen rows a workgroup (not 32) so that a
// 128-row chunk of 32 heads is 256 workgroups, one per CU.
typedef float float4v_t __attribute__((ext_vector_type(4)));

template <typename T>
__device__ inline float4 load4_f32(const T* p);
template <>
__device__ inline float4 load4_f32<float>(const float* p) {
  return *reinterpret_cast<const float4*>(p);
}
template <>
__device__ inline float4 load4_f32<__half>(const __half* p) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  const __half2 a = __builtin_bit_cast(__half2, raw.x), b = __builtin_bit_cast(__half2, raw.y);
  return make_float4(__low2float(a), __high2float(a), __low2float(b), __high2float(b));
}

template <typename XT, typename ST, int D, int WAVES, int RB>
__global__ __launch_bounds__(64 * WAVES) void attention_rows_kernel(
    const XT* __restrict__ q, const XT* __restrict__ ins_k, const XT* __restrict__ ins_v,
    ST* __restrict__ slot_k, ST* __restrict__ slot_v, XT* __restrict__ out,
    GenericArgs a, uint32_t flags) {
  constexpr uint32_t kBlock = 64u * WAVES;
  constexpr int kRows = 16 * RB;              // query rows of a workgroup: RB blocks of 16
  constexpr int kRow = D + 4;                 // floats of a parked row
  constexpr int DT = D / 16;                  // output tiles of 16 dims
  constexpr int kQuarter = D / 4;             // dims a lane group walks
  constexpr int kPieces = D / 4;              // 4-element pieces of a row
  constexpr int kRowsPerLoad = 64 / kPieces;
  constexpr int kLoads = 32 / kRowsPerLoad;
  __shared__ __align__(16) float s_k[WAVES][32 * kRow];
  __shared__ __align__(16) float s_v[WAVES][32 * kRow];
  __shared__ float s_m[WAVES][kRows], s_l[WAVES][kRows];

  const uint32_t z = blockIdx.x, row0 = blockIdx.y * (uint32_t)kRows;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  uint32_t past = a.past, query = a.query;
  if (!device_lengths(a.lengths, a.chunk_rows, a.capacity, a.window, past, query)) return;

  const bool row_major = (flags & KRM_CHUNK_OUT_ROW_MAJOR) != 0;
  const bool out_f16 = (flags & KRM_CHUNK_OUT_F16) != 0;  // fp16 `out` beside f32 q / k / v
  auto out_index = [&](uint32_t row, uint32_t d) -> size_t {
    if (row_major) {  // [B, M, H, D]
      const uint32_t b = z / a.heads, head = z - b * a.heads;
      return (((size_t)b * a.chunk_rows + row) * a.heads + head) * D + d;
    }
    return ((size_t)z * a.chunk_rows + row) * D + d;
  };
  // The chunk's own K / V rows of this block go to the state slots here when asked for (the
  // first query head of each kv plane does it).  Without a window no reader of this launch
  // touches them: slot rows are read for columns < past only, these are rows past + row.
  if ((flags & KRM_CHUNK_APPEND) && z % (a.heads / a.kv_heads) == 0) {
    const uint32_t plane = z / (a.heads / a.kv_heads);
    for (uint32_t i = tid; i < (uint32_t)kRows * kPieces; i += kBlock) {
      const uint32_t rr = i / kPieces, piece = i - rr * kPieces;
      const uint32_t row = row0 + rr;
      if (row >= query) continue;
      const size_t src = ((size_t)plane * a.chunk_rows + row) * D + 4 * piece;
      const size_t dst = ((size_t)plane * a.capacity + past + row) * D + 4 * piece;
      const float4 kv = load4_f32<XT>(ins_k + src), vv = load4_f32<XT>(ins_v + src);
      st_f32<ST>(slot_k, dst, kv.x); st_f32<ST>(slot_k, dst + 1, kv.y);
      st_f32<ST>(slot_k, dst + 2, kv.z); st_f32<ST>(slot_k, dst + 3, kv.w);
      st_f32<ST>(slot_v, dst, vv.x); st_f32<ST>(slot_v, dst + 1, vv.y);
      st_f32<ST>(slot_v, dst + 2, vv.z); st_f32<ST>(slot_v, dst + 3, vv.w);
    }
  }
  if (row0 >= query) {  // a block of pad rows: exact zeros, nothing is read
    for (uint32_t i = tid; i < (uint32_t)kRows * D; i += kBlock) {
      const uint32_t row = row0 + i / D;
      if (row >= a.chunk_rows) continue;
      if (out_f16)
        st_f32<__half>(reinterpret_cast<__half*>(out), out_index(row, i % D), 0.0f);
      else
        st_f32<XT>(out, out_index(row, i % D), 0.0f);
    }
    return;
  }
  const uint32_t kv_plane = z / (a.heads / a.kv_heads);

  // Q block -> LDS (scaled), then each lane's B operands: Q[r][g * D/4 + s]
  for (uint32_t i = tid; i < (uint32_t)kRows * kPieces; i += kBlock) {
    const uint32_t rr = i / kPieces, piece = i - rr * kPieces;
    const uint32_t row = min(row0 + rr, a.chunk_rows - 1);
    float4 v = load4_f32<XT>(q + ((size_t)z * a.chunk_rows + row) * D + 4 * piece);
    v.x *= a.scale; v.y *= a.scale; v.z *= a.scale; v.w *= a.scale;
    *reinterpret_cast<float4*>(&s_k[0][rr * kRow + 4 * piece]) = v;
  }
  __syncthreads();
  float qf[RB][kQuarter];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int i = 0; i < kQuarter / 4; ++i) {
      const float4 v = *reinterpret_cast<const float4*>(
          &s_k[0][(16 * rb + r) * kRow + g * kQuarter + 4 * i]);
      qf[rb][4 * i] = v.x; qf[rb][4 * i + 1] = v.y; qf[rb][4 * i + 2] = v.z; qf[rb][4 * i + 3] = v.w;
    }
  __syncthreads();

  // columns the block's rows can see: [c_lo, limit_hi]
  const uint32_t last_row = min(row0 + (uint32_t)kRows - 1u, query - 1u);
  const uint64_t limit_hi = (uint64_t)past + last_row;
  const uint64_t c_lo = window_low(a.window, (uint64_t)past + row0);
  const uint32_t blocks = (uint32_t)((limit_hi - c_lo) / 32u) + 1u;
  uint64_t my_limit[RB], my_low[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    my_limit[rb] = (uint64_t)past + row0 + (uint32_t)(16 * rb + r);
    my_low[rb] = window_low(a.window, my_limit[rb]);
  }

  float* mk = s_k[wave];
  float* mv = s_v[wave];
  auto wave_sync = [] {  // the areas are the wave's own: its LDS queue orders them
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  float run_m[RB], run_l[RB];
  float4v_t acc[RB][DT];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    run_m[rb] = -INFINITY;
    run_l[rb] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[rb][dt][i] = 0.f;
  }

  for (uint32_t kb = (uint32_t)wave; kb < blocks; kb += (uint32_t)WAVES) {
    const uint64_t c0 = c_lo + (uint64_t)kb * 32u;
    // park the K (scaled) and V rows of the block
    float4 kraw[kLoads], vraw[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      const uint32_t key = j * kRowsPerLoad + lane / kPieces, piece = lane % kPieces;
      uint64_t c = c0 + key;
      c = c < limit_hi ? c : limit_hi;  // beyond the last column: any valid row, masked below
      if (c < past) {
        const uint32_t prow = a.window ? (uint32_t)c % a.window : (uint32_t)c;  // c < past: a u32
        const size_t at = ((size_t)kv_plane * a.capacity + prow) * D + 4 * piece;
        kraw[j] = load4_f32<ST>(slot_k + at);
        vraw[j] = load4_f32<ST>(slot_v + at);
      } else {
        const size_t at = ((size_t)kv_plane * a.chunk_rows + (size_t)(c - past)) * D + 4 * piece;
        kraw[j] = load4_f32<XT>(ins_k + at);
        vraw[j] = load4_f32<XT>(ins_v + at);
      }
    }
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      const uint32_t key = j * kRowsPerLoad + lane / kPieces, piece = lane % kPieces;
      float4 kv = kraw[j];
      kv.x *= a.scale; kv.y *= a.scale; kv.z *= a.scale; kv.w *= a.scale;
      *reinterpret_cast<float4*>(&mk[key * kRow + 4 * piece]) = kv;
      *reinterpret_cast<float4*>(&mv[key * kRow + 4 * piece]) = vraw[j];
    }
    wave_sync();

#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      // (a block past every column these 16 rows can see is skipped: the workgroup's other
      // rows see further)
      if (c0 > (uint64_t)past + row0 + (uint32_t)(16 * rb + 15)) continue;
      // S^T[key][query row], tile t = keys 16 t ..: A = K[16 t + r][g * D/4 + s], B = Q^T
      float4v_t st[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int i = 0; i < 4; ++i) st[t][i] = 0.f;
#pragma unroll
        for (int i = 0; i < kQuarter / 4; ++i) {
          const float4 kf =
              *reinterpret_cast<const float4*>(&mk[(16 * t + r) * kRow + g * kQuarter + 4 * i]);
          st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf.x, qf[rb][4 * i], st[t], 0, 0, 0);
          st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf.y, qf[rb][4 * i + 1], st[t], 0, 0, 0);
          st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf.z, qf[rb][4 * i + 2], st[t], 0, 0, 0);
          st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf.w, qf[rb][4 * i + 3], st[t], 0, 0, 0);
        }
      }
      // this lane: query row 16 rb + r, keys 16 t + 4 g + i
      float block_max = -INFINITY;
      bool valid[2][4];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint64_t c = c0 + (uint32_t)(16 * t + 4 * g + i);
          valid[t][i] = c <= my_limit[rb] && c >= my_low[rb];
          block_max = fmaxf(block_max, valid[t][i] ? st[t][i] : -INFINITY);
        }
      block_max = fmaxf(block_max, __shfl_xor(block_max, 16, kWave));
      block_max = fmaxf(block_max, __shfl_xor(block_max, 32, kWave));
      const float new_m = fmaxf(run_m[rb], block_max);
      const float ref = new_m == -INFINITY ? 0.f : new_m;  // nothing seen yet: exp(-inf - 0) = 0
      const float alpha = expf(run_m[rb] - ref);
      float p[2][4], sum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          p[t][i] = valid[t][i] ? expf(st[t][i] - ref) : 0.f;
          sum += p[t][i];
        }
      run_l[rb] = run_l[rb] * alpha + sum;
      run_m[rb] = new_m;
      // O^T[d][query row] = alpha * O^T + V^T P^T: step (t, i) carries the keys 16 t + 4 g + i
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[rb][dt][i] *= alpha;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float vf = mv[(16 * t + 4 * g + i) * kRow + 16 * dt + r];
            acc[rb][dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf, p[t][i], acc[rb][dt], 0, 0, 0);
          }
      }
    }
    wave_sync();  // the block's rows have been read: the next block may be parked
  }

  // the wave's state: (max, sum) per query row and O[row][d] in its own area
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    run_l[rb] += __shfl_xor(run_l[rb], 16, kWave);
    run_l[rb] += __shfl_xor(run_l[rb], 32, kWave);
    if (g == 0) {
      s_m[wave][16 * rb + r] = run_m[rb];
      s_l[wave][16 * rb + r] = run_l[rb];
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)  // registers 0..3: dims 16 dt + 4 g + 0..3
      *reinterpret_cast<float4*>(&mk[(16 * rb + r) * kRow + 16 * dt + 4 * g]) =
          make_float4(acc[rb][dt][0], acc[rb][dt][1], acc[rb][dt][2], acc[rb][dt][3]);
  }
  __syncthreads();

  // merge of the waves, wave order; 16 threads a row (256 row-part units, dealt over the
  // workgroup's threads: a workgroup of two waves takes two rounds)
  for (uint32_t unit = tid; unit < 256u; unit += kBlock) {
   for (uint32_t rb = 0; rb < (uint32_t)RB; ++rb) {
    constexpr int kPer = D / 16;
    const uint32_t rr = 16u * rb + (unit >> 4), d0 = (unit & 15u) * kPer;
    const uint32_t row = row0 + rr;
    float top = s_m[0][rr];
#pragma unroll
    for (int wv = 1; wv < WAVES; ++wv) top = fmaxf(top, s_m[wv][rr]);  // finite: the own column
    float wgt[WAVES], total_l = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) {
      wgt[wv] = expf(s_m[wv][rr] - top);
      total_l = fmaf(wgt[wv], s_l[wv][rr], total_l);
    }
    const float inv = 1.0f / total_l;
    if (row < a.chunk_rows) {
#pragma unroll
      for (int e = 0; e < kPer; ++e) {
        float o = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) o = fmaf(wgt[wv], s_k[wv][rr * kRow + d0 + e], o);
        float value = row < query ? o * inv : 0.0f;
        if (out_f16 && sizeof(XT) == 4) value = rounded_f32(value);  // the f32 result, rounded again
        if (out_f16)
          st_f32<__half>(reinterpret_cast<__half*>(out), out_index(row, d0 + e), value);
        else
          st_f32<XT>(out, out_index(row, d0 + e), value);
      }
    }
   }
  }
}

// ------------------------------------------------------------------------------ decode

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// Value of lane `src` (0..15) of the caller's 16-lane row, in every lane of that row.
template <int SRC>
__device__ inline float row_broadcast_from(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x150 + SRC, 0xf, 0xf, true));
}
__device__ inline float row_broadcast(float v, int src) {  // `src` is a constant after unrolling
  switch (src) {
    case 0: return row_broadcast_from<0>(v);
    case 1: return row_broadcast_from<1>(v);
    case 2: return row_broadcast_from<2>(v);
    case 3: return row_broadcast_from<3>(v);
    case 4: return row_broadcast_from<4>(v);
    case 5: return row_broadcast_from<5>(v);
    case 6: return row_broadcast_from<6>(v);
    default: return row_broadcast_from<7>(v);
  }
}

// Sum over the LPR consecutive lanes that share one K/V row; all of them get the total.
template <int LPR>
__device__ inline float group_sum(float v) {
  if constexpr (LPR >= 2) {
    int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true);
    v += __builtin_bit_cast(float, t);  // quad_perm [1,0,3,2]
  }
  if constexpr (LPR >= 4) {
    int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true);
    v += __builtin_bit_cast(float, t);  // quad_perm [2,3,0,1]
  }
  if constexpr (LPR >= 8) {
    int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true);
    v += __builtin_bit_cast(float, t);  // row_half_mirror
  }
  if constexpr (LPR >= 16) {
    int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true);
    v += __builtin_bit_cast(float, t);  // row_mirror
  }
  if constexpr (LPR >= 32) v += __shfl_xor(v, 16, kWave);
  if constexpr (LPR >= 64) v += __shfl_xor(v, 32, kWave);
  return v;
}

template <typename ST>
struct RowChunk;  // 16 bytes of a K/V row
template <>
struct RowChunk<__half> {
  static constexpr int E = 8;
  __device__ static inline void unpack(const uint4& raw, float (&f)[8]) {
    const __half2* h = reinterpret_cast<const __half2*>(&raw);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float2 v = __half22float2(h[i]);
      f[2 * i] = v.x;
      f[2 * i + 1] = v.y;
    }
  }
};
template <>
struct RowChunk<float> {
  static constexpr int E = 4;
  __device__ static inline void unpack(const uint4& raw, float (&f)[4]) {
    f[0] = __uint_as_float(raw.x);
    f[1] = __uint_as_float(raw.y);
    f[2] = __uint_as_float(raw.z);
    f[3] = __uint_as_float(raw.w);
  }
};

struct DecodeArgs {
  uint32_t heads, kv_heads;
  uint32_t repeat;           // query heads per kv head (H / Hkv)
  uint32_t head_groups;      // workgroups one kv head's query heads are spread over
  uint32_t window;           // 0 = full context
  uint32_t past;             // single sequence: P.  ragged batch: unused
  uint64_t slot_batch_stride;  // elements between batches of the slot (0 for a ragged batch)
  uint64_t slot_plane_stride;  // elements between kv heads of the slot
  float scale;
  uint32_t nseq;             // ragged batch: sequences; single: batch
  const int32_t* cu_rows;    // ragged batch: [nseq+1] first slot row of each sequence
  const int32_t* split_prefix;  // ragged batch: [nseq+1] first global split of each sequence
  uint32_t* tickets;         // arrival counter (sequence, head unit) at index * kTicketStride, zero between launches
  uint32_t* lengths;         // single sequence: device {past, query, fault} or null
  uint32_t capacity;         // single sequence: slot rows (checked against device lengths)
};

// Columns are walked in chunks of kDecodeIter * G rows (G = 256 / lanes-per-row groups, each
// owning one row per iteration).  Short pasts (<= kSingleSplitChunks chunks) stay in ONE split
// that loops over its chunks — no partials, no merge; longer ones get one chunk per split.
// The rule is a pure function of the number of past columns and the chunk size, so a sequence
// is partitioned the same way alone and inside a ragged batch.
constexpr uint32_t kSingleSplitChunks = 4;
__host__ __device__ inline uint32_t decode_split_columns(uint32_t lanes_per_row) {
  return kDecodeIter * (kThreads / lanes_per_row);
}
__host__ __device__ inline uint32_t decode_chunks(uint64_t slot_columns, uint32_t chunk_columns) {
  return (uint32_t)((slot_columns + chunk_columns - 1) / chunk_columns);
}
// Chunks a split of a long past walks.  Two (both requested before the first is scored) halve
// the partials and help a launch that is bandwidth-bound — the 16-sequence ragged batch went
// from 36.7 to 33.9 us — but a single 4096-column sequence then has 256 workgroups instead of
// 512 and went from 10.1 to 12.6 us; the partition has to be the same function of a
// sequence's columns in both launches (a sequence gives the same bits alone and in a batch),
// so it stays at one.
#ifndef KRM_SPLIT_CHUNKS
#define KRM_SPLIT_CHUNKS 1
#endif
constexpr uint32_t kSplitChunks = KRM_SPLIT_CHUNKS;
__host__ __device__ inline uint32_t decode_splits(uint64_t slot_columns, uint32_t chunk_columns) {
  const uint32_t chunks = decode_chunks(slot_columns, chunk_columns);
  return chunks <= kSingleSplitChunks ? 1u : (chunks + kSplitChunks - 1) / kSplitChunks;
}

constexpr float kLog2e = 1.4426950408889634f;

// Device-scope store / load of one float: written through to (read from) memory that every
// XCD sees, without touching the rest of the cache.
__device__ inline void publish(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline float observe(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
constexpr int kMergeChunk = 32;  // split partials merged per pass (all requested at once)

// Workgroup = (split, kv head, batch | -): 256 threads = G groups of LPR lanes; a group owns
// one K/V row per iteration, a lane 16 bytes of it.  Every group keeps its own running
// (max, sum, weighted V) over the rows it sees — no workgroup barrier inside the column walk —
// and the G group states are merged once at the end, in ascending group order.  Scores live
// in the base-2 domain (q carries scale^2 * log2 e), so exponentials are single v_exp_f32.
// With several splits every workgroup publishes its merged partial; the one that arrives last
// at the (sequence, kv head) counter merges the partials of its r heads in ascending split
// order — the result does not depend on which workgroup that is.
template <typename XT, typename ST, int R, int LPR, bool RAGGED>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 2)))
void attention_decode_kernel(
    const XT* __restrict__ q, const XT* __restrict__ ins_k, const XT* __restrict__ ins_v,
    const ST* __restrict__ slot_k, const ST* __restrict__ slot_v, XT* __restrict__ out,
    float* ws_ml, float* ws_acc, DecodeArgs a) {
  constexpr int E = RowChunk<ST>::E;
  constexpr int D = LPR * E;
  constexpr int G = kThreads / LPR;
  constexpr int kChunkCols = kDecodeIter * G;
  // fp16 queries and fp16 rows of 128 dims: the scores run on the matrix cores
  constexpr bool kMfma = sizeof(XT) == 2 && sizeof(ST) == 2 && LPR == 16 && kDecodeIter == 8;
  constexpr int kOuts = (R * D + kThreads - 1) / kThreads;
  __shared__ float s_m[G][R];
  __shared__ float s_l[G][R];
  __shared__ float s_acc[G][R][D];
  __shared__ float s_w[R][kMergeChunk];
  __shared__ float s_wl[R][kMergeChunk];
  __shared__ uint32_t s_ticket;

  const int tid = threadIdx.x;
  const int sub = tid % LPR;   // which 16 bytes of the row
  const int group = tid / LPR;
  const uint32_t hk = blockIdx.y / a.head_groups;
  const uint32_t head0 = hk * a.repeat + (blockIdx.y - hk * a.head_groups) * R;  // first head

  // The rows of a chunk as they arrive: K pieces (row-owner layout, or the MFMA A-operand
  // layout: piece tile*4 + t) and V pieces (row-owner layout).
  struct ChunkRows {
    uint4 k[kDecodeIter];
    uint4 v[kDecodeIter];
  };
  const int wave = tid >> 6, lane = tid & 63;
  const int frag_row = lane & 15, frag_g = lane >> 4;
  // offset inside a chunk of the column that (lane group, iteration) owns
  auto column_of = [&](int it) -> uint32_t {
    if constexpr (kMfma)
      return (uint32_t)((wave * 2 + it / 4) * 16 + 4 * frag_g + (it & 3));
    else
      return (uint32_t)(it * G + group);
  };
  // Requests only: every K row, then every V row of the `width` columns from c_begin of a slot;
  // unconditional (a column past the end re-reads the first column and is masked when used).
  auto request_rows = [&](const ST* kslot, const ST* vslot, uint32_t first_row, uint32_t c_begin,
                          uint32_t width, ChunkRows& rows) {
    // Physical row of column c_begin, found once; the columns of a chunk follow it and wrap
    // at most once (a launch's live slot columns number fewer than the window).  A modulo per
    // request cost about 35 instructions and a branch each: 0.9 us to ask for a chunk's rows.
    const uint32_t r_begin = a.window ? c_begin % a.window : c_begin;
    const uint32_t wrap = a.window ? a.window : 0xFFFFFFFFu;
    auto slot_row = [&](uint32_t offset) {  // element offset of the row's first dim
      const uint32_t r = r_begin + (offset < width ? offset : 0u);
      return (size_t)(first_row + (r >= wrap ? r - wrap : r)) * D;
    };
    if constexpr (kMfma) {
      // lane (r = lane % 16, g = lane / 16) takes 16 bytes of K row r of each 16-row tile at
      // dims 32t + 8g..: the A-operand layout of v_mfma_f32_16x16x32_f16
#pragma unroll
      for (int tile = 0; tile < 2; ++tile) {
        const size_t at = slot_row((uint32_t)((wave * 2 + tile) * 16 + frag_row));
#pragma unroll
        for (int t = 0; t < 4; ++t)
          rows.k[tile * 4 + t] =
              *reinterpret_cast<const uint4*>(kslot + at + 32 * t + 8 * frag_g);
      }
    } else {
#pragma unroll
      for (int it = 0; it < kDecodeIter; ++it)
        rows.k[it] = *reinterpret_cast<const uint4*>(kslot + slot_row(column_of(it)) + sub * E);
    }
#pragma unroll
    for (int it = 0; it < kDecodeIter; ++it)
      rows.v[it] = *reinterpret_cast<const uint4*>(vslot + slot_row(column_of(it)) + sub * E);
  };

  // Lengths that live on the device (a recorded decode step) cost a dependent round trip before
  // the first address is known.  Without a window the first chunk of a split does not depend
  // on them — only how many of its columns count does — so its rows are asked for right away,
  // bounded by the slot's capacity instead of the past; columns that turn out to lie beyond
  // the past are masked when the chunk is used, like any ragged end.
  ChunkRows rows0;
  bool early = false;
  if constexpr (!RAGGED) {
    early = a.lengths != nullptr && a.window == 0;
    if (early) {
      const size_t base = (size_t)blockIdx.z * a.slot_batch_stride + (size_t)hk * a.slot_plane_stride;
      const uint32_t want = blockIdx.x * (kSplitChunks * (uint32_t)kChunkCols);
      const uint32_t c_begin = want < a.capacity ? want : a.capacity - 1u;
      const uint32_t room = a.capacity - c_begin;
      request_rows(slot_k + base, slot_v + base, 0u, c_begin,
                   room < (uint32_t)kChunkCols ? room : (uint32_t)kChunkCols, rows0);
    }
  }

  // Columns and slot rows are 32-bit (pastLength is a u32, a ragged batch holds < 2^31 rows);
  // only the final byte address is 64-bit: 64-bit index math per load costs more than the
  // attention arithmetic of a short past.
  uint32_t seq, split, nsplit, first_split;
  uint32_t past, row_base;
  if constexpr (RAGGED) {
    // binary search: last sequence whose first split is <= blockIdx.x
    uint32_t lo_i = 0, hi_i = a.nseq;
    while (hi_i - lo_i > 1) {
      const uint32_t mid = (lo_i + hi_i) >> 1;
      if ((uint32_t)a.split_prefix[mid] <= blockIdx.x) lo_i = mid; else hi_i = mid;
    }
    seq = lo_i;
    first_split = (uint32_t)a.split_prefix[seq];
    nsplit = (uint32_t)a.split_prefix[seq + 1] - first_split;
    split = blockIdx.x - first_split;
    if (split >= nsplit) return;  // a grid sized for the most splits the batch may need
    row_base = (uint32_t)a.cu_rows[seq];
    past = (uint32_t)a.cu_rows[seq + 1] - row_base;
  } else {
    seq = blockIdx.z;
    uint32_t p32 = a.past, q32 = 1;
    if (!device_lengths(a.lengths, 1, a.capacity, a.window, p32, q32)) return;
    past = p32;
    row_base = 0;
    nsplit = decode_splits(past - window_low(a.window, past), kChunkCols);
    split = blockIdx.x;
    // The grid and the workspace were sized on the host for the longest past the launch may
    // see.  A replay whose device-side past needs more splits than that would never complete a
    // ticket round and would index partials beyond the workspace: raise the fault word and
    // leave everything untouched instead.
    if (nsplit > gridDim.x) {
      if (a.lengths && blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) a.lengths[2] = 1u;
      return;
    }
    if (split >= nsplit) return;  // the grid is sized for the longest past it may see
    first_split = seq * nsplit;
  }
  const uint32_t low = (uint32_t)window_low(a.window, past);  // limit of row 0 is `past`
  const uint32_t total_chunks = decode_chunks(past - low, kChunkCols);
  const uint32_t my_chunks =
      nsplit == 1 ? total_chunks : min(kSplitChunks, total_chunks - split * kSplitChunks);
  const uint32_t c_first = low + split * (kSplitChunks * kChunkCols);  // < past (split 0 alone)
  const bool last = split + 1 == nsplit;

  const size_t slot_base = (size_t)seq * a.slot_batch_stride + (size_t)hk * a.slot_plane_stride;
  const ST* kslot = slot_k + slot_base;
  const ST* vslot = slot_v + slot_base;

  // this step's own row and the query heads (valid addresses for every lane)
  const bool own = last && group == 0;  // the lanes that also take this step's own column
  float kx[E], vx[E];
  {
    const size_t ins_base = ((size_t)seq * a.kv_heads + hk) * D + sub * E;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      kx[e] = ld_f32<XT>(ins_k, ins_base + e);
      vx[e] = ld_f32<XT>(ins_v, ins_base + e);
    }
  }
  float qf[R][E];
#pragma unroll
  for (int h = 0; h < R; ++h) {
    const size_t q_base = ((size_t)seq * a.heads + head0 + h) * D + sub * E;
#pragma unroll
    for (int e = 0; e < E; ++e)
      qf[h][e] = ((ld_f32<XT>(q, q_base + e) * a.scale) * a.scale) * kLog2e;
  }

  // B operand of the score MFMAs: lane (n = lane % 16, g = lane / 16) holds head n's query at
  // dims 32t + 8g.. as raw fp16 (exact products; the scale is applied to the f32 score)
  half8_t qb[kMfma ? 4 : 1];
  if constexpr (kMfma) {
    const int n = tid & 15, g = (tid & 63) >> 4;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const size_t at = ((size_t)seq * a.heads + head0 + (n < R ? n : 0)) * D + 32 * t + 8 * g;
      uint4 raw = *reinterpret_cast<const uint4*>(reinterpret_cast<const __half*>(q) + at);
      const uint32_t keep_bits = n < R ? 0xFFFFFFFFu : 0u;
      raw.x &= keep_bits; raw.y &= keep_bits; raw.z &= keep_bits; raw.w &= keep_bits;
      qb[t] = __builtin_bit_cast(half8_t, raw);
    }
  }

  float run_m[R], run_l[R], acc[R][E];
#pragma unroll
  for (int h = 0; h < R; ++h) {
    run_m[h] = -INFINITY;
    run_l[h] = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) acc[h][e] = 0.f;
  }

  auto chunk_begin = [&](uint32_t chunk) { return c_first + chunk * kChunkCols; };
  auto chunk_end = [&](uint32_t c_begin) {  // c_begin < past: no overflow
    return past - c_begin > (uint32_t)kChunkCols ? c_begin + kChunkCols : past;
  };
  auto load_chunk = [&](uint32_t chunk, ChunkRows& rows) {
    const uint32_t c_begin = chunk_begin(chunk);
    request_rows(kslot, vslot, row_base, c_begin, chunk_end(c_begin) - c_begin, rows);
  };
  auto consume_chunk = [&](uint32_t chunk, ChunkRows& rows) {
    const uint32_t c_begin = chunk_begin(chunk), width = chunk_end(c_begin) - c_begin;
    bool valid[kDecodeIter];
#pragma unroll
    for (int it = 0; it < kDecodeIter; ++it) valid[it] = column_of(it) < width;
    float sc[kDecodeIter][R];
    float cm[R];
#pragma unroll
    for (int h = 0; h < R; ++h) cm[h] = -INFINITY;
    if constexpr (kMfma) {
      // Scores on the matrix cores: the query heads are the B operand (one column per head);
      // lane (h, g) receives the scores of columns 4g..4g+3 of a tile for head h, and lane
      // group g owns exactly those columns for P*V, so a score reaches its group with one
      // broadcast inside the 16-lane row.
      float4_t scores[2];
#pragma unroll
      for (int tile = 0; tile < 2; ++tile) {
        scores[tile] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 4; ++t)
          scores[tile] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
              __builtin_bit_cast(half8_t, rows.k[tile * 4 + t]), qb[t], scores[tile], 0, 0, 0);
      }
      const float qscale = (a.scale * a.scale) * kLog2e;
#pragma unroll
      for (int it = 0; it < kDecodeIter; ++it) {
        const float mine = scores[it / 4][it & 3] * qscale;  // (column of `it`, head lane % 16)
#pragma unroll
        for (int h = 0; h < R; ++h) {
          sc[it][h] = valid[it] ? row_broadcast(mine, h) : -INFINITY;
          cm[h] = fmaxf(cm[h], sc[it][h]);
        }
      }
    } else {
#pragma unroll
      for (int it = 0; it < kDecodeIter; ++it) {
        float kf[E];
        RowChunk<ST>::unpack(rows.k[it], kf);
#pragma unroll
        for (int h = 0; h < R; ++h) {
          float part = 0.f;
#pragma unroll
          for (int e = 0; e < E; ++e) part = fmaf(qf[h][e], kf[e], part);
          part = group_sum<LPR>(part);
          sc[it][h] = valid[it] ? part : -INFINITY;
          cm[h] = fmaxf(cm[h], sc[it][h]);
        }
      }
    }
    float keep[R], ref[R];
#pragma unroll
    for (int h = 0; h < R; ++h) {
      const float m_new = fmaxf(run_m[h], cm[h]);
      ref[h] = m_new == -INFINITY ? 0.f : m_new;      // nothing seen yet: 2^(-inf - 0) = 0
      keep[h] = __builtin_amdgcn_exp2f(run_m[h] - ref[h]);
      run_m[h] = m_new;
      run_l[h] *= keep[h];
#pragma unroll
      for (int e = 0; e < E; ++e) acc[h][e] *= keep[h];
    }
#pragma unroll
    for (int it = 0; it < kDecodeIter; ++it) {
      uint4 raw = rows.v[it];
      const uint32_t keep_bits = valid[it] ? 0xFFFFFFFFu : 0u;  // a masked column: no Inf * 0
      raw.x &= keep_bits; raw.y &= keep_bits; raw.z &= keep_bits; raw.w &= keep_bits;
      float vf[E];
      RowChunk<ST>::unpack(raw, vf);
#pragma unroll
      for (int h = 0; h < R; ++h) {
        const float p = __builtin_amdgcn_exp2f(sc[it][h] - ref[h]);  // 0 outside the chunk
        run_l[h] += p;
#pragma unroll
        for (int e = 0; e < E; ++e) acc[h][e] = fmaf(p, vf[e], acc[h][e]);
      }
    }
  };
  // One head, a short past walked by this workgroup alone: the rows of the first two or three
  // chunks are requested together (a chunk costs 0.95 us when each waits for its own round
  // trip; 3 x 32 registers of rows fit beside one head's state).  Each case holds its loads and
  // their uses in one branch: a branch between a load and its use makes the compiler wait
  // inside it.
  if (!early) load_chunk(0, rows0);  // harmless when the split has no column at all
  bool walked = false;
  if constexpr (R == 1) {
    if (nsplit == 1 && total_chunks == 2) {
      ChunkRows rows1;
      load_chunk(1, rows1);
      consume_chunk(0, rows0);
      consume_chunk(1, rows1);
      walked = true;
    } else if (nsplit == 1 && total_chunks > 2) {
      // (the variant that scores on the matrix cores holds more state: two chunks at once keep
      // it within 256 registers, i.e. two workgroups a CU for its many-split launches)
      ChunkRows rows1;
      load_chunk(1, rows1);
      if constexpr (!kMfma) {
        ChunkRows rows2;
        load_chunk(2, rows2);
        consume_chunk(0, rows0);
        consume_chunk(1, rows1);
        consume_chunk(2, rows2);
      } else {
        consume_chunk(0, rows0);
        consume_chunk(1, rows1);
      }
      for (uint32_t chunk = kMfma ? 2 : 3; chunk < total_chunks; ++chunk) {
        load_chunk(chunk, rows0);
        consume_chunk(chunk, rows0);
      }
      walked = true;
    }
  }
  if (!walked && my_chunks > 0) {
    if (kSplitChunks == 2 && nsplit > 1 && my_chunks == 2) {
      // a split of a long past: both chunks requested before the first is scored
      ChunkRows rows1;
      load_chunk(1, rows1);
      consume_chunk(0, rows0);
      consume_chunk(1, rows1);
    } else {
      consume_chunk(0, rows0);
      for (uint32_t chunk = 1; chunk < my_chunks; ++chunk) {
        load_chunk(chunk, rows0);
        consume_chunk(chunk, rows0);
      }
    }
  }
  // this step's own column: one more row for group 0 of the last split (for every other lane
  // the update below is the identity, so the other splits skip it)
  if (last) {
#pragma unroll
    for (int h = 0; h < R; ++h) {
      float part = 0.f;
#pragma unroll
      for (int e = 0; e < E; ++e) part = fmaf(qf[h][e], kx[e], part);
      part = group_sum<LPR>(part);
      const float s_own = own ? part : -INFINITY;
      const float m_new = fmaxf(run_m[h], s_own);
      const float ref = m_new == -INFINITY ? 0.f : m_new;
      const float keep = __builtin_amdgcn_exp2f(run_m[h] - ref);
      const float p = __builtin_amdgcn_exp2f(s_own - ref);
      run_m[h] = m_new;
      run_l[h] = run_l[h] * keep + p;
#pragma unroll
      for (int e = 0; e < E; ++e)
        acc[h][e] = fmaf(p, own ? vx[e] : 0.f, acc[h][e] * keep);  // 0 * NaN must not leak
    }
  }

  // merge of the G group states, ascending group order
#pragma unroll
  for (int h = 0; h < R; ++h) {
#pragma unroll
    for (int e = 0; e < E; ++e) s_acc[group][h][sub * E + e] = acc[h][e];
    if (sub == 0) {
      s_m[group][h] = run_m[h];
      s_l[group][h] = run_l[h];
    }
  }
  __syncthreads();
  const uint32_t gsplit = first_split + split;
  float part_o[kOuts], part_l[kOuts], part_m[kOuts];
#pragma unroll
  for (int i = 0; i < kOuts; ++i) {
    const int o = tid + i * kThreads;
    part_o[i] = part_l[i] = 0.f;
    part_m[i] = -INFINITY;
    if (o >= R * D) continue;
    const int h = o / D, d = o - h * D;
    float m = s_m[0][h];
#pragma unroll
    for (int g = 1; g < G; ++g) m = fmaxf(m, s_m[g][h]);  // finite: the split holds a column
    float total = 0.f, l = 0.f;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float wgt = __builtin_amdgcn_exp2f(s_m[g][h] - m);
      total = fmaf(wgt, s_acc[g][h][d], total);
      l = fmaf(wgt, s_l[g][h], l);
    }
    part_o[i] = total;
    part_l[i] = l;
    part_m[i] = m;
    if (nsplit == 1) {
      st_f32<XT>(out, ((size_t)seq * a.heads + head0 + h) * D + d, total / l);
    } else {
      const size_t slot_index = (size_t)gsplit * a.heads + head0 + h;
      publish(&ws_acc[slot_index * D + d], total);
      if (d == 0) {
        publish(&ws_ml[slot_index * 2], m);
        publish(&ws_ml[slot_index * 2 + 1], l);
      }
    }
  }
  if (nsplit == 1) return;

  // Arrival: the partial was written through to memory (device-scope stores); once every
  // thread's stores have completed, take a ticket.  The last arrival merges, reading the
  // partials with device-scope loads.  No cache-wide write-back or invalidate is involved.
  // The wait is spelled out: a workgroup-scope release fence does not wait for global stores
  // on this target, and a device-scope one writes the whole L2 back.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  uint32_t* ticket = &a.tickets[(size_t)(seq * gridDim.y + blockIdx.y) * kTicketStride];
  if (tid == 0)
    s_ticket = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (s_ticket + 1 != nsplit) return;

  // Merge nsplit partials of each of the R heads, kMergeChunk at a time, ascending order; the
  // partial rows of a pass are all requested before any is used.
  // Every output element tracks the running (max, sum) of its own head: the same numbers in
  // all elements of a head, and one exponential per partial instead of one per use.
  float tot_m[kOuts], tot_l[kOuts], tot_o[kOuts];
#pragma unroll
  for (int i = 0; i < kOuts; ++i) {
    tot_m[i] = -INFINITY;
    tot_l[i] = 0.f;
    tot_o[i] = 0.f;
  }
  for (uint32_t s0 = 0; s0 < nsplit; s0 += kMergeChunk) {
    const uint32_t cnt = nsplit - s0 < (uint32_t)kMergeChunk ? nsplit - s0 : (uint32_t)kMergeChunk;
    // the weighted rows first (long latency), the small (max, sum) pairs next
    float rows[kOuts][kMergeChunk];
#pragma unroll
    for (int i = 0; i < kOuts; ++i) {
      const int o = tid + i * kThreads;
      const int oo = o < R * D ? o : 0;
      const int h = oo / D, d = oo - h * D;
      const float* src = ws_acc + ((size_t)(first_split + s0) * a.heads + head0 + h) * D + d;
      const size_t stride = (size_t)a.heads * D;
#pragma unroll
      for (int j = 0; j < kMergeChunk; ++j)
        rows[i][j] = observe(&src[(size_t)((uint32_t)j < cnt ? j : 0) * stride]);
    }
    __syncthreads();
    for (uint32_t i = tid; i < R * kMergeChunk; i += kThreads) {
      const uint32_t h = i / kMergeChunk, s = i - h * kMergeChunk;
      const size_t slot_index = (size_t)(first_split + s0 + (s < cnt ? s : 0)) * a.heads + head0 + h;
      s_w[h][s] = s < cnt ? observe(&ws_ml[slot_index * 2]) : -INFINITY;
      s_wl[h][s] = s < cnt ? observe(&ws_ml[slot_index * 2 + 1]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kOuts; ++i) {
      const int o = tid + i * kThreads;
      const int h = (o < R * D ? o : 0) / D;
      float m = tot_m[i];
#pragma unroll
      for (int j = 0; j < kMergeChunk; ++j) m = fmaxf(m, s_w[h][j]);
      const float keep = __builtin_amdgcn_exp2f(tot_m[i] - m);  // 0 on the first pass
      float l = tot_l[i] * keep, total = tot_o[i] * keep;
#pragma unroll
      for (int j = 0; j < kMergeChunk; ++j) {
        const float wgt = __builtin_amdgcn_exp2f(s_w[h][j] - m);
        l = fmaf(wgt, s_wl[h][j], l);
        total = fmaf(wgt, rows[i][j], total);
      }
      tot_m[i] = m;
      tot_l[i] = l;
      tot_o[i] = total;
    }
  }
#pragma unroll
  for (int i = 0; i < kOuts; ++i) {
    const int o = tid + i * kThreads;
    if (o >= R * D) break;
    const int h = o / D, d = o - h * D;
    st_f32<XT>(out, ((size_t)seq * a.heads + head0 + h) * D + d, tot_o[i] / tot_l[i]);
  }
  if (tid == 0)  // ready for the next launch
    __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct DecodeLaunch {
  krm_buf q, ins_k, ins_v, slot_k, slot_v, out;
  float* ws_ml;
  float* ws_acc;
  DecodeArgs args;
  uint32_t grid_x, grid_z;     // splits (or total splits), batch
  uint32_t ticket_slots = kTicketSlots;  // counters behind args.tickets
  bool clear_tickets = false;  // zero the counters this launch uses before it runs
};

// Fill kernel for arrival counters (a kernel, not a memset, so that a caller may record it).
__global__ void clear_tickets_kernel(uint32_t* tickets, uint32_t count) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) tickets[(size_t)i * kTicketStride] = 0u;
}

template <typename XT, typename ST, int R, int LPR, bool RAGGED>
int32_t launch_decode(krm_ctx* ctx, const DecodeLaunch& L) {
  attention_decode_kernel<XT, ST, R, LPR, RAGGED>
      <<<dim3(L.grid_x, L.args.kv_heads * L.args.head_groups, L.grid_z), dim3(kThreads), 0,
         ctx->stream>>>(
          ptr<const XT>(L.q), ptr<const XT>(L.ins_k), ptr<const XT>(L.ins_v),
          ptr<const ST>(L.slot_k), ptr<const ST>(L.slot_v), ptr<XT>(L.out), L.ws_ml, L.ws_acc,
          L.args);
  return launched(ctx, "attention_decode_kernel");
}

// `per_block` = query heads one workgroup carries (a divisor of H / Hkv).  A head's result
// does not depend on it: every head keeps its own running state and its own merge.
template <typename XT, typename ST, int LPR, bool RAGGED>
int32_t decode_by_repeat(krm_ctx* ctx, const DecodeLaunch& L, uint32_t per_block) {
  switch (per_block) {
    case 1: return launch_decode<XT, ST, 1, LPR, RAGGED>(ctx, L);
    case 2: return launch_decode<XT, ST, 2, LPR, RAGGED>(ctx, L);
    case 4: return launch_decode<XT, ST, 4, LPR, RAGGED>(ctx, L);
    case 8:
      // (rows that span a whole wave: eight heads' state does not fit the registers)
      if constexpr (LPR < 64) return launch_decode<XT, ST, 8, LPR, RAGGED>(ctx, L);
      [[fallthrough]];
    default: return fail(ctx, KRM_ERR_VALIDATION, "decode attention: %u heads per block", per_block);
  }
}

template <typename XT, typename ST, bool RAGGED>
int32_t decode_by_depth(krm_ctx* ctx, const DecodeLaunch& L, uint32_t per_block, uint32_t lpr) {
  switch (lpr) {
    case 4: return decode_by_repeat<XT, ST, 4, RAGGED>(ctx, L, per_block);
    case 8: return decode_by_repeat<XT, ST, 8, RAGGED>(ctx, L, per_block);
    case 16: return decode_by_repeat<XT, ST, 16, RAGGED>(ctx, L, per_block);
    case 32: return decode_by_repeat<XT, ST, 32, RAGGED>(ctx, L, per_block);
    case 64: return decode_by_repeat<XT, ST, 64, RAGGED>(ctx, L, per_block);
    default: return fail(ctx, KRM_ERR_VALIDATION, "decode attention: %u lanes per row", lpr);
  }
}

// Few (split, kv head) pairs leave most of the chip idle while each workgroup walks its
// columns once per query head; the query heads of a kv head are then spread over several
// workgroups (each re-reads the K/V rows, which the L2 serves) until the grid covers the CUs.
template <bool RAGGED>
int32_t decode_dispatch(krm_ctx* ctx, DecodeLaunch& L, uint32_t repeat, uint32_t lpr,
                        int32_t io_dtype, int32_t kv_dtype) {
  uint32_t per_block = repeat;
  uint64_t blocks = (uint64_t)L.grid_x * L.grid_z * L.args.kv_heads;
  while (per_block > 1 && (blocks < 2ull * (uint64_t)ctx->num_cus || (lpr == 64 && per_block > 4))) {
    per_block >>= 1;
    blocks <<= 1;
  }

  L.args.repeat = repeat;
  L.args.head_groups = repeat / per_block;
  const uint64_t counters = (uint64_t)L.args.nseq * L.args.kv_heads * L.args.head_groups;
  if ((uint64_t)L.args.kv_heads * L.args.head_groups > 65535 || counters > L.ticket_slots)
    return fail(ctx, KRM_ERR_VALIDATION, "decode attention: B * H = %llu exceeds %u",
                (unsigned long long)counters, L.ticket_slots);
  if (L.clear_tickets) {
    clear_tickets_kernel<<<dim3(((uint32_t)counters + 255) / 256), dim3(256), 0, ctx->stream>>>(
        L.args.tickets, (uint32_t)counters);
    KRM_TRY(launched(ctx, "clear_tickets_kernel"));
  }
  if (io_dtype == KRM_F16 && kv_dtype == KRM_F16)
    return decode_by_depth<__half, __half, RAGGED>(ctx, L, per_block, lpr);
  if (io_dtype == KRM_F32 && kv_dtype == KRM_F32)
    return decode_by_depth<float, float, RAGGED>(ctx, L, per_block, lpr);
  if (io_dtype == KRM_F32 && kv_dtype == KRM_F16)
    return decode_by_depth<float, __half, RAGGED>(ctx, L, per_block, lpr);
  return decode_by_depth<__half, float, RAGGED>(ctx, L, per_block, lpr);
}

// lanes a K/V row of `depth` elements spans with 16-byte pieces; 0 = not covered
uint32_t decode_lanes_per_row(uint32_t depth, int32_t kv_dtype) {
  const uint32_t row_bytes = depth * (uint32_t)dtype_bytes(kv_dtype);
  if (row_bytes % 16) return 0;
  const uint32_t lpr = row_bytes / 16;
  return (lpr == 4 || lpr == 8 || lpr == 16 || lpr == 32 || lpr == 64) ? lpr : 0;
}

bool decode_repeat_ok(uint32_t repeat) {
  return repeat == 1 || repeat == 2 || repeat == 4 || repeat == 8;
}

template <typename XT, typename ST>
int32_t launch_generic(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v, krm_buf slot_k,
                       krm_buf slot_v, krm_buf out, uint32_t batch, const GenericArgs& a) {
  attention_generic_kernel<XT, ST>
      <<<dim3(batch * a.heads, a.chunk_rows), dim3(kThreads), 0, ctx->stream>>>(
          ptr<const XT>(q), ptr<const XT>(ins_k), ptr<const XT>(ins_v), ptr<const ST>(slot_k),
          ptr<const ST>(slot_v), ptr<XT>(out), a);
  return launched(ctx, "attention_generic_kernel");
}

template <typename XT, typename ST>
int32_t launch_rows(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v, krm_buf slot_k,
                    krm_buf slot_v, krm_buf out, uint32_t batch, const GenericArgs& a,
                    uint32_t flags) {
  // D = 64: eight waves, two a SIMD, so that one wave's softmax and LDS traffic run under the
  // other's MFMAs; the parked blocks of eight waves of D = 128 would not fit the LDS.  A
  // workgroup takes one block of 16 query rows, or two (the parked K / V blocks then serve
  // both) once that still leaves two workgroups per CU.  A row's arithmetic is the same in
  // both forms and the wave count depends on D only, so its bits depend neither on the chunk
  // length, the batch, the past or the capacity nor on the lengths form.
  const uint32_t row_blocks = (a.chunk_rows + 15) / 16;
  // (with a window the key blocks start at the first row's lower bound, which a second row
  // block would not share: one block a workgroup there)
  const bool two = a.window == 0 && a.depth != 256 &&
                   (uint64_t)batch * a.heads * ((row_blocks + 1) / 2) >= 2ull * ctx->num_cus;
  const dim3 grid(batch * a.heads, two ? (row_blocks + 1) / 2 : row_blocks);
#define KRM_ROWS_ATTENTION(DEPTH, WAVES, RB)                                                   \
  attention_rows_kernel<XT, ST, DEPTH, WAVES, RB><<<grid, dim3(64 * WAVES), 0, ctx->stream>>>( \
      ptr<const XT>(q), ptr<const XT>(ins_k), ptr<const XT>(ins_v), ptr<ST>(slot_k),           \
      ptr<ST>(slot_v), ptr<XT>(out), a, flags)
  if (a.depth == 256) {
    // two waves: a parked block of 32 rows of 256 floats is 33 KB for K and as much for V
    KRM_ROWS_ATTENTION(256, 2, 1);
  } else if (a.depth == 64) {
    if (two) KRM_ROWS_ATTENTION(64, 8, 2); else KRM_ROWS_ATTENTION(64, 8, 1);
  } else {
    if (two) KRM_ROWS_ATTENTION(128, 4, 2); else KRM_ROWS_ATTENTION(128, 4, 1);
  }
#undef KRM_ROWS_ATTENTION
  return launched(ctx, "attention_rows_kernel");
}

// smallest split any dtype uses for this head dim (f32 rows span the most lanes)
uint32_t min_split_columns(uint32_t depth) {
  uint32_t lpr = decode_lanes_per_row(depth, KRM_F32);
  if (!lpr) lpr = decode_lanes_per_row(depth, KRM_F16);
  return lpr ? decode_split_columns(lpr) : 0;
}

}  // namespace

extern "C" {

int32_t krm_attention_state_workspace(uint32_t batch, uint32_t heads, uint32_t kv_heads,
                                      uint32_t chunk_rows, uint32_t depth, uint32_t window,
                                      uint32_t max_past, uint32_t max_query, size_t* bytes) {
  (void)kv_heads;
  (void)chunk_rows;
  (void)max_query;
  if (!bytes) return fail(nullptr, KRM_ERR_VALIDATION, "krm_attention_state_workspace: NULL");
  const uint32_t sc = min_split_columns(depth);
  uint64_t columns = max_past;
  if (window && columns > window - 1) columns = window - 1;
  const uint64_t nsplit = sc ? decode_splits(columns, sc) : 1;
  *bytes = (size_t)batch * heads * nsplit * ((size_t)depth + 2) * sizeof(float) + 256;
  return KRM_OK;
}

// `lengths` == 0: past / query are this run's values.  Otherwise they are read on the device
// and `past` is the largest pastLength the launch has to be sized for.
// `tickets` == nullptr: the context's arrival counters.  Otherwise counters supplied by the
// caller (`ticket_slots` of them, kTicketStride words apart), which this call clears first.
static int32_t attention_state_impl(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                                    krm_buf slot_k, krm_buf slot_v, krm_buf out, uint32_t batch,
                                    uint32_t heads, uint32_t kv_heads, uint32_t chunk_rows,
                                    uint32_t depth, uint32_t capacity, uint32_t window,
                                    float half_scale, uint32_t past, uint32_t query,
                                    krm_buf lengths, int32_t io_dtype, int32_t kv_dtype,
                                    krm_buf workspace, size_t workspace_bytes,
                                    uint32_t* tickets = nullptr, uint32_t ticket_slots = 0,
                                    uint32_t chunk_flags = 0, bool chunk_only = false) {
  KRM_TRY(enter(ctx));
  const bool dyn = lengths != 0;
  KRM_REQUIRE(ctx, aligned(lengths, 4), "krm_attention_state: misaligned lengths buffer");
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(kv_dtype),
              "krm_attention_state: io_dtype %d / kv_dtype %d", io_dtype, kv_dtype);
  KRM_REQUIRE(ctx,
              batch >= 1 && heads >= 1 && kv_heads >= 1 && chunk_rows >= 1 && depth >= 1 &&
                  capacity >= 1,
              "krm_attention_state: B / H / Hkv / M / D / C must be positive "
              "(%u / %u / %u / %u / %u / %u)",
              batch, heads, kv_heads, chunk_rows, depth, capacity);
  KRM_REQUIRE(ctx, heads % kv_heads == 0, "krm_attention_state: H = %u is not a multiple of Hkv = %u",
              heads, kv_heads);
  KRM_REQUIRE(ctx, window <= capacity, "krm_attention_state: window %u exceeds capacity %u",
              window, capacity);
  KRM_REQUIRE(ctx, std::isfinite(half_scale), "krm_attention_state: scale is not finite");
  KRM_REQUIRE(ctx, depth <= 1024, "krm_attention_state: D = %u exceeds 1024", depth);
  KRM_REQUIRE(ctx, (uint64_t)batch * heads <= 0x7fffffffull && chunk_rows <= 65535,
              "krm_attention_state: B*H = %llu or M = %u exceeds the launch grid",
              (unsigned long long)batch * heads, chunk_rows);
  if (!dyn && (query < 1 || query > chunk_rows))
    return fail(ctx, KRM_ERR_EXECUTION, "krm_attention_state: queryLength %u is outside 1..%u",
                query, chunk_rows);
  if (!dyn && (uint64_t)past + query > 0xffffffffull)
    return fail(ctx, KRM_ERR_EXECUTION,
                "krm_attention_state: pastLength %u + queryLength %u does not fit in 32 bits",
                past, query);
  if (!dyn && window == 0 && (uint64_t)past + query > capacity)
    return fail(ctx, KRM_ERR_EXECUTION,
                "krm_attention_state: pastLength %u + queryLength %u exceeds capacity %u", past,
                query, capacity);
  KRM_REQUIRE(ctx, q && ins_k && ins_v && slot_k && slot_v && out,
              "krm_attention_state: NULL buffer");
  const size_t io_b = dtype_bytes(io_dtype), kv_b = dtype_bytes(kv_dtype);
  KRM_REQUIRE(ctx,
              aligned(q, io_b) && aligned(ins_k, io_b) && aligned(ins_v, io_b) &&
                  aligned(out, io_b) && aligned(slot_k, kv_b) && aligned(slot_v, kv_b),
              "krm_attention_state: misaligned buffer");

  const uint32_t repeat = heads / kv_heads;
  const uint32_t lpr = decode_lanes_per_row(depth, kv_dtype);
  const bool fast = !chunk_only && (dyn || query == 1) && chunk_rows == 1 && lpr &&
                    decode_repeat_ok(repeat) &&
                    aligned(slot_k, 16) && aligned(slot_v, 16) && aligned(q, 16) && batch <= 65535 &&
                    heads <= 65535 &&
                    (uint64_t)batch * heads <= (tickets ? ticket_slots : kTicketSlots);
  if (fast) {
    const uint64_t low = window_low(window, past);
    const uint32_t nsplit = decode_splits((uint64_t)past - low, decode_split_columns(lpr));
    DecodeLaunch L{};
    L.q = q; L.ins_k = ins_k; L.ins_v = ins_v; L.slot_k = slot_k; L.slot_v = slot_v; L.out = out;
    L.args.heads = heads;
    L.args.kv_heads = kv_heads;
    L.args.window = window;
    L.args.past = past;
    L.args.slot_batch_stride = (uint64_t)kv_heads * capacity * depth;
    L.args.slot_plane_stride = (uint64_t)capacity * depth;
    L.args.scale = half_scale;
    L.args.nseq = batch;
    L.grid_x = nsplit;
    L.grid_z = batch;
    L.args.tickets = tickets ? tickets : ctx->tickets;
    L.ticket_slots = tickets ? ticket_slots : kTicketSlots;
    L.clear_tickets = tickets != nullptr;
    L.args.lengths = ptr<uint32_t>(lengths);
    L.args.capacity = capacity;
    if (nsplit > 1) {
      // split partials + arrival counters: the context's counters assume launch order
      if (!tickets) KRM_TRY(needs_serial_scratch(ctx, "the split decode attention"));
      const size_t ml_floats = (size_t)batch * nsplit * heads * 2;
      const size_t need = (ml_floats + (size_t)batch * nsplit * heads * depth) * sizeof(float);
      if (tickets && workspace_bytes < need + 16)
        return fail(ctx, KRM_ERR_VALIDATION,
                    "krm_attention_state_noalloc: this call needs %zu bytes of split partials, the "
                    "built-in scratch holds %zu (use krm_attention_state with a workspace)",
                    need + 16, workspace_bytes);
      KRM_REQUIRE(ctx, workspace && aligned(workspace, 16) && workspace_bytes >= need,
                  "krm_attention_state: workspace of %zu bytes, %zu needed", workspace_bytes,
                  need);
      L.ws_ml = ptr<float>(workspace);
      L.ws_acc = L.ws_ml + ((ml_floats + 3) & ~(size_t)3);
      KRM_REQUIRE(ctx, workspace_bytes >= (size_t)((char*)(L.ws_acc + (size_t)batch * nsplit *
                                                           heads * depth) - (char*)L.ws_ml),
                  "krm_attention_state: workspace of %zu bytes is too small", workspace_bytes);
    }
    return decode_dispatch<false>(ctx, L, repeat, lpr, io_dtype, kv_dtype);
  }

  GenericArgs a{heads, kv_heads, chunk_rows, depth, capacity, window, past, query, half_scale,
                ptr<uint32_t>(lengths)};
  // chunks of rows with the usual head dims: the MFMA form
  if ((chunk_rows > 1 || chunk_only) && (depth == 64 || depth == 128 || depth == 256) &&
      aligned(q, 16) &&
      aligned(ins_k, 16) && aligned(ins_v, 16) && aligned(slot_k, 16) && aligned(slot_v, 16) &&
      (uint64_t)batch * heads <= 0x7fffffffull && (chunk_rows + 31) / 32 <= 65535) {
    const uint32_t f = chunk_flags;
    if (io_dtype == KRM_F32 && kv_dtype == KRM_F32)
      return launch_rows<float, float>(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, a, f);
    if (io_dtype == KRM_F16 && kv_dtype == KRM_F16)
      return launch_rows<__half, __half>(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, a, f);
    if (io_dtype == KRM_F32 && kv_dtype == KRM_F16)
      return launch_rows<float, __half>(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, a, f);
    return launch_rows<__half, float>(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, a, f);
  }
  if (chunk_only)
    return fail(ctx, KRM_ERR_VALIDATION,
                "krm_attention_chunk: covers D = 64, 128 or 256 and 16-byte aligned buffers (D = %u); "
                "use krm_attention_state, krm_state_append and krm_transpose_01", depth);
  if (io_dtype == KRM_F32 && kv_dtype == KRM_F32)
    return launch_generic<float, float>(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, a);
  if (io_dtype == KRM_F16 && kv_dtype == KRM_F16)
    return launch_generic<__half, __half>(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, a);
  if (io_dtype == KRM_F32 && kv_dtype == KRM_F16)
    return launch_generic<float, __half>(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, a);
  return launch_generic<__half, float>(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, a);
}

int32_t krm_attention_state(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                            krm_buf slot_k, krm_buf slot_v, krm_buf out, uint32_t batch,
                            uint32_t heads, uint32_t kv_heads, uint32_t chunk_rows,
                            uint32_t depth, uint32_t capacity, uint32_t window,
                            float half_scale, uint32_t past, uint32_t query, int32_t io_dtype,
                            int32_t kv_dtype, krm_buf workspace, size_t workspace_bytes) {
  return attention_state_impl(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, heads, kv_heads,
                              chunk_rows, depth, capacity, window, half_scale, past, query, 0,
                              io_dtype, kv_dtype, workspace, workspace_bytes);
}

int32_t krm_attention_state_lengths(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                                    krm_buf slot_k, krm_buf slot_v, krm_buf out, uint32_t batch,
                                    uint32_t heads, uint32_t kv_heads, uint32_t chunk_rows,
                                    uint32_t depth, uint32_t capacity, uint32_t window,
                                    float half_scale, krm_buf lengths, uint32_t max_past,
                                    int32_t io_dtype, int32_t kv_dtype, krm_buf workspace,
                                    size_t workspace_bytes) {
  if (!lengths) return fail(ctx, KRM_ERR_VALIDATION, "krm_attention_state_lengths: NULL lengths");
  return attention_state_impl(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, heads, kv_heads,
                              chunk_rows, depth, capacity, window, half_scale, max_past,
                              chunk_rows, lengths, io_dtype, kv_dtype, workspace, workspace_bytes);
}

int32_t krm_attention_chunk(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v, krm_buf slot_k,
                            krm_buf slot_v, krm_buf out, uint32_t batch, uint32_t heads,
                            uint32_t kv_heads, uint32_t chunk_rows, uint32_t depth,
                            uint32_t capacity, uint32_t window, float half_scale, uint32_t past,
                            uint32_t query, krm_buf lengths, int32_t io_dtype, int32_t kv_dtype,
                            uint32_t flags) {
  KRM_REQUIRE(ctx, (flags & ~(uint32_t)(KRM_CHUNK_OUT_ROW_MAJOR | KRM_CHUNK_APPEND |
                                        KRM_CHUNK_OUT_F16)) == 0,
              "krm_attention_chunk: unknown flags 0x%x", flags);
  KRM_REQUIRE(ctx, !(flags & KRM_CHUNK_APPEND) || window == 0,
              "krm_attention_chunk: the fused append needs window == 0 (a ring overwrites rows "
              "this launch still reads); call krm_state_append after the attention");
  return attention_state_impl(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, heads, kv_heads,
                              chunk_rows, depth, capacity, window, half_scale,
                              lengths ? capacity - 1 : past, lengths ? chunk_rows : query, lengths,
                              io_dtype, kv_dtype, 0, 0, nullptr, 0, flags, true);
}

int32_t krm_attention_varlen_workspace(uint32_t nseq, uint32_t heads, uint32_t kv_heads,
                                       uint32_t depth, uint64_t total_rows, size_t* bytes) {
  (void)kv_heads;
  if (!bytes) return fail(nullptr, KRM_ERR_VALIDATION, "krm_attention_varlen_workspace: NULL");
  const uint32_t sc = min_split_columns(depth);
  // every sequence rounds its split count up, so at most total/sc + nseq splits
  const uint64_t splits = sc ? total_rows / sc + nseq : nseq;
  *bytes = 2 * ((size_t)nseq + 1) * sizeof(int32_t) + 64 +
           (size_t)splits * heads * ((size_t)depth + 2) * sizeof(float) + 256;
  return KRM_OK;
}

int32_t krm_attention_varlen(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                             krm_buf slot_k, krm_buf slot_v, krm_buf out,
                             const int32_t* cu_seqlens, uint32_t nseq, uint32_t heads,
                             uint32_t kv_heads, uint32_t depth, uint64_t total_rows,
                             float half_scale, int32_t io_dtype, int32_t kv_dtype,
                             krm_buf workspace, size_t workspace_bytes) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(kv_dtype),
              "krm_attention_varlen: io_dtype %d / kv_dtype %d", io_dtype, kv_dtype);
  KRM_REQUIRE(ctx, nseq >= 1 && heads >= 1 && kv_heads >= 1 && depth >= 1,
              "krm_attention_varlen: nseq / H / Hkv / D must be positive");
  KRM_REQUIRE(ctx, heads % kv_heads == 0, "krm_attention_varlen: H = %u is not a multiple of Hkv = %u",
              heads, kv_heads);
  KRM_REQUIRE(ctx, std::isfinite(half_scale), "krm_attention_varlen: scale is not finite");
  KRM_REQUIRE(ctx, cu_seqlens != nullptr, "krm_attention_varlen: cu_seqlens is NULL");
  KRM_REQUIRE(ctx, total_rows <= 0x7fffffffull, "krm_attention_varlen: total_rows too large");
  KRM_REQUIRE(ctx, heads <= 65535 && (uint64_t)nseq * heads <= kTicketSlots,
              "krm_attention_varlen: nseq * H = %llu exceeds %u", (unsigned long long)nseq * heads,
              kTicketSlots);
  const uint32_t repeat = heads / kv_heads;
  const uint32_t lpr = decode_lanes_per_row(depth, kv_dtype);
  KRM_REQUIRE(ctx, lpr && decode_repeat_ok(repeat),
              "krm_attention_varlen: D = %u with this slot dtype or H/Hkv = %u is not covered "
              "by the split-K decode kernel",
              depth, repeat);
  KRM_REQUIRE(ctx, q && ins_k && ins_v && slot_k && slot_v && out && workspace,
              "krm_attention_varlen: NULL buffer");
  KRM_REQUIRE(ctx, aligned(slot_k, 16) && aligned(slot_v, 16) && aligned(workspace, 16) &&
                       aligned(q, 16),
              "krm_attention_varlen: q, slots and workspace must be 16-byte aligned");
  KRM_REQUIRE(ctx, cu_seqlens[0] >= 0, "krm_attention_varlen: cu_seqlens[0] is negative");

  // Host-side tables: slot row offsets and the first global split of each sequence.
  const size_t table_ints = 2 * ((size_t)nseq + 1);
  KRM_REQUIRE(ctx, table_ints * sizeof(int32_t) <= ctx->pinned_bytes,
              "krm_attention_varlen: %u sequences exceed the staging table", nseq);
  KRM_TRY(not_recording(ctx, "krm_attention_varlen"));
  // The staging area may still feed the previous call's copy.
  KRM_TRY(hip_status(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"));
  int32_t* stage = static_cast<int32_t*>(ctx->pinned);
  int32_t* cu = stage;
  int32_t* prefix = stage + nseq + 1;
  const uint32_t sc = decode_split_columns(lpr);
  uint64_t splits = 0;
  for (uint32_t i = 0; i <= nseq; ++i) {
    cu[i] = cu_seqlens[i];
    if (i > 0) {
      KRM_REQUIRE(ctx, cu_seqlens[i] >= cu_seqlens[i - 1],
                  "krm_attention_varlen: cu_seqlens is not ascending at %u", i);
      prefix[i - 1] = (int32_t)splits;
      const uint32_t ns = decode_splits((uint64_t)(cu_seqlens[i] - cu_seqlens[i - 1]), sc);
      splits += ns;
    }
  }
  prefix[nseq] = (int32_t)splits;
  KRM_REQUIRE(ctx, (uint64_t)cu_seqlens[nseq] <= total_rows,
              "krm_attention_varlen: cu_seqlens[%u] = %d exceeds total_rows %llu", nseq,
              cu_seqlens[nseq], (unsigned long long)total_rows);
  KRM_REQUIRE(ctx, splits <= 0x7fffffffull, "krm_attention_varlen: too many splits");

  const size_t table_bytes = (table_ints * sizeof(int32_t) + 63) & ~(size_t)63;
  const size_t ml_floats = ((size_t)splits * heads * 2 + 3) & ~(size_t)3;
  const size_t need = table_bytes + (ml_floats + (size_t)splits * heads * depth) * sizeof(float);
  KRM_REQUIRE(ctx, workspace_bytes >= need, "krm_attention_varlen: workspace of %zu bytes, %zu needed",
              workspace_bytes, need);
  KRM_TRY(hip_status(ctx,
                     hipMemcpyAsync(ptr<void>(workspace), stage, table_ints * sizeof(int32_t),
                                    hipMemcpyHostToDevice, ctx->stream),
                     "hipMemcpyAsync(tables)"));

  DecodeLaunch L{};
  L.q = q; L.ins_k = ins_k; L.ins_v = ins_v; L.slot_k = slot_k; L.slot_v = slot_v; L.out = out;
  L.args.heads = heads;
  L.args.kv_heads = kv_heads;
  L.args.window = 0;
  L.args.past = 0;
  L.args.slot_batch_stride = 0;
  L.args.slot_plane_stride = total_rows * depth;
  L.args.scale = half_scale;
  L.args.nseq = nseq;
  L.args.cu_rows = ptr<const int32_t>(workspace);
  L.args.split_prefix = L.args.cu_rows + nseq + 1;
  L.ws_ml = ptr<float>(workspace + table_bytes);
  L.ws_acc = L.ws_ml + ml_floats;
  L.grid_x = (uint32_t)splits;
  L.grid_z = 1;
  KRM_TRY(needs_serial_scratch(ctx, "krm_attention_varlen"));
  L.args.tickets = ctx->tickets;
  return decode_dispatch<true>(ctx, L, repeat, lpr, io_dtype, kv_dtype);
}

}  // extern "C"

// ---- ragged batch whose tables are built on the device -------------------------------------

// plan layout (int32): cu_rows[nseq + 1], split_prefix[nseq + 1], fault
__global__ void varlen_plan_kernel(const int32_t* __restrict__ cu_seqlens, int32_t* __restrict__ plan,
                                   uint32_t nseq, uint32_t chunk_columns, uint64_t total_rows,
                                   uint32_t max_splits) {
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  int32_t* cu = plan;
  int32_t* prefix = plan + nseq + 1;
  int32_t* fault = plan + 2 * (nseq + 1);
  bool ok = cu_seqlens[0] >= 0;
  uint64_t splits = 0;
  cu[0] = cu_seqlens[0];
  for (uint32_t i = 1; i <= nseq; ++i) {
    const int32_t lo = cu_seqlens[i - 1], hi = cu_seqlens[i];
    cu[i] = hi;
    ok = ok && hi >= lo;
    prefix[i - 1] = (int32_t)splits;
    splits += ok ? decode_splits((uint64_t)(hi - lo), chunk_columns) : 0u;
  }
  ok = ok && (uint64_t)cu_seqlens[nseq] <= total_rows && splits <= max_splits;
  prefix[nseq] = (int32_t)splits;
  if (!ok)  // no workgroup of the attention launch finds a split: nothing is read or written
    for (uint32_t i = 0; i <= nseq; ++i) prefix[i] = 0;
  *fault = ok ? 0 : 1;
}

extern "C" {

int32_t krm_attention_varlen_plan_bytes(uint32_t nseq, size_t* bytes) {
  if (!bytes) return fail(nullptr, KRM_ERR_VALIDATION, "krm_attention_varlen_plan_bytes: NULL");
  *bytes = ((2 * ((size_t)nseq + 1) + 1) * sizeof(int32_t) + 63) & ~(size_t)63;
  return KRM_OK;
}

int32_t krm_attention_varlen_max_splits(uint32_t nseq, uint32_t depth, int32_t kv_dtype,
                                        uint64_t total_rows, uint32_t* max_splits) {
  if (!max_splits) return fail(nullptr, KRM_ERR_VALIDATION, "krm_attention_varlen_max_splits: NULL");
  if (!valid_dtype(kv_dtype))
    return fail(nullptr, KRM_ERR_VALIDATION, "krm_attention_varlen_max_splits: kv_dtype %d", kv_dtype);
  const uint32_t lpr = decode_lanes_per_row(depth, kv_dtype);
  if (!lpr)
    return fail(nullptr, KRM_ERR_VALIDATION,
                "krm_attention_varlen_max_splits: D = %u is not covered by the decode kernel", depth);
  // every sequence rounds its split count up
  const uint64_t splits = total_rows / decode_split_columns(lpr) + nseq;
  if (splits > 0x7fffffffull)
    return fail(nullptr, KRM_ERR_VALIDATION, "krm_attention_varlen_max_splits: too many splits");
  *max_splits = (uint32_t)splits;
  return KRM_OK;
}

int32_t krm_attention_varlen_plan(krm_ctx* ctx, krm_buf cu_seqlens_i32, krm_buf plan,
                                  uint32_t nseq, uint32_t depth, int32_t kv_dtype,
                                  uint64_t total_rows, uint32_t max_splits) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(kv_dtype), "krm_attention_varlen_plan: kv_dtype %d", kv_dtype);
  KRM_REQUIRE(ctx, nseq >= 1 && total_rows <= 0x7fffffffull,
              "krm_attention_varlen_plan: nseq must be positive and total_rows < 2^31");
  const uint32_t lpr = decode_lanes_per_row(depth, kv_dtype);
  KRM_REQUIRE(ctx, lpr, "krm_attention_varlen_plan: D = %u with this slot dtype is not covered",
              depth);
  KRM_REQUIRE(ctx, cu_seqlens_i32 && plan && aligned(cu_seqlens_i32, 4) && aligned(plan, 4),
              "krm_attention_varlen_plan: NULL or misaligned buffer");
  varlen_plan_kernel<<<dim3(1), dim3(64), 0, ctx->stream>>>(
      ptr<const int32_t>(cu_seqlens_i32), ptr<int32_t>(plan), nseq, decode_split_columns(lpr),
      total_rows, max_splits);
  return launched(ctx, "varlen_plan_kernel");
}

int32_t krm_attention_varlen_planned(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                                     krm_buf slot_k, krm_buf slot_v, krm_buf out, krm_buf plan,
                                     uint32_t nseq, uint32_t heads, uint32_t kv_heads,
                                     uint32_t depth, uint64_t total_rows, uint32_t max_splits,
                                     float half_scale, int32_t io_dtype, int32_t kv_dtype,
                                     krm_buf workspace, size_t workspace_bytes) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, valid_dtype(io_dtype) && valid_dtype(kv_dtype),
              "krm_attention_varlen_planned: io_dtype %d / kv_dtype %d", io_dtype, kv_dtype);
  KRM_REQUIRE(ctx, nseq >= 1 && heads >= 1 && kv_heads >= 1 && depth >= 1 && max_splits >= 1,
              "krm_attention_varlen_planned: nseq / H / Hkv / D / max_splits must be positive");
  KRM_REQUIRE(ctx, heads % kv_heads == 0,
              "krm_attention_varlen_planned: H = %u is not a multiple of Hkv = %u", heads, kv_heads);
  KRM_REQUIRE(ctx, std::isfinite(half_scale), "krm_attention_varlen_planned: scale is not finite");
  KRM_REQUIRE(ctx, total_rows <= 0x7fffffffull && max_splits <= 0x7fffffffu,
              "krm_attention_varlen_planned: total_rows or max_splits too large");
  KRM_REQUIRE(ctx, heads <= 65535 && (uint64_t)nseq * heads <= kTicketSlots,
              "krm_attention_varlen_planned: nseq * H = %llu exceeds %u",
              (unsigned long long)nseq * heads, kTicketSlots);
  const uint32_t repeat = heads / kv_heads;
  const uint32_t lpr = decode_lanes_per_row(depth, kv_dtype);
  KRM_REQUIRE(ctx, lpr && decode_repeat_ok(repeat),
              "krm_attention_varlen_planned: D = %u with this slot dtype or H/Hkv = %u is not "
              "covered by the split-K decode kernel", depth, repeat);
  KRM_REQUIRE(ctx, q && ins_k && ins_v && slot_k && slot_v && out && workspace && plan,
              "krm_attention_varlen_planned: NULL buffer");
  KRM_REQUIRE(ctx, aligned(slot_k, 16) && aligned(slot_v, 16) && aligned(workspace, 16) &&
                       aligned(q, 16) && aligned(plan, 4),
              "krm_attention_varlen_planned: q, slots and workspace must be 16-byte aligned");
  const size_t ml_floats = ((size_t)max_splits * heads * 2 + 3) & ~(size_t)3;
  const size_t need = (ml_floats + (size_t)max_splits * heads * depth) * sizeof(float);
  KRM_REQUIRE(ctx, workspace_bytes >= need,
              "krm_attention_varlen_planned: workspace of %zu bytes, %zu needed", workspace_bytes,
              need);
  DecodeLaunch L{};
  L.q = q; L.ins_k = ins_k; L.ins_v = ins_v; L.slot_k = slot_k; L.slot_v = slot_v; L.out = out;
  L.args.heads = heads;
  L.args.kv_heads = kv_heads;
  L.args.window = 0;
  L.args.past = 0;
  L.args.slot_batch_stride = 0;
  L.args.slot_plane_stride = total_rows * depth;
  L.args.scale = half_scale;
  L.args.nseq = nseq;
  L.args.cu_rows = ptr<const int32_t>(plan);
  L.args.split_prefix = L.args.cu_rows + nseq + 1;
  L.ws_ml = ptr<float>(workspace);
  L.ws_acc = L.ws_ml + ml_floats;
  L.grid_x = max_splits;
  L.grid_z = 1;
  KRM_TRY(needs_serial_scratch(ctx, "krm_attention_varlen_planned"));
  L.args.tickets = ctx->tickets;
  return decode_dispatch<true>(ctx, L, repeat, lpr, io_dtype, kv_dtype);
}

}  // extern "C"
// ---- the decode attention for callers that cannot allocate ----------------------------------
//
// Split partials and arrival counters live in one file-scope device array instead of a
// caller-supplied workspace and the context's counters.  Each GPU holds its own copy of the
// array at its own address; the address is looked up once per device and that pointer — never
// the array's name, which in host code is only a stand-in — is what kernels and fills receive.
namespace {

constexpr size_t kStaticTicketSlots = 512;
constexpr size_t kStaticTicketBytes = kStaticTicketSlots * kTicketStride * sizeof(uint32_t);
constexpr size_t kStaticScratchBytes = 4u << 20;  // counters + split partials, per GPU
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

unsigned char* g_scratch_ptr[kMaxDevices] = {};

// Device address of this device's copy of `scratch` (the context's device is current).
int32_t static_scratch(krm_ctx* ctx, unsigned char** out) {
  KRM_REQUIRE(ctx, ctx->device >= 0 && ctx->device < kMaxDevices,
              "krm_attention_state_noalloc: device %d is outside 0..%d", ctx->device,
              kMaxDevices - 1);
  unsigned char* p = __atomic_load_n(&g_scratch_ptr[ctx->device], __ATOMIC_ACQUIRE);
  if (!p) {
    void* address = nullptr;
    KRM_TRY(hip_status(ctx, hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)),
                       "hipGetSymbolAddress(scratch)"));
    KRM_REQUIRE(ctx, address != nullptr, "krm_attention_state_noalloc: scratch has no address");
    p = static_cast<unsigned char*>(address);
    __atomic_store_n(&g_scratch_ptr[ctx->device], p, __ATOMIC_RELEASE);
  }
  *out = p;
  return KRM_OK;
}

}  // namespace

namespace krm {
// Called when a context is created on a device, so that the address is known before any caller
// starts recording a graph (the lookup is a runtime call that does not belong in a capture).
int32_t resolve_static_scratch(krm_ctx* ctx) {
  unsigned char* unused = nullptr;
  return static_scratch(ctx, &unused);
}
}  // namespace krm

extern "C" {

int32_t krm_attention_state_noalloc(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                                    krm_buf slot_k, krm_buf slot_v, krm_buf out, uint32_t batch,
                                    uint32_t heads, uint32_t kv_heads, uint32_t chunk_rows,
                                    uint32_t depth, uint32_t capacity, uint32_t window,
                                    float half_scale, uint32_t past, uint32_t query,
                                    int32_t io_dtype, int32_t kv_dtype) {
  KRM_TRY(enter(ctx));
  unsigned char* base = nullptr;
  KRM_TRY(static_scratch(ctx, &base));
  // Only the split decode form needs scratch; it checks its partials against `room` and words
  // the error for this entry.  Chunks of rows and head dims the decode form does not cover run
  // without any, and a call with more heads than the array has counters takes the generic
  // kernel.
  const size_t room = kStaticScratchBytes - kStaticTicketBytes;
  return attention_state_impl(ctx, q, ins_k, ins_v, slot_k, slot_v, out, batch, heads, kv_heads,
                              chunk_rows, depth, capacity, window, half_scale, past, query, 0,
                              io_dtype, kv_dtype,
                              static_cast<krm_buf>(reinterpret_cast<uintptr_t>(
                                  base + kStaticTicketBytes)),
                              room, reinterpret_cast<uint32_t*>(base),
                              (uint32_t)kStaticTicketSlots);
}

}  // extern "C"
