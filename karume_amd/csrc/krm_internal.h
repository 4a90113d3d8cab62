// Internal declarations shared by the translation units of libkarume_hip.so (gfx950 only).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "../../include/karume_hip.h"

struct krm_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  bool owns_stream = false;
  int num_cus = 256;
  // Host staging for small per-call tables (pinned, allocated once at context creation).
  void* pinned = nullptr;
  size_t pinned_bytes = 0;
  // Arrival counters of the split-K attention (device memory, zeroed at creation; the last
  // workgroup of every (sequence, kv head) puts its counter back to zero).
  uint32_t* tickets = nullptr;
  // Scratch of the unit-dealt GEMM: two 128 x 256 f32 partials per CU (64 MiB on 256 CUs),
  // allocated with the context so that launches can be recorded into graphs.
  float* gemm_partials = nullptr;
  // Per-row scales {2^e, 2^-e} of the f32-class prefill GEMM (kMaxSplitRows rows), written by
  // a pre-pass of every such launch.
  float* row_scales = nullptr;
  bool recording = false;  // between krm_graph_begin and krm_graph_end
  // Parallel branches of a recording (krm_graph_branch): `stream` is the stream launches go
  // to, which is `main_stream` except while a side branch is selected.  Side streams are
  // created on first use (default priority) and live as long as the context.
  hipStream_t main_stream = nullptr;
  static constexpr int kMaxBranches = 4;
  hipStream_t branch_stream[kMaxBranches] = {nullptr, nullptr, nullptr, nullptr};
  hipEvent_t branch_event[kMaxBranches] = {nullptr, nullptr, nullptr, nullptr};
  bool branch_forked[kMaxBranches] = {false, false, false, false};
  char error[512] = {0};
};

struct krm_event {
  hipEvent_t ev;
};

struct krm_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

namespace krm {

constexpr int kWave = 64;
constexpr uint32_t kTicketSlots = 1u << 16;
// Words between two arrival counters: one counter per 128 bytes.  Atomics on one cache line
// execute one after the other (11 ns each, measured); the 512 workgroups of a 4096-column
// decode step, counting on 16 neighbouring words, spent 5.8 us queueing there.
constexpr uint32_t kTicketStride = 32;
constexpr size_t kGemmPartialBytes = 128u * 256u * sizeof(float);
constexpr uint32_t kMaxSplitRows = 1u << 16;

// Records the message on the context (or on the context-less slot) and returns `code`.
int32_t fail(krm_ctx* ctx, int32_t code, const char* fmt, ...);

#if defined(__HIPCC__)
// `v` as the f32 it has been rounded to.  Without this the compiler may fold the product that
// made `v` and a conversion to fp16 that follows into one mixed-precision instruction with a
// single rounding — a different fp16 on ties than the f32 value stored and rounded later.
__device__ inline float rounded_f32(float v) {
  asm volatile("" : "+v"(v));
  return v;
}

// Order of (value, index) pairs for argmax: NaN counts as the maximum, larger values win, ties
// go to the smaller index (packages/runtime/src/kernels/argmax.ts:16-34).  Lexicographic, so
// any tree of pairwise comparisons gives the same winner.
__device__ inline bool argmax_beats(float va, uint32_t ia, float vb, uint32_t ib) {
  const bool na = va != va, nb = vb != vb;
  if (na != nb) return na;
  if (!na && va != vb) return va > vb;
  return ia < ib;
}
#endif

// Maps a HIP runtime status to an error class; 0 when `status` is hipSuccess.
int32_t hip_status(krm_ctx* ctx, hipError_t status, const char* what);

// Makes the context's device current on the calling thread (calls may arrive on any thread).
int32_t enter(krm_ctx* ctx);

// Rejects calls that have to wait for the device while a launch sequence is being recorded.
int32_t not_recording(krm_ctx* ctx, const char* what);

// Error check of the launch that was just queued.
int32_t launched(krm_ctx* ctx, const char* kernel);

// The context's own scratch (arrival counters, GEMM partials, row scales) assumes that the ops
// using it run one after the other, which only the main stream guarantees: ops recorded on a
// side branch of a graph (krm_graph_branch) may run beside the main branch and beside each
// other.  Entry points call this before they hand that scratch to a kernel.
int32_t needs_serial_scratch(krm_ctx* ctx, const char* what);

inline bool valid_dtype(int32_t dtype) { return dtype == KRM_F32 || dtype == KRM_F16; }
inline size_t dtype_bytes(int32_t dtype) { return dtype == KRM_F16 ? 2 : 4; }
inline bool is_pow2(uint32_t v) { return v != 0 && (v & (v - 1)) == 0; }
inline bool aligned(krm_buf address, size_t bytes) { return (address % bytes) == 0; }

template <typename T>
inline T* ptr(krm_buf address) {
  return reinterpret_cast<T*>(static_cast<uintptr_t>(address));
}

// What the few-row MFMA GEMM (gemm_i4.hip) does with a finished sum besides storing it.
struct RowsFusion {
  const void* residual = nullptr;  // [m, n_out] added to the result (the activation type)
  // 0: plain; 1: columns (2i, 2i+1) = (gate_i, up_i), out[., i] = silu(gate) * up;
  // 2: a fused [q; k; v] projection whose q and k columns are interleaved per head as
  //    (0, D/2, 1, D/2 + 1, ...): half-split RoPE by positions[row], results head-major
  int mode = 0;
  const int32_t* positions = nullptr;
  const float* cos_table = nullptr;
  const float* sin_table = nullptr;
  void* q_out = nullptr;  // [H, m, D]
  void* k_out = nullptr;  // [Hkv, m, D]
  void* v_out = nullptr;  // [Hkv, m, D]
  uint32_t heads = 0, kv_heads = 0, depth = 0, table_rows = 0;
};

}  // namespace krm

#define KRM_TRY(expr)                  \
  do {                                 \
    int32_t krm_status_ = (expr);      \
    if (krm_status_ != KRM_OK) return krm_status_; \
  } while (0)

#define KRM_REQUIRE(ctx, cond, ...)                                   \
  do {                                                                \
    if (!(cond)) return krm::fail((ctx), KRM_ERR_VALIDATION, __VA_ARGS__); \
  } while (0)
