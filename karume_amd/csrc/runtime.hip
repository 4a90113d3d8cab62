// Context, buffers, events and error plumbing of libkarume_hip.so.
//
// Replaces, for the ops this library serves, what the reference does through WebGPU:
// acquireGpu / GpuContext (packages/runtime/src/gpu/device.ts), createBuffer +
// queue.writeBuffer + readback (packages/runtime/src/runtime/executor.ts:870-896,1272) and the
// opt-in timestamp diagnostics (packages/runtime/src/gpu/submit.ts:54-63).
#include "krm_internal.h"

namespace {
thread_local char g_error[512] = "";
}

namespace krm {

int32_t fail(krm_ctx* ctx, int32_t code, const char* fmt, ...) {
  char* dst = ctx ? ctx->error : g_error;
  va_list args;
  va_start(args, fmt);
  vsnprintf(dst, 512, fmt, args);
  va_end(args);
  return code;
}

int32_t hip_status(krm_ctx* ctx, hipError_t status, const char* what) {
  if (status == hipSuccess) return KRM_OK;
  const int32_t code =
      status == hipErrorOutOfMemory || status == hipErrorMemoryAllocation
          ? KRM_ERR_OUT_OF_MEMORY
          : (status == hipErrorInvalidValue || status == hipErrorInvalidDevice ||
                     status == hipErrorInvalidDevicePointer
                 ? KRM_ERR_VALIDATION
                 : KRM_ERR_DEVICE_LOST);
  return fail(ctx, code, "%s: %s (%s)", what, hipGetErrorString(status),
              hipGetErrorName(status));
}

int32_t enter(krm_ctx* ctx) {
  if (!ctx) return fail(nullptr, KRM_ERR_VALIDATION, "context is NULL");
  return hip_status(ctx, hipSetDevice(ctx->device), "hipSetDevice");
}

int32_t not_recording(krm_ctx* ctx, const char* what) {
  if (ctx->recording)
    return fail(ctx, KRM_ERR_VALIDATION, "%s cannot be called while a graph is being recorded",
                what);
  return KRM_OK;
}

int32_t launched(krm_ctx* ctx, const char* kernel) {
  return hip_status(ctx, hipGetLastError(), kernel);
}

int32_t needs_serial_scratch(krm_ctx* ctx, const char* what) {
  if (ctx->stream != ctx->main_stream)
    return fail(ctx, KRM_ERR_VALIDATION,
                "%s uses the context's scratch (arrival counters, partial sums or row scales), "
                "which ops share in launch order: record it on the main branch, not on a side "
                "branch of the graph", what);
  return KRM_OK;
}

}  // namespace krm

using namespace krm;

namespace krm {
int32_t resolve_static_scratch(krm_ctx* ctx);  // attention_state.hip
}

// Measurement floors: what a launch of a given grid costs when it does nothing, and when it
// only streams `bytes` with 16-byte loads (every thread folds what it read into one word that
// is stored only if it equals a value the data never has, so the loads stay).
__global__ void krm_probe_empty_kernel() {}

// PER 16-byte loads per thread are requested before any is used (one memory round trip for
// the whole launch when the grid covers `pieces` in one pass); larger buffers take more passes.
template <int PER>
__global__ void krm_probe_read_kernel(const uint4* __restrict__ src, size_t pieces,
                                      uint32_t* __restrict__ sink) {
  const size_t threads = (size_t)gridDim.x * blockDim.x;
  const size_t tid = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  uint32_t fold = 0;
  for (size_t base = 0; base < pieces; base += threads * PER) {
    uint4 v[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const size_t i = base + (size_t)j * threads + tid;  // a wave reads 1 KiB in a row
      v[j] = src[i < pieces ? i : 0];
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) fold |= (v[j].x ^ v[j].y) + (v[j].z ^ v[j].w);
  }
  if (fold == 0x9E3779B9u && sink) sink[0] = fold;
}

// What one all-to-all hand-over of a vector between the workgroups of ONE launch costs — the
// step a persistent decode kernel would pay where today's decode step ends one kernel and
// starts the next.  Every workgroup owns n / grid entries of the vector.  Phase p: wave 0 polls
// the producers' flags (agent-scope 16-byte loads, four flags a lane) until all have reached p,
// loads the vector (agent-scope 16-byte loads, all in flight) into LDS, barrier; the other
// waves compute this workgroup's entries from LDS (a few adds: stand-in work), barrier; wave 0
// stores the entries with agent-scope stores, waits for their acknowledgement and stores its
// flag p + 1.  Vectors are double-buffered by phase parity.  Every wait is bounded: a poll that
// exceeds `spin_limit` rounds raises the fault word and the workgroup leaves.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ inline void probe_load_agent_b128(u32x4_t& v, const void* p) {
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
}
__device__ inline void probe_wait_loads(u32x4_t& a) {
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(a)::"memory");  // ties the register to the wait
}

template <int N>
__global__ __launch_bounds__(576) void krm_probe_exchange_kernel(float* vec, uint32_t* flags,
                                                                 uint32_t* fault, uint32_t phases,
                                                                 uint32_t spin_limit) {
  __shared__ __attribute__((aligned(16))) float s_x[N];
  __shared__ float s_out[64];
  __shared__ int s_ok;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t nwg = gridDim.x;
  const uint32_t per_wg = N / nwg;
  constexpr int kPieces = N / 4, kPerLane = (kPieces + 63) / 64;
  if (threadIdx.x == 0) s_ok = 1;
  __syncthreads();
  for (uint32_t p = 0; p < phases; ++p) {
    float* cur = vec + (size_t)(p & 1) * N;
    float* nxt = vec + (size_t)((p + 1) & 1) * N;
    if (wave == 0) {
      bool ok = true;
      if (p > 0) {
        uint32_t spins = 0;
        while (true) {
          u32x4_t f;
          probe_load_agent_b128(f, flags + ((uint32_t)lane * 4 < nwg ? lane * 4 : 0));
          probe_wait_loads(f);
          const bool mine = (uint32_t)lane * 4 >= nwg ||
                            (f.x >= p && f.y >= p && f.z >= p && f.w >= p);
          if (__all(mine)) break;
          if (++spins > spin_limit) { ok = false; break; }
        }
      }
      if (!ok && lane == 0) { *fault = 1u; s_ok = 0; }
      u32x4_t v[kPerLane];
#pragma unroll
      for (int j = 0; j < kPerLane; ++j) {
        const int piece = j * 64 + lane;
        probe_load_agent_b128(v[j], cur + 4 * (piece < kPieces ? piece : 0));
      }
#pragma unroll
      for (int j = 0; j < kPerLane; ++j) probe_wait_loads(v[j]);
#pragma unroll
      for (int j = 0; j < kPerLane; ++j) {
        const int piece = j * 64 + lane;
        if (piece < kPieces)
          *reinterpret_cast<float4*>(&s_x[4 * piece]) =
              p > 0 ? make_float4(__uint_as_float(v[j].x), __uint_as_float(v[j].y),
                                  __uint_as_float(v[j].z), __uint_as_float(v[j].w))
                    : make_float4(1.f, 1.f, 1.f, 1.f);
      }
    }
    __syncthreads();
    if (!s_ok) break;
    if (wave > 0) {
      const uint32_t t = threadIdx.x - 64;
      if (t < per_wg) {
        float sum = 0.f;
        for (int j = 0; j < 8; ++j) sum += s_x[(t * 37 + j * 101 + blockIdx.x) % N];
        s_out[t] = sum * 0.125f;
      }
    }
    __syncthreads();
    if (wave == 0) {
      if ((uint32_t)lane < per_wg)
        __hip_atomic_store(&nxt[blockIdx.x * per_wg + lane], s_out[lane], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_s_waitcnt(0);  // the stores are acknowledged
      if (lane == 0)
        __hip_atomic_store(&flags[blockIdx.x], p + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

extern "C" {

const char* krm_version(void) { return "karume-hip 0.1 gfx950"; }

int32_t krm_ctx_create_on_stream(int32_t device, void* hip_stream, krm_ctx** out) {
  if (!out) return fail(nullptr, KRM_ERR_VALIDATION, "krm_ctx_create: out is NULL");
  *out = nullptr;
  int count = 0;
  KRM_TRY(hip_status(nullptr, hipGetDeviceCount(&count), "hipGetDeviceCount"));
  if (device < 0 || device >= count)
    return fail(nullptr, KRM_ERR_VALIDATION, "krm_ctx_create: device %d of %d", device, count);
  KRM_TRY(hip_status(nullptr, hipSetDevice(device), "hipSetDevice"));
  hipDeviceProp_t prop;
  KRM_TRY(hip_status(nullptr, hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties"));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(nullptr, KRM_ERR_VALIDATION,
                "krm_ctx_create: device %d is %s; this library only carries gfx950 code", device,
                prop.gcnArchName);
  krm_ctx* ctx = new krm_ctx();
  ctx->device = device;
  ctx->num_cus = prop.multiProcessorCount;
  ctx->stream = static_cast<hipStream_t>(hip_stream);
  ctx->main_stream = ctx->stream;
  ctx->owns_stream = false;
  ctx->pinned_bytes = 1 << 20;
  hipError_t st = hipHostMalloc(&ctx->pinned, ctx->pinned_bytes, hipHostMallocDefault);
  if (st != hipSuccess) {
    delete ctx;
    return hip_status(nullptr, st, "hipHostMalloc");
  }
  const size_t ticket_bytes = (size_t)kTicketSlots * kTicketStride * sizeof(uint32_t);
  st = hipMalloc(reinterpret_cast<void**>(&ctx->tickets), ticket_bytes);
  if (st == hipSuccess) st = hipMemset(ctx->tickets, 0, ticket_bytes);
  if (st == hipSuccess)
    st = hipMalloc(reinterpret_cast<void**>(&ctx->gemm_partials),
                   (size_t)2 * ctx->num_cus * kGemmPartialBytes);
  if (st == hipSuccess)
    st = hipMalloc(reinterpret_cast<void**>(&ctx->row_scales),
                   (size_t)kMaxSplitRows * 2 * sizeof(float));
  if (st == hipSuccess) st = hipDeviceSynchronize();
  if (st != hipSuccess) {
    if (ctx->row_scales) (void)hipFree(ctx->row_scales);
    if (ctx->gemm_partials) (void)hipFree(ctx->gemm_partials);
    if (ctx->tickets) (void)hipFree(ctx->tickets);
    (void)hipHostFree(ctx->pinned);
    delete ctx;
    return hip_status(nullptr, st, "hipMalloc(tickets)");
  }
  // The device address of the built-in scratch of krm_attention_state_noalloc is looked up now,
  // with this device current, so that the entry's first call may already sit inside a graph
  // recording.  A failure here is not fatal: the entry repeats the lookup and reports it.
  if (resolve_static_scratch(ctx) != KRM_OK) ctx->error[0] = 0;
  *out = ctx;
  return KRM_OK;
}

int32_t krm_ctx_create(int32_t device, krm_ctx** out) {
  KRM_TRY(krm_ctx_create_on_stream(device, nullptr, out));
  krm_ctx* ctx = *out;
  // Default priority on purpose: mixed stream priorities are not used anywhere.
  hipError_t st = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
  if (st != hipSuccess) {
    (void)hipFree(ctx->row_scales);
    (void)hipFree(ctx->gemm_partials);
    (void)hipFree(ctx->tickets);
    (void)hipHostFree(ctx->pinned);
    delete ctx;
    *out = nullptr;
    return hip_status(nullptr, st, "hipStreamCreateWithFlags");
  }
  ctx->main_stream = ctx->stream;
  ctx->owns_stream = true;
  return KRM_OK;
}

int32_t krm_ctx_destroy(krm_ctx* ctx) {
  if (!ctx) return KRM_OK;
  (void)hipSetDevice(ctx->device);
  ctx->stream = ctx->main_stream;
  (void)hipStreamSynchronize(ctx->stream);
  for (int i = 1; i < krm_ctx::kMaxBranches; ++i) {
    if (ctx->branch_stream[i]) (void)hipStreamDestroy(ctx->branch_stream[i]);
    if (ctx->branch_event[i]) (void)hipEventDestroy(ctx->branch_event[i]);
  }
  if (ctx->branch_event[0]) (void)hipEventDestroy(ctx->branch_event[0]);
  if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
  if (ctx->pinned) (void)hipHostFree(ctx->pinned);
  if (ctx->tickets) (void)hipFree(ctx->tickets);
  if (ctx->gemm_partials) (void)hipFree(ctx->gemm_partials);
  if (ctx->row_scales) (void)hipFree(ctx->row_scales);
  delete ctx;
  return KRM_OK;
}

const char* krm_last_error(krm_ctx* ctx) { return ctx ? ctx->error : g_error; }

int32_t krm_sync(krm_ctx* ctx) {
  KRM_TRY(enter(ctx));
  KRM_TRY(not_recording(ctx, "krm_sync"));
  return hip_status(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

int32_t krm_buf_alloc(krm_ctx* ctx, size_t bytes, krm_buf* out) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, out != nullptr, "krm_buf_alloc: out is NULL");
  void* p = nullptr;
  // A zero-byte request still returns a distinct, freeable address.
  KRM_TRY(hip_status(ctx, hipMalloc(&p, bytes ? bytes : 16), "hipMalloc"));
  *out = static_cast<krm_buf>(reinterpret_cast<uintptr_t>(p));
  return KRM_OK;
}

int32_t krm_buf_free(krm_ctx* ctx, krm_buf buf) {
  KRM_TRY(enter(ctx));
  if (!buf) return KRM_OK;
  KRM_TRY(not_recording(ctx, "krm_buf_free"));
  // Work queued on the stream may still use the buffer ("flush before destroy").
  KRM_TRY(hip_status(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"));
  return hip_status(ctx, hipFree(ptr<void>(buf)), "hipFree");
}

int32_t krm_buf_upload(krm_ctx* ctx, krm_buf dst, size_t dst_offset, const void* host,
                       size_t bytes) {
  KRM_TRY(enter(ctx));
  KRM_TRY(not_recording(ctx, "krm_buf_upload"));
  if (bytes == 0) return KRM_OK;
  KRM_REQUIRE(ctx, dst != 0 && host != nullptr, "krm_buf_upload: NULL buffer");
  // The host array is only valid during the call, so the copy completes before returning.
  KRM_TRY(hip_status(ctx,
                     hipMemcpyAsync(ptr<char>(dst) + dst_offset, host, bytes,
                                    hipMemcpyHostToDevice, ctx->stream),
                     "hipMemcpyAsync(H2D)"));
  return hip_status(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

int32_t krm_buf_download(krm_ctx* ctx, krm_buf src, size_t src_offset, void* host,
                         size_t bytes) {
  KRM_TRY(enter(ctx));
  KRM_TRY(not_recording(ctx, "krm_buf_download"));
  if (bytes == 0) return hip_status(ctx, hipStreamSynchronize(ctx->stream), "sync");
  KRM_REQUIRE(ctx, src != 0 && host != nullptr, "krm_buf_download: NULL buffer");
  KRM_TRY(hip_status(ctx,
                     hipMemcpyAsync(host, ptr<char>(src) + src_offset, bytes,
                                    hipMemcpyDeviceToHost, ctx->stream),
                     "hipMemcpyAsync(D2H)"));
  return hip_status(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

__global__ void krm_zero_kernel(uint32_t* __restrict__ dst, size_t words) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < words; i += stride) dst[i] = 0u;
}

int32_t krm_buf_zero(krm_ctx* ctx, krm_buf dst, size_t dst_offset, size_t bytes) {
  KRM_TRY(enter(ctx));
  if (bytes == 0) return KRM_OK;
  KRM_REQUIRE(ctx, dst != 0, "krm_buf_zero: NULL buffer");
  KRM_REQUIRE(ctx, (dst + dst_offset) % 4 == 0 && bytes % 4 == 0,
              "krm_buf_zero: address and size must be multiples of 4 bytes");
  // A fill kernel rather than a memset node, so the call stays safe under graph capture.
  const size_t words = bytes / 4;
  size_t blocks = (words + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  krm_zero_kernel<<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(
      ptr<uint32_t>(dst + dst_offset), words);
  return launched(ctx, "krm_zero_kernel");
}

__global__ void krm_copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                size_t pieces) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < pieces; i += stride) dst[i] = src[i];
}

int32_t krm_buf_copy(krm_ctx* ctx, krm_buf dst, krm_buf src, size_t bytes) {
  KRM_TRY(enter(ctx));
  if (bytes == 0) return KRM_OK;
  KRM_REQUIRE(ctx, dst && src, "krm_buf_copy: NULL buffer");
  KRM_REQUIRE(ctx, dst % 16 == 0 && src % 16 == 0 && bytes % 16 == 0,
              "krm_buf_copy: addresses and size must be multiples of 16 bytes");
  const size_t pieces = bytes / 16;
  size_t blocks = (pieces + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  krm_copy_kernel<<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(
      ptr<uint4>(dst), ptr<const uint4>(src), pieces);
  return launched(ctx, "krm_copy_kernel");
}

int32_t krm_graph_begin(krm_ctx* ctx) {
  KRM_TRY(enter(ctx));
  KRM_TRY(not_recording(ctx, "krm_graph_begin"));
  KRM_TRY(hip_status(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal),
                     "hipStreamBeginCapture"));
  ctx->recording = true;
  return KRM_OK;
}

int32_t krm_graph_branch(krm_ctx* ctx, uint32_t branch) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, ctx->recording, "krm_graph_branch: no recording in progress");
  KRM_REQUIRE(ctx, branch < (uint32_t)krm_ctx::kMaxBranches, "krm_graph_branch: branch %u of %d",
              branch, krm_ctx::kMaxBranches);
  if (branch == 0) {
    ctx->stream = ctx->main_stream;
    return KRM_OK;
  }
  if (!ctx->branch_stream[branch]) {
    // default priority, like every stream of this library
    KRM_TRY(hip_status(ctx, hipStreamCreateWithFlags(&ctx->branch_stream[branch],
                                                     hipStreamNonBlocking),
                       "hipStreamCreateWithFlags(branch)"));
    KRM_TRY(hip_status(ctx, hipEventCreateWithFlags(&ctx->branch_event[branch],
                                                    hipEventDisableTiming),
                       "hipEventCreate(branch)"));
  }
  if (!ctx->branch_event[0])
    KRM_TRY(hip_status(ctx, hipEventCreateWithFlags(&ctx->branch_event[0], hipEventDisableTiming),
                       "hipEventCreate(fork)"));
  if (!ctx->branch_forked[branch]) {
    // fork: the side stream joins the capture behind what the main branch holds so far
    KRM_TRY(hip_status(ctx, hipEventRecord(ctx->branch_event[0], ctx->main_stream),
                       "hipEventRecord(fork)"));
    KRM_TRY(hip_status(ctx, hipStreamWaitEvent(ctx->branch_stream[branch], ctx->branch_event[0], 0),
                       "hipStreamWaitEvent(fork)"));
    ctx->branch_forked[branch] = true;
  }
  ctx->stream = ctx->branch_stream[branch];
  return KRM_OK;
}

int32_t krm_graph_end(krm_ctx* ctx, krm_graph** out) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, out != nullptr, "krm_graph_end: out is NULL");
  KRM_REQUIRE(ctx, ctx->recording, "krm_graph_end: no recording in progress");
  ctx->recording = false;
  ctx->stream = ctx->main_stream;
  hipError_t st = hipSuccess;
  // join: the main branch waits for every side branch before the recording closes
  for (int i = 1; i < krm_ctx::kMaxBranches; ++i) {
    if (!ctx->branch_forked[i]) continue;
    ctx->branch_forked[i] = false;
    if (st == hipSuccess) st = hipEventRecord(ctx->branch_event[i], ctx->branch_stream[i]);
    if (st == hipSuccess) st = hipStreamWaitEvent(ctx->main_stream, ctx->branch_event[i], 0);
  }
  krm_graph* g = new krm_graph();
  hipError_t end = hipStreamEndCapture(ctx->main_stream, &g->graph);
  if (st == hipSuccess) st = end;
  if (st == hipSuccess) st = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
  if (st != hipSuccess) {
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
    return hip_status(ctx, st, "hipStreamEndCapture/hipGraphInstantiate");
  }
  *out = g;
  return KRM_OK;
}

int32_t krm_graph_launch(krm_ctx* ctx, krm_graph* graph) {
  KRM_TRY(enter(ctx));
  KRM_TRY(not_recording(ctx, "krm_graph_launch"));
  KRM_REQUIRE(ctx, graph && graph->exec, "krm_graph_launch: graph is NULL");
  return hip_status(ctx, hipGraphLaunch(graph->exec, ctx->stream), "hipGraphLaunch");
}

int32_t krm_graph_destroy(krm_ctx* ctx, krm_graph* graph) {
  KRM_TRY(enter(ctx));
  if (!graph) return KRM_OK;
  (void)hipStreamSynchronize(ctx->stream);
  if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
  if (graph->graph) (void)hipGraphDestroy(graph->graph);
  delete graph;
  return KRM_OK;
}

int32_t krm_probe_launch(krm_ctx* ctx, int32_t kind, krm_buf src, size_t bytes, uint32_t grid,
                         uint32_t block) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, kind == KRM_PROBE_EMPTY || kind == KRM_PROBE_READ, "krm_probe_launch: kind %d",
              kind);
  KRM_REQUIRE(ctx, grid >= 1 && grid <= 0x7fffffffu && block >= 64 && block <= 1024 &&
                       block % 64 == 0,
              "krm_probe_launch: grid %u x block %u", grid, block);
  if (kind == KRM_PROBE_EMPTY) {
    krm_probe_empty_kernel<<<dim3(grid), dim3(block), 0, ctx->stream>>>();
    return launched(ctx, "krm_probe_empty_kernel");
  }
  KRM_REQUIRE(ctx, src && src % 16 == 0 && bytes % 16 == 0 && bytes > 0,
              "krm_probe_launch: the read probe needs a 16-byte aligned buffer and size");
  const size_t pieces = bytes / 16, threads = (size_t)grid * block;
  uint32_t* sink = ctx->tickets + (size_t)(kTicketSlots - 1) * kTicketStride;
  const size_t per = (pieces + threads - 1) / threads;
  if (per <= 1)
    krm_probe_read_kernel<1><<<dim3(grid), dim3(block), 0, ctx->stream>>>(ptr<const uint4>(src), pieces, sink);
  else if (per <= 2)
    krm_probe_read_kernel<2><<<dim3(grid), dim3(block), 0, ctx->stream>>>(ptr<const uint4>(src), pieces, sink);
  else if (per <= 4)
    krm_probe_read_kernel<4><<<dim3(grid), dim3(block), 0, ctx->stream>>>(ptr<const uint4>(src), pieces, sink);
  else
    krm_probe_read_kernel<8><<<dim3(grid), dim3(block), 0, ctx->stream>>>(ptr<const uint4>(src), pieces, sink);
  return launched(ctx, "krm_probe_read_kernel");
}

int32_t krm_probe_exchange(krm_ctx* ctx, krm_buf work, size_t work_bytes, uint32_t entries,
                           uint32_t phases, uint32_t spin_limit) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, entries == 2048 || entries == 4096 || entries == 8192,
              "krm_probe_exchange: entries %u (2048, 4096 or 8192)", entries);
  KRM_REQUIRE(ctx, phases >= 1 && spin_limit >= 1, "krm_probe_exchange: phases / spin_limit");
  // one workgroup per CU, all resident: 256 of them (a multiple of 4 that divides `entries`)
  const uint32_t grid = 256;
  KRM_REQUIRE(ctx, (uint32_t)ctx->num_cus >= grid,
              "krm_probe_exchange: %d CUs cannot hold %u resident workgroups", ctx->num_cus, grid);
  const size_t need = (size_t)2 * entries * sizeof(float) + (size_t)grid * 4 + 16;
  KRM_REQUIRE(ctx, work && work % 16 == 0 && work_bytes >= need,
              "krm_probe_exchange: work buffer of %zu bytes, %zu needed", work_bytes, need);
  KRM_TRY(krm_buf_zero(ctx, work, 0, need));
  float* vec = ptr<float>(work);
  uint32_t* flags = reinterpret_cast<uint32_t*>(vec + 2 * (size_t)entries);
  uint32_t* fault = flags + grid;
  if (entries == 2048)
    krm_probe_exchange_kernel<2048><<<dim3(grid), dim3(576), 0, ctx->stream>>>(vec, flags, fault, phases, spin_limit);
  else if (entries == 4096)
    krm_probe_exchange_kernel<4096><<<dim3(grid), dim3(576), 0, ctx->stream>>>(vec, flags, fault, phases, spin_limit);
  else
    krm_probe_exchange_kernel<8192><<<dim3(grid), dim3(576), 0, ctx->stream>>>(vec, flags, fault, phases, spin_limit);
  return launched(ctx, "krm_probe_exchange_kernel");
}

int32_t krm_event_create(krm_ctx* ctx, krm_event** out) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, out != nullptr, "krm_event_create: out is NULL");
  krm_event* ev = new krm_event();
  hipError_t st = hipEventCreate(&ev->ev);
  if (st != hipSuccess) {
    delete ev;
    return hip_status(ctx, st, "hipEventCreate");
  }
  *out = ev;
  return KRM_OK;
}

int32_t krm_event_record(krm_ctx* ctx, krm_event* ev) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, ev != nullptr, "krm_event_record: event is NULL");
  return hip_status(ctx, hipEventRecord(ev->ev, ctx->stream), "hipEventRecord");
}

int32_t krm_event_elapsed_ms(krm_ctx* ctx, krm_event* start, krm_event* stop, float* ms) {
  KRM_TRY(enter(ctx));
  KRM_REQUIRE(ctx, start && stop && ms, "krm_event_elapsed_ms: NULL argument");
  KRM_TRY(hip_status(ctx, hipEventSynchronize(stop->ev), "hipEventSynchronize"));
  return hip_status(ctx, hipEventElapsedTime(ms, start->ev, stop->ev), "hipEventElapsedTime");
}

int32_t krm_event_destroy(krm_ctx* ctx, krm_event* ev) {
  KRM_TRY(enter(ctx));
  if (!ev) return KRM_OK;
  hipError_t st = hipEventDestroy(ev->ev);
  delete ev;
  return hip_status(ctx, st, "hipEventDestroy");
}

}  // extern "C"
