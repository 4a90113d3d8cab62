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
  char error[512] = {0};
};

struct krm_event {
  hipEvent_t ev;
};

namespace krm {

constexpr int kWave = 64;

// Records the message on the context (or on the context-less slot) and returns `code`.
int32_t fail(krm_ctx* ctx, int32_t code, const char* fmt, ...);

// Maps a HIP runtime status to an error class; 0 when `status` is hipSuccess.
int32_t hip_status(krm_ctx* ctx, hipError_t status, const char* what);

// Makes the context's device current on the calling thread (calls may arrive on any thread).
int32_t enter(krm_ctx* ctx);

// Error check of the launch that was just queued.
int32_t launched(krm_ctx* ctx, const char* kernel);

inline bool valid_dtype(int32_t dtype) { return dtype == KRM_F32 || dtype == KRM_F16; }
inline size_t dtype_bytes(int32_t dtype) { return dtype == KRM_F16 ? 2 : 4; }
inline bool is_pow2(uint32_t v) { return v != 0 && (v & (v - 1)) == 0; }
inline bool aligned(krm_buf address, size_t bytes) { return (address % bytes) == 0; }

template <typename T>
inline T* ptr(krm_buf address) {
  return reinterpret_cast<T*>(static_cast<uintptr_t>(address));
}

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
