// int4 `linear` for M > 16 rows (prefill).  Placeholder body: runs the f32 GEMV over blocks of
// 16 rows until the MFMA kernel lands in this file.
#include "krm_internal.h"

namespace krm {

int32_t linear_i4_gemv(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                       krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                       int32_t io_dtype, int32_t scale_dtype);

int32_t linear_i4_gemm_f16(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                           krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                           int32_t io_dtype, int32_t scale_dtype) {
  const size_t eb = dtype_bytes(io_dtype);
  for (uint32_t r = 0; r < m; r += 16) {
    const uint32_t rows = m - r < 16 ? m - r : 16;
    KRM_TRY(linear_i4_gemv(ctx, x + (size_t)r * k * eb, w, scales, bias,
                           out + (size_t)r * n * eb, rows, n, k, group, io_dtype, scale_dtype));
  }
  return KRM_OK;
}

}  // namespace krm
