/*
 * karume_oracle.c — TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, CPU restatement of the Karume IR runtime's reference semantics for the
 * int4 `linear` op, the states-form `attention` op and `state_append`, plus the few glue
 * ops a Llama-style decoder needs.  It exists so the HIP kernels can be checked against
 * the reference's own algorithm; it is never linked into, imported by, or called from the
 * product library.  Only the test-suite, the smoke check and the benchmark's CPU-baseline
 * leg may load it.
 *
 * Every function cites the reference file:line it restates (paths relative to the
 * reference repository root).  Accumulations are in double and rounded to float once at
 * the store, exactly like the reference's JavaScript (`number` is an IEEE double and
 * `Math.fround` is the single rounding).
 *
 * Pinning status (which reference-held vector or independent check fixes each function)
 * is listed in oracle/README.md; a function without one is marked "parity unpinned" there.
 *
 * Build: `make -C oracle`  (gcc -O2 -fopenmp -shared).  The `_mt` entry points are the
 * same loops with an OpenMP `parallel for` over independent output rows; results are
 * bit-identical to the single-threaded entry points because no reduction is split.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define KRMO_OK 0
#define KRMO_ERR_SHAPE (-1)

/* ---------------------------------------------------------------------------------------
 * f16 bits -> f32 (exact).  packages/runtime/src/format/f16.ts:23-36
 * exponent 0: signed zero / subnormal = mantissa * 2^-24; exponent 31: inf / NaN;
 * otherwise (1 + mantissa/1024) * 2^(exp-15).
 * ------------------------------------------------------------------------------------- */
float krmo_f16_bits_to_f32(uint16_t bits) {
  const double sign = (bits & 0x8000u) ? -1.0 : 1.0;
  const int exponent = (bits >> 10) & 0x1f;
  const int mantissa = bits & 0x3ff;
  if (exponent == 0) return (float)(sign * (double)mantissa * ldexp(1.0, -24));
  if (exponent == 0x1f) return mantissa == 0 ? (float)(sign * INFINITY) : NAN;
  return (float)(sign * (1.0 + (double)mantissa / 1024.0) * ldexp(1.0, exponent - 15));
}

void krmo_decode_f16(const uint16_t* bits, size_t count, float* out) {
  for (size_t i = 0; i < count; ++i) out[i] = krmo_f16_bits_to_f32(bits[i]);
}

/* f32 -> f16 bits, round-to-nearest-even (what Math.f16round does,
 * packages/runtime/src/format/f16.ts:68).  Written against the IEEE definition through a
 * double so subnormals, overflow to inf (>= 65520) and ties are handled by construction. */
uint16_t krmo_f32_to_f16_bits(float value) {
  uint32_t u;
  memcpy(&u, &value, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  if (isnan(value)) return (uint16_t)(sign | 0x7e00u);
  double a = fabs((double)value);
  if (isinf(value) || a >= 65520.0) return (uint16_t)(sign | 0x7c00u);
  if (a < ldexp(1.0, -14)) {
    /* subnormal (or zero): units of 2^-24, nearbyint is ties-to-even in the default mode */
    double q = nearbyint(a * ldexp(1.0, 24));
    return (uint16_t)(sign | (uint16_t)q); /* q == 1024 rolls into the smallest normal */
  }
  int e;
  double m = frexp(a, &e); /* a = m * 2^e, m in [0.5, 1) */
  double scaled = nearbyint(m * 2048.0); /* 11 significant bits */
  if (scaled == 2048.0) {
    scaled = 1024.0;
    e += 1;
  }
  int exponent = e - 1 + 15;
  if (exponent >= 31) return (uint16_t)(sign | 0x7c00u);
  return (uint16_t)(sign | (uint16_t)(exponent << 10) | ((uint16_t)scaled & 0x3ffu));
}

/* ---------------------------------------------------------------------------------------
 * Packed int4 -> f32.  packages/runtime/src/format/i4.ts:63-118
 *   element i lives in byte i>>1; odd i = high nibble, even i = low nibble; stored value
 *   u = q + 8; out[i] = fround((u - 8) * scale[row*groups + group]) — ONE f32 rounding of
 *   the exact (double) product.  Scale shape is [rows, width/group] (i4.ts:44-50).
 * Rejections mirror i4.ts:70-97 (byte length, group divisibility); the scale-shape checks
 * live in the caller because C receives no shape objects.
 * ------------------------------------------------------------------------------------- */
int krmo_decode_i4(const uint8_t* bytes, size_t byte_len, size_t rows, size_t width,
                   const float* scale, size_t group, float* out) {
  const size_t count = rows * width;
  if (count % 2 != 0 || byte_len * 2 != count) return KRMO_ERR_SHAPE;
  if (group < 1 || width % group != 0) return KRMO_ERR_SHAPE;
  const size_t groups = width / group;
  size_t i = 0;
  for (size_t row = 0; row < rows; ++row) {
    const size_t scale_base = row * groups;
    for (size_t g = 0; g < groups; ++g) {
      const double s = (double)scale[scale_base + g];
      for (size_t e = 0; e < group; ++e, ++i) {
        const uint8_t byte = bytes[i >> 1];
        const int u = (i & 1) ? (byte >> 4) : (byte & 0x0f);
        out[i] = (float)((double)(u - 8) * s);
      }
    }
  }
  return KRMO_OK;
}

/* Packer (the inverse used to build test inputs).  tools/exporter/src/karume/emit.py:292-322:
 * u = q + 8, element 2j -> low nibble of byte j, element 2j+1 -> high nibble. */
int krmo_pack_i4(const int8_t* q, size_t count, uint8_t* bytes) {
  if (count % 2 != 0) return KRMO_ERR_SHAPE;
  for (size_t j = 0; j < count / 2; ++j) {
    const int lo = q[2 * j] + 8, hi = q[2 * j + 1] + 8;
    if (lo < 0 || lo > 15 || hi < 0 || hi > 15) return KRMO_ERR_SHAPE;
    bytes[j] = (uint8_t)(lo | (hi << 4));
  }
  return KRMO_OK;
}

/* ---------------------------------------------------------------------------------------
 * linear.  packages/runtime/src/reference/ops.ts:879-897
 *   out[row, col] = fround( (sum_i x[row,i] * w[col,i], ascending i, in double) + bias[col] )
 *   weight is [N, K] with K contiguous ("transposed" layout).
 * ------------------------------------------------------------------------------------- */
static void linear_rows(const float* x, const float* w, const float* bias, size_t row0,
                        size_t row1, size_t n, size_t k, float* out) {
  for (size_t row = row0; row < row1; ++row) {
    for (size_t col = 0; col < n; ++col) {
      double acc = 0.0;
      for (size_t i = 0; i < k; ++i) acc += (double)x[row * k + i] * (double)w[col * k + i];
      out[row * n + col] = (float)(acc + (double)bias[col]);
    }
  }
}

void krmo_linear(const float* x, const float* w, const float* bias, size_t m, size_t n,
                 size_t k, float* out) {
  linear_rows(x, w, bias, 0, m, n, k, out);
}

/* Same loops, OpenMP over (row, col) pairs — each output still owns its whole K loop. */
void krmo_linear_mt(const float* x, const float* w, const float* bias, size_t m, size_t n,
                    size_t k, float* out) {
  const long long total = (long long)m * (long long)n;
#pragma omp parallel for schedule(static)
  for (long long idx = 0; idx < total; ++idx) {
    const size_t row = (size_t)(idx / (long long)n), col = (size_t)(idx % (long long)n);
    double acc = 0.0;
    for (size_t i = 0; i < k; ++i) acc += (double)x[row * k + i] * (double)w[col * k + i];
    out[row * n + col] = (float)(acc + (double)bias[col]);
  }
}

/* int4 linear without materialising the whole dequantised matrix: decodes one weight row
 * at a time with the decode formula above, then applies the linear formula above.  Used for
 * shapes whose f32 weight matrix would be large; bit-identical to decode + krmo_linear. */
int krmo_linear_i4_mt(const float* x, const uint8_t* bytes, const float* scale,
                      const float* bias, size_t m, size_t n, size_t k, size_t group,
                      float* out) {
  if (group < 1 || k % group != 0 || k % 2 != 0) return KRMO_ERR_SHAPE;
  const size_t groups = k / group;
  int failed = 0;
#pragma omp parallel
  {
    float* wrow = (float*)malloc(sizeof(float) * (k ? k : 1));
    if (!wrow) {
#pragma omp atomic write
      failed = 1;
    }
#pragma omp for schedule(static)
    for (long long col = 0; col < (long long)n; ++col) {
      if (!wrow) continue;
      const uint8_t* rb = bytes + (size_t)col * (k / 2);
      for (size_t i = 0; i < k; ++i) {
        const uint8_t byte = rb[i >> 1];
        const int u = (i & 1) ? (byte >> 4) : (byte & 0x0f);
        wrow[i] = (float)((double)(u - 8) * (double)scale[(size_t)col * groups + i / group]);
      }
      for (size_t row = 0; row < m; ++row) {
        double acc = 0.0;
        for (size_t i = 0; i < k; ++i) acc += (double)x[row * k + i] * (double)wrow[i];
        out[row * n + (size_t)col] = (float)(acc + (double)bias[col]);
      }
    }
    free(wrow);
  }
  return failed ? KRMO_ERR_SHAPE : KRMO_OK;
}

/* ---------------------------------------------------------------------------------------
 * w4a8: per-token int8 activations x int4 group-quantised weights, integer dot products.
 * ------------------------------------------------------------------------------------- */

/* Per-row (= per-token) symmetric int8 quantisation.
 * packages/runtime/src/reference/i8a8.ts:92-118 (kernel: src/kernels/quantize-rows.ts:89-146):
 *   amax = max |x| over the row, NaN propagates to the row's scale;
 *   s    = max(f32(amax * f32(1/127)), f32 tiny)   -- a multiplication, never amax / 127;
 *   q    = clamp(round-half-to-even(f32(x / s)), -127, +127).
 * The JavaScript computes amax * (1/127) and x / s in double and rounds once to f32; both
 * equal the IEEE f32 operation (the product of two f32 is exact in double, and a double
 * quotient rounded to f32 is the correctly rounded f32 quotient), so plain float arithmetic
 * is used here.  A NaN quotient (NaN or Inf scale) stores 0, like an Int8Array store. */
void krmo_quantize_rows(const float* x, size_t rows, size_t dim, int8_t* q, float* scale) {
  const float inv_abs_max = (float)(1.0 / 127.0);
  const float tiny = 1.1754943508222875e-38f;
  for (size_t row = 0; row < rows; ++row) {
    const float* xr = x + row * dim;
    float amax = 0.0f;
    int saw_nan = 0;
    for (size_t i = 0; i < dim; ++i) {
      const float value = fabsf(xr[i]);
      if (isnan(value)) saw_nan = 1;
      else if (value > amax) amax = value;
    }
    float s = amax * inv_abs_max;
    if (!(s > tiny)) s = tiny;  /* Math.max(s, tiny); s is never NaN here */
    if (saw_nan) s = NAN;
    scale[row] = s;
    for (size_t i = 0; i < dim; ++i) {
      float r = rintf(xr[i] / s);  /* default rounding mode: ties to even */
      if (isnan(r)) r = 0.0f;
      if (r > 127.0f) r = 127.0f;
      if (r < -127.0f) r = -127.0f;
      q[row * dim + i] = (int8_t)r;
    }
  }
}

/* Smallest distance of x / s from a half-integer over all finite quotients
 * (packages/runtime/src/reference/i8a8.ts:129-146): data with a large margin quantises the
 * same way under a division that is a few ulp off. */
double krmo_quantize_rows_tie_margin(const float* x, size_t rows, size_t dim) {
  double margin = INFINITY;
  int8_t* q = (int8_t*)malloc((rows * dim) ? rows * dim : 1);
  float* s = (float*)malloc(sizeof(float) * (rows ? rows : 1));
  if (!q || !s) { free(q); free(s); return -1.0; }
  krmo_quantize_rows(x, rows, dim, q, s);
  for (size_t row = 0; row < rows; ++row)
    for (size_t i = 0; i < dim; ++i) {
      const float ratio = x[row * dim + i] / s[row];
      if (!isfinite(ratio)) continue;
      const double fraction = (double)ratio - floor((double)ratio);
      const double d = fabs(fraction - 0.5);
      if (d < margin) margin = d;
    }
  free(q);
  free(s);
  return margin;
}

/* w4a8 linear.  packages/runtime/src/reference/i8a8.ts:209-231 (contract:
 * docs/decisions/0076-w4a8-linear-execution.md:40-60):
 *   accf = 0;  for each group gi, ascending:
 *       acci = sum over the group of xq[row, i] * wq[col, i]           exact integer
 *       accf = fma(f32(acci), wscale[col, gi], accf)                   one rounding per group
 *   out = fma(accf, xs[row], bias[col])
 * The activation scale is applied once, last; groups are never merged into one integer sum.
 * fused != 0: each fma is a true fused multiply-add (what the reference's GPU kernel
 * executes).  fused == 0: the JavaScript reference's stand-in, (double)a * b + c rounded to
 * f32 -- the product is exact in double; the sum is rounded twice, which can differ from the
 * fused result only when the exact sum needs more than 53 bits.
 * Weights are the packed int4 bytes (flat element i in byte i / 2, low nibble first, stored
 * u = q + 8); `group` may be any divisor of k (the reference's known-answer cases use 2). */
int krmo_linear_w4a8(const float* x, const uint8_t* bytes, const float* wscale,
                     const float* bias, size_t m, size_t n, size_t k, size_t group, int fused,
                     float* out) {
  if (group < 1 || k % group != 0 || (n * k) % 2 != 0) return KRMO_ERR_SHAPE;
  const size_t groups = k / group;
  int8_t* q = (int8_t*)malloc((m * k) ? m * k : 1);
  float* xs = (float*)malloc(sizeof(float) * (m ? m : 1));
  if (!q || !xs) { free(q); free(xs); return KRMO_ERR_SHAPE; }
  krmo_quantize_rows(x, m, k, q, xs);
#pragma omp parallel for schedule(static)
  for (long long col = 0; col < (long long)n; ++col) {
    for (size_t row = 0; row < m; ++row) {
      float accf = 0.0f;
      for (size_t gi = 0; gi < groups; ++gi) {
        int64_t acci = 0;
        for (size_t i = gi * group; i < (gi + 1) * group; ++i) {
          const size_t flat = (size_t)col * k + i;
          const uint8_t byte = bytes[flat >> 1];
          const int u = (flat & 1) ? (byte >> 4) : (byte & 0x0f);
          acci += (int64_t)q[row * k + i] * (int64_t)(u - 8);
        }
        const float a = (float)acci, w = wscale[(size_t)col * groups + gi];
        accf = fused ? fmaf(a, w, accf) : (float)((double)a * (double)w + (double)accf);
      }
      out[row * n + (size_t)col] =
          fused ? fmaf(accf, xs[row], bias[col])
                : (float)((double)accf * (double)xs[row] + (double)bias[col]);
    }
  }
  free(q);
  free(xs);
  return KRMO_OK;
}

/* ---------------------------------------------------------------------------------------
 * states-form attention geometry.  packages/runtime/src/kernels/state-attention.ts:714-733
 * ------------------------------------------------------------------------------------- */
static int sliding(uint64_t window) { return window > 0; } /* state-attention.ts:148 */

uint64_t krmo_state_column_base(uint64_t window, uint64_t past) {
  if (!sliding(window)) return 0;
  const uint64_t keep = past < window - 1 ? past : window - 1;
  return past - keep;
}

uint64_t krmo_state_live_columns(uint64_t window, uint64_t past, uint64_t query) {
  return past - krmo_state_column_base(window, past) + query;
}

uint64_t krmo_state_effective_rows(uint64_t rows_block, uint64_t row_offset, uint64_t query) {
  const uint64_t left = query > row_offset ? query - row_offset : 0;
  return rows_block < left ? rows_block : left;
}

/* logical column -> physical slot row.  reference/state-attention.ts:101 */
static uint64_t slot_row(uint64_t window, uint64_t col) {
  return sliding(window) ? col % window : col;
}

/* Mutations the reference's own gates must catch
 * (packages/runtime/tests/gpu_state_attention_test.ts:714-765,793-815).  The test-suite
 * runs the oracle with each one switched on to prove its fixtures are sensitive to the
 * fault; 0 = faithful. */
enum {
  KRMO_MUT_NONE = 0,
  KRMO_MUT_DROP_LOWER_BOUND = 1,   /* sliding window lower bound removed */
  KRMO_MUT_RING_MOD_CAPACITY = 2,  /* read-side ring map col % C instead of col % W */
  KRMO_MUT_PAD_ROWS_COMPUTED = 3,  /* pad rows are computed instead of being exact 0 */
  KRMO_MUT_IGNORE_KV_REPEAT = 4,   /* kv plane = plane % (B*Hkv) instead of floor(plane / r) */
  KRMO_MUT_SCALE_ONE_SIDE = 6,     /* half-scale applied to q only */
  KRMO_MUT_APPEND_NO_RING = 7,     /* state_append ignores the ring map */
  KRMO_MUT_OVERFLOW_FORM = 8       /* u32 `col + W > limit` form of the lower bound */
};

/* ---------------------------------------------------------------------------------------
 * states-form attention.  packages/runtime/src/reference/state-attention.ts:110-181
 * (shape checks :63-86).  Three naive stages per (plane, row): S over the live columns
 * (outside the predicate = -inf), safe softmax with weights rounded to f32, then P @ V;
 * double accumulation, one float rounding per stage.  Rows >= query stay exact 0.
 * ------------------------------------------------------------------------------------- */
int krmo_state_attention_mut(const float* q, const float* ins_k, const float* ins_v,
                             const float* slot_k, const float* slot_v, float* out,
                             uint64_t batch, uint64_t heads, uint64_t kv_heads,
                             uint64_t chunk_rows, uint64_t depth, uint64_t capacity,
                             uint64_t window, uint64_t past, uint64_t query, float scale_in,
                             float* scratch /* 2*live floats */, int mutation) {
  if (batch < 1 || heads < 1 || kv_heads < 1 || chunk_rows < 1 || depth < 1 || capacity < 1)
    return KRMO_ERR_SHAPE;
  if (heads % kv_heads != 0) return KRMO_ERR_SHAPE;
  if (query < 1 || query > chunk_rows) return KRMO_ERR_SHAPE;
  if (sliding(window)) {
    if (window > capacity) return KRMO_ERR_SHAPE;
  } else if (past + query > capacity) {
    return KRMO_ERR_SHAPE;
  }
  const uint64_t repeat = heads / kv_heads;
  const double scale = (double)scale_in; /* Math.fround(input.scale): already a float */
  const uint64_t base = krmo_state_column_base(window, past);
  const uint64_t live = krmo_state_live_columns(window, past, query);
  float* scores = scratch;
  float* weights = scratch + live;
  memset(out, 0, sizeof(float) * batch * heads * chunk_rows * depth);
  const uint64_t rows_to_run = mutation == KRMO_MUT_PAD_ROWS_COMPUTED ? chunk_rows : query;
  for (uint64_t plane = 0; plane < batch * heads; ++plane) {
    const uint64_t kv_plane = mutation == KRMO_MUT_IGNORE_KV_REPEAT
                                  ? plane % (batch * kv_heads)
                                  : plane / repeat;
    for (uint64_t row = 0; row < rows_to_run; ++row) {
      const uint64_t q_base = (plane * chunk_rows + row) * depth;
      const uint64_t limit = past + row;
      for (uint64_t cl = 0; cl < live; ++cl) {
        const uint64_t col = base + cl;
        int in_window = col <= limit;
        if (in_window && sliding(window) && mutation != KRMO_MUT_DROP_LOWER_BOUND) {
          if (mutation == KRMO_MUT_OVERFLOW_FORM)
            in_window = (uint32_t)((uint32_t)col + (uint32_t)window) > (uint32_t)limit;
          else
            in_window = (limit - col) < window;
        }
        if (!in_window) {
          scores[cl] = -INFINITY;
          continue;
        }
        const float* source;
        uint64_t k_base;
        if (col < past) {
          const uint64_t prow =
              mutation == KRMO_MUT_RING_MOD_CAPACITY && sliding(window) ? col % capacity
                                                                        : slot_row(window, col);
          k_base = (kv_plane * capacity + prow) * depth;
          source = slot_k;
        } else {
          k_base = (kv_plane * chunk_rows + (col - past)) * depth;
          source = ins_k;
        }
        double acc = 0.0;
        const double kscale = mutation == KRMO_MUT_SCALE_ONE_SIDE ? 1.0 : scale;
        for (uint64_t d = 0; d < depth; ++d)
          acc += ((double)q[q_base + d] * scale) * ((double)source[k_base + d] * kscale);
        scores[cl] = (float)acc;
      }
      double amax = -INFINITY;
      for (uint64_t cl = 0; cl < live; ++cl)
        if ((double)scores[cl] > amax) amax = (double)scores[cl];
      if (amax == -INFINITY) continue; /* empty row: exact 0 */
      double total = 0.0;
      for (uint64_t cl = 0; cl < live; ++cl) total += exp((double)scores[cl] - amax);
      for (uint64_t cl = 0; cl < live; ++cl)
        weights[cl] = (float)(exp((double)scores[cl] - amax) / total);
      for (uint64_t d = 0; d < depth; ++d) {
        double acc = 0.0;
        for (uint64_t cl = 0; cl < live; ++cl) {
          const uint64_t col = base + cl;
          const float* source;
          uint64_t v_base;
          if (col < past) {
            const uint64_t prow =
                mutation == KRMO_MUT_RING_MOD_CAPACITY && sliding(window) ? col % capacity
                                                                          : slot_row(window, col);
            v_base = (kv_plane * capacity + prow) * depth;
            source = slot_v;
          } else {
            v_base = (kv_plane * chunk_rows + (col - past)) * depth;
            source = ins_v;
          }
          acc += (double)weights[cl] * (double)source[v_base + d];
        }
        out[q_base + d] = (float)acc;
      }
    }
  }
  return KRMO_OK;
}

int krmo_state_attention(const float* q, const float* ins_k, const float* ins_v,
                         const float* slot_k, const float* slot_v, float* out, uint64_t batch,
                         uint64_t heads, uint64_t kv_heads, uint64_t chunk_rows, uint64_t depth,
                         uint64_t capacity, uint64_t window, uint64_t past, uint64_t query,
                         float scale, float* scratch) {
  return krmo_state_attention_mut(q, ins_k, ins_v, slot_k, slot_v, out, batch, heads, kv_heads,
                                  chunk_rows, depth, capacity, window, past, query, scale,
                                  scratch, KRMO_MUT_NONE);
}

/* ---------------------------------------------------------------------------------------
 * state_append.  packages/runtime/src/reference/state-attention.ts:211-241
 * Writes the first `query` rows of x[planes, M, D] into slot[planes, C, D] at
 * slot_row(past + row), ascending row (so with query > window the last logical row wins).
 * `slot` is updated in place: callers that need the reference's "returns a copy" behaviour
 * copy first.
 * ------------------------------------------------------------------------------------- */
int krmo_state_append_mut(const float* x, float* slot, uint64_t kv_planes, uint64_t chunk_rows,
                          uint64_t depth, uint64_t capacity, uint64_t window, uint64_t past,
                          uint64_t query, int mutation) {
  if (kv_planes < 1 || chunk_rows < 1 || depth < 1 || capacity < 1) return KRMO_ERR_SHAPE;
  if (query < 1 || query > chunk_rows) return KRMO_ERR_SHAPE;
  if (sliding(window)) {
    if (window > capacity) return KRMO_ERR_SHAPE;
  } else if (past + query > capacity) {
    return KRMO_ERR_SHAPE;
  }
  for (uint64_t plane = 0; plane < kv_planes; ++plane) {
    for (uint64_t row = 0; row < query; ++row) {
      const uint64_t src = (plane * chunk_rows + row) * depth;
      uint64_t prow = slot_row(window, past + row);
      if (mutation == KRMO_MUT_APPEND_NO_RING) prow = (past + row) % capacity;
      const uint64_t dst = (plane * capacity + prow) * depth;
      for (uint64_t d = 0; d < depth; ++d) slot[dst + d] = x[src + d];
    }
  }
  return KRMO_OK;
}

int krmo_state_append(const float* x, float* slot, uint64_t kv_planes, uint64_t chunk_rows,
                      uint64_t depth, uint64_t capacity, uint64_t window, uint64_t past,
                      uint64_t query) {
  return krmo_state_append_mut(x, slot, kv_planes, chunk_rows, depth, capacity, window, past,
                               query, KRMO_MUT_NONE);
}

/* ---------------------------------------------------------------------------------------
 * allclose.  packages/runtime/src/reference/allclose.ts:47-82
 * pass iff every element satisfies |x - y| <= atol + rtol*|y| and both sides are finite.
 * Returns the number of failing elements; writes max abs error (inf if any non-finite).
 * ------------------------------------------------------------------------------------- */
size_t krmo_allclose(const float* actual, const float* expected, size_t count, double atol,
                     double rtol, double* max_abs_out, size_t* worst_index_out) {
  size_t fail = 0, worst = 0, non_finite = 0;
  double max_abs = 0.0;
  for (size_t i = 0; i < count; ++i) {
    const double x = actual[i], y = expected[i];
    if (!isfinite(x) || !isfinite(y)) {
      if (non_finite == 0) worst = i;
      ++non_finite;
      ++fail;
      max_abs = INFINITY;
      continue;
    }
    const double a = fabs(x - y);
    if (a > max_abs && non_finite == 0) {
      max_abs = a;
      worst = i;
    }
    if (a > atol + rtol * fabs(y)) ++fail;
  }
  if (max_abs_out) *max_abs_out = max_abs;
  if (worst_index_out) *worst_index_out = worst;
  return fail;
}

/* ---------------------------------------------------------------------------------------
 * Glue ops of a Llama-style decoder layer (needed only by the whole-model check).
 * ------------------------------------------------------------------------------------- */

/* rms_norm.  packages/runtime/src/reference/ops.ts:948-970
 * out = fround( x * (1/sqrt(mean(x^2) + eps)) * weight ), squares summed in double. */
void krmo_rms_norm(const float* x, const float* weight, size_t rows, size_t dim, double eps,
                   float* out) {
  for (size_t row = 0; row < rows; ++row) {
    const size_t base = row * dim;
    double squares = 0.0;
    for (size_t i = 0; i < dim; ++i) squares += (double)x[base + i] * (double)x[base + i];
    const double inv = 1.0 / sqrt(squares / (double)dim + eps);
    for (size_t i = 0; i < dim; ++i)
      out[base + i] = (float)((double)x[base + i] * inv * (double)weight[i]);
  }
}

/* argmax over the last dimension, ties -> smallest index, NaN counts as the maximum.
 * packages/runtime/src/reference/ops.ts:533-560, packages/runtime/src/kernels/argmax.ts:16-34 */
void krmo_argmax(const float* x, size_t rows, size_t dim, int32_t* out) {
  for (size_t row = 0; row < rows; ++row) {
    const float* r = x + row * dim;
    size_t best = 0;
    for (size_t i = 1; i < dim; ++i) {
      const float v = r[i], b = r[best];
      if (isnan(b)) break;
      if (isnan(v) || v > b) best = i;
    }
    out[row] = (int32_t)best;
  }
}

/* half-split RoPE.  packages/runtime/src/kernels/rope.ts:5-20,52-80 (the fused kernel keeps
 * the primitive chain's roundings: both products are rounded to f32 before the add, as the
 * reference's mul -> mul -> add oracle chain does, packages/runtime/src/reference/ops.ts:297).
 *   rotate_half(x) = cat(-x[D/2:], x[:D/2]);  out = fround(fround(x*cos) + fround(rot*sin))
 * x is [planes, S, D]; cos/sin are [S, D] tables indexed by the row's position in S. */
void krmo_rope_half(const float* x, const float* cos_table, const float* sin_table,
                    size_t planes, size_t sequence, size_t head_dim, float* out) {
  const size_t half = head_dim / 2;
  for (size_t p = 0; p < planes; ++p) {
    for (size_t t = 0; t < sequence; ++t) {
      const size_t base = (p * sequence + t) * head_dim;
      for (size_t d = 0; d < head_dim; ++d) {
        const float rotated = d < half ? -x[base + d + half] : x[base + d - half];
        const float direct = (float)((double)x[base + d] * (double)cos_table[t * head_dim + d]);
        const float cross = (float)((double)rotated * (double)sin_table[t * head_dim + d]);
        out[base + d] = (float)((double)direct + (double)cross);
      }
    }
  }
}

/* SwiGLU gate: silu(gate) * up as the reference's op chain sigmoid -> mul -> mul, each op
 * rounding its result to f32 once.  sigmoid oracle = 1/(1+exp(-x)) in double
 * (packages/runtime/src/reference/ops.ts:150); the fused silu kernel stores the rounded
 * sigmoid and then multiplies (packages/runtime/src/kernels/silu.ts:47-93). */
void krmo_silu_mul(const float* gate, const float* up, size_t count, float* out) {
  for (size_t i = 0; i < count; ++i) {
    const float sig = (float)(1.0 / (1.0 + exp(-(double)gate[i])));
    const float act = (float)((double)gate[i] * (double)sig);
    out[i] = (float)((double)act * (double)up[i]);
  }
}

/* embedding row gather; an out-of-range index is an error, never a clamp.
 * packages/runtime/src/reference/ops.ts:1110-1131 */
int krmo_embedding(const float* weight, const int32_t* index, size_t count, size_t vocab,
                   size_t hidden, float* out) {
  for (size_t row = 0; row < count; ++row) {
    const int32_t pick = index[row];
    if (pick < 0 || (size_t)pick >= vocab) return KRMO_ERR_SHAPE;
    memcpy(out + row * hidden, weight + (size_t)pick * hidden, sizeof(float) * hidden);
  }
  return KRMO_OK;
}
