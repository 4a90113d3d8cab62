/*
 * karume_hip.h — C ABI of libkarume_hip.so, the gfx950 (MI355X, wave64) backend for the
 * Karume IR runtime's int4 `linear`, states-form `attention` and `state_append` ops.
 *
 * The reference has no FFI: every op reaches the device as a WebGPU DispatchRecipe = a
 * params struct + an ordered list of buffer bindings + a grid
 * (packages/runtime/src/runtime/recipe.ts:87-96).  Each entry point below takes exactly what
 * the corresponding recipe carries — the params words as scalar arguments, the bindings as
 * device addresses — so a Deno host can `Deno.dlopen` this library and call it where the
 * reference would have pushed the recipe.  Citations are `path:line` in the reference tree.
 *
 * Conventions
 *  - every function returns int32: 0 = ok, negative = error class (below).  The text of the
 *    last error of a context is available from krm_last_error().
 *  - `krm_buf` is a raw device address (uint64).  Offsets are applied by the caller
 *    (address + bytes).  The caller owns every buffer; the library owns its context, its
 *    stream and whatever scratch it allocated itself.
 *  - launches are asynchronous on the context's stream; krm_buf_download and krm_sync fence.
 *  - host pointers are only read/written during the call.
 *  - one context = one stream, externally serialised (the reference serialises runs per
 *    Session, packages/runtime/src/runtime/generation-context.ts:103-106).  The device is set
 *    on entry of every call, so calls may come from any OS thread.
 *  - nothing is approximated silently: an unsupported combination is rejected before launch.
 */
#ifndef KARUME_HIP_H
#define KARUME_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct krm_ctx krm_ctx;
typedef uint64_t krm_buf;
typedef struct krm_event krm_event;

/* Error classes; they mirror the reference's public error types
 * (packages/runtime/mod.ts:25-35,112). */
#define KRM_OK 0
#define KRM_ERR_VALIDATION (-1)    /* GpuValidationError: shapes / attrs / alignment rejected */
#define KRM_ERR_OUT_OF_MEMORY (-2) /* GpuOutOfMemoryError */
#define KRM_ERR_DEVICE_LOST (-3)   /* GpuDeviceLostError: the HIP runtime reported a failure */
#define KRM_ERR_EXECUTION (-4)     /* ExecutionError: contract of a run violated (P+Q > C ...) */

/* Element encodings of activation / scale / KV-slot buffers. */
#define KRM_F32 0
#define KRM_F16 1

/* `linear` arithmetic, the reference's SessionOptions.linearCompute
 * (packages/runtime/src/runtime/session-types.ts:127-195).  M <= 16 always runs the
 * bandwidth-bound GEMV (exact products, f32 accumulation).  For M > 16:
 *   KRM_COMPUTE_F32  — f32-class results for every M (the reference default).  f32 activations
 *                      on large shapes run on the matrix cores: x * 2^e = hi + lo (two fp16,
 *                      22 bits, e per row), weights as the exact integers (u - 8), products
 *                      exact, f32 sums, the group scale applied to the f32 sum of each group;
 *                      gated at the GEMV's tolerance.  fp16 activations need no split.  Other
 *                      shapes take the GEMV over blocks of 16 rows.
 *   KRM_COMPUTE_F16  — f32 activations are rounded to fp16 once.  Large shapes (the (tile,
 *                      stage) units of 64 x 512 tiles cover every CU at least twice, group >= 64,
 *                      k % 32 == 0): exact integer weights as above, so with fp16 activations
 *                      the result is of f32 class.  Smaller shapes: every weight rounded once
 *                      to fp16((u - 8) * scale), which bounds an output's error by about
 *                      2^-11 * sqrt(k) * rms(x * w).  (The reference rejects f16 compute with
 *                      i4 weights, packages/runtime/src/kernels/gemm.ts:1204-1209: no
 *                      same-numerics counterpart there.) */
#define KRM_COMPUTE_F32 0
#define KRM_COMPUTE_F16 1

/* ---- context (acquireGpu / GpuContext.destroy, packages/runtime/mod.ts:13-113) ---------- */
/* A context owns, besides its stream, 1 MiB of pinned host staging and device scratch that its
 * kernels share: 8 MiB of arrival counters (split attention, shared GEMM tiles) and two
 * 128 x 256 f32 tile partials per CU (64 MiB on 256 CUs) for the prefill GEMM.  Calls on one
 * context are ordered on its stream; two contexts never share scratch. */
int32_t krm_ctx_create(int32_t device, krm_ctx** out);
/* Same, but launches go to an existing hipStream_t (0 = the device's default stream); the
 * stream stays owned by the caller. */
int32_t krm_ctx_create_on_stream(int32_t device, void* hip_stream, krm_ctx** out);
int32_t krm_ctx_destroy(krm_ctx* ctx);
/* Text of the last error on `ctx` (or of the last context-less failure when ctx is NULL).
 * Valid until the next failing call on the same context. */
const char* krm_last_error(krm_ctx* ctx);
/* Fence: returns when everything queued on the context's stream has finished. */
int32_t krm_sync(krm_ctx* ctx);
/* Library identification: "karume-hip <version> gfx950". */
const char* krm_version(void);

/* ---- buffers (createBuffer / queue.writeBuffer / readback mapAsync,
 *      packages/runtime/src/runtime/executor.ts:870-896,1272) ------------------------------ */
int32_t krm_buf_alloc(krm_ctx* ctx, size_t bytes, krm_buf* out);
int32_t krm_buf_free(krm_ctx* ctx, krm_buf buf);
int32_t krm_buf_upload(krm_ctx* ctx, krm_buf dst, size_t dst_offset, const void* host,
                       size_t bytes);
int32_t krm_buf_download(krm_ctx* ctx, krm_buf src, size_t src_offset, void* host, size_t bytes);
/* State slots are zero-initialised at creation
 * (packages/runtime/tests/gpu_state_execution_test.ts:159-164). */
int32_t krm_buf_zero(krm_ctx* ctx, krm_buf dst, size_t dst_offset, size_t bytes);

/* Device-to-device copy on the context's stream (copyBufferToBuffer); 16-byte granularity. */
int32_t krm_buf_copy(krm_ctx* ctx, krm_buf dst, krm_buf src, size_t bytes);

/* ---- timing (timestamp-query diagnostics, packages/runtime/src/gpu/submit.ts:54-63) ------ */
int32_t krm_event_create(krm_ctx* ctx, krm_event** out);
int32_t krm_event_record(krm_ctx* ctx, krm_event* ev);
/* Waits for `stop`, then writes the milliseconds between the two recorded events. */
int32_t krm_event_elapsed_ms(krm_ctx* ctx, krm_event* start, krm_event* stop, float* ms);
int32_t krm_event_destroy(krm_ctx* ctx, krm_event* ev);
/* ---- recorded launch sequences (the reference bakes a step's dispatch recipes once and
 *      replays them: executeBakedPlan, packages/runtime/src/runtime/recipe.ts:357-394) ------
 * Between krm_graph_begin and krm_graph_end the op entry points record instead of running
 * (HIP stream capture); krm_graph_launch replays the recorded sequence on the context's
 * stream with the pointers and scalars it was recorded with.  Calls that must wait for the
 * device (upload, download, free, sync, krm_attention_varlen) are rejected while recording. */
typedef struct krm_graph krm_graph;
int32_t krm_graph_begin(krm_ctx* ctx);
/* While recording: the ops that follow go to parallel branch `branch` (0 = the main branch,
 * 1..3 = side branches).  A side branch forks from the main branch at its first selection
 * (it depends on what the main branch held at that moment) and every side branch joins the
 * main branch in krm_graph_end.  Ops on different branches must not depend on one another;
 * the device may run them at the same time (the recipes of one step that the reference
 * submits in one command buffer without barriers between independent dispatches,
 * packages/runtime/src/runtime/recipe.ts:385-394).
 * Ops that use the context's own scratch share it in launch order and therefore belong on the
 * main branch; while a side branch is selected they fail with KRM_ERR_VALIDATION and record
 * nothing: the decode attention when it splits the columns (more than four chunks),
 * krm_attention_varlen / _planned, the unit-dealt MFMA GEMMs of krm_linear_i4 and every
 * f32-class (KRM_COMPUTE_F32 with f32 x) MFMA product.  GEMVs (m <= 16), the fp16-operand
 * few-row products, krm_attention_state_noalloc (its own scratch: still one call at a time per
 * GPU) and the glue ops carry no such state. */
int32_t krm_graph_branch(krm_ctx* ctx, uint32_t branch);
int32_t krm_graph_end(krm_ctx* ctx, krm_graph** out);
int32_t krm_graph_launch(krm_ctx* ctx, krm_graph* graph);
int32_t krm_graph_destroy(krm_ctx* ctx, krm_graph* graph);

/* ---- int4 storage (packages/runtime/src/format/i4.ts:63-118,
 *      packages/runtime/src/kernels/weight-storage.ts:152-187) ------------------------------
 * Expands packed int4 `w` ([rows, width] elements, 2 per byte, element 2j = low nibble,
 * stored u = q + 8) into f32: out[i] = f32(u - 8) * scale[row*(width/group) + (i%width)/group],
 * one f32 multiply — bit-identical to decodeI4.  Requires group >= 1, width % group == 0,
 * (rows*width) % 8 == 0 and 4-byte aligned `w`. */
int32_t krm_dequant_i4(krm_ctx* ctx, krm_buf w, krm_buf scales, krm_buf out_f32, uint64_t rows,
                       uint64_t width, uint32_t group, int32_t scale_dtype);

/* ---- linear with int4 weights (bindings 1-5 + Dims{m,n,k}:
 *      packages/runtime/src/kernels/gemm.ts:115,315-327,1223-1227;
 *      builder packages/runtime/src/runtime/recipe-builder.ts:1311-1392) --------------------
 * out[m, n] = (sum_k x[m,k] * dequant(w)[n,k]) + bias[n]
 *   x      [m, k]  io_dtype, row-major
 *   w      [n, k]  packed int4, k contiguous (k/2 bytes per row)
 *   scales [n, k/group]  scale_dtype
 *   bias   [n]     io_dtype, or 0 for "no bias" (the reference always binds one; zeros)
 *   out    [m, n]  io_dtype
 * group must be a power of two >= 16 dividing k (docs/ir-v1.md:135-150).
 * The kernel is a pure function of (m, n, k, group, dtypes, compute); for m <= 16 a row of
 * `out` does not depend on the other rows in the call (same reduction order for every m). */
int32_t krm_linear_i4(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                      krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                      int32_t io_dtype, int32_t scale_dtype, int32_t compute);

/* Decode-step fusion of the same op (m <= 16): what the reference's peephole fusion pass does
 * at the recipe level (packages/runtime/src/runtime/fusion.ts), done here inside the GEMV:
 *   norm_weight_f32 != 0 : x is first rms-normalised,  x' = x * rsqrt(mean(x^2) + eps) * weight
 *                          (krm_rms_norm folded in; the normalised row is not rounded in between)
 *   residual != 0        : out = linear(...) + residual        ([m, n_out], io_dtype)
 *   KRM_EPILOGUE_SILU_PAIRS : weight rows are interleaved (2i, 2i+1) = (gate_i, up_i) and
 *                          out[m, i] = silu(gate_i) * up_i with n_out = n / 2 (krm_silu_mul folded in)
 * Each output row still depends on its own x row only. */
#define KRM_EPILOGUE_NONE 0
#define KRM_EPILOGUE_SILU_PAIRS 1
int32_t krm_linear_i4_fused(krm_ctx* ctx, krm_buf x, krm_buf norm_weight_f32, float norm_eps,
                            krm_buf w, krm_buf scales, krm_buf bias, krm_buf residual,
                            krm_buf out, uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                            int32_t io_dtype, int32_t scale_dtype, int32_t epilogue);

/* The same op for a chunk of rows (prefill; any m >= 1) with the epilogues of the fused form,
 * on the matrix cores: weights enter as the exact integers (u - 8), the group scale multiplies
 * the f32 sum of a group; KRM_COMPUTE_F16 rounds x to fp16 once, KRM_COMPUTE_F32 with f32 x
 * splits it into fp16 hi + lo (as krm_linear_i4 does for large shapes).
 *   residual != 0           : out = linear(...) + residual   ([m, n_out], io_dtype; `out` may be
 *                             the residual buffer itself: an element is read and written by
 *                             one thread)
 *   KRM_EPILOGUE_SILU_PAIRS : rows (2i, 2i+1) of w = (gate_i, up_i), out[m, i] = silu(gate) * up,
 *                             n_out = n / 2; gate and up are not rounded to io_dtype in between
 * x_dtype is the element type of x: io_dtype, or KRM_F16 beside io_dtype KRM_F32 under
 * KRM_COMPUTE_F16 — an fp16 copy of the activations (krm_rms_norm_cast, KRM_CHUNK_OUT_F16, an
 * fp16-io call of this function write one) holding exactly what f32 activations are rounded to
 * in that class, so the result is the same bit for bit and x costs half the bytes; bias,
 * residual and out stay io_dtype.
 * Covers group_size >= 64, k % 32 == 0, 16-byte aligned x and w; anything else is rejected
 * (krm_linear_i4 + krm_silu_mul + krm_add remain).  A pure function of the shape and dtypes.
 * Fuses packages/runtime/src/kernels/linear.ts:34-64 with the elementwise add / silu-mul that
 * follow it in a decoder layer (packages/runtime/src/runtime/fusion.ts). */
int32_t krm_linear_i4_rows(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                           krm_buf residual, krm_buf out, uint32_t m, uint32_t n, uint32_t k,
                           uint32_t group, int32_t io_dtype, int32_t scale_dtype, int32_t compute,
                           int32_t epilogue, int32_t x_dtype);

/* ---- states-form attention (Params 10 words + Lengths{past,query} + bindings:
 *      packages/runtime/src/kernels/state-attention.ts:169-180,190-193,284-294,476-487;
 *      builder packages/runtime/src/runtime/recipe-builder.ts:1856-2002;
 *      contract docs/ir-v1.md:296-351) -------------------------------------------------------
 * One call replaces the reference's three dispatches (QK -> row stats -> PV); the score
 * matrix is never materialised.
 *   q      [B, H,   M, D]  io_dtype
 *   ins_k  [B, Hkv, M, D]  io_dtype   this step's keys   (valid rows: first `query`)
 *   ins_v  [B, Hkv, M, D]  io_dtype   this step's values
 *   slot_k [B, Hkv, C, D]  kv_dtype   past keys   (logical column c < past lives in physical
 *   slot_v [B, Hkv, C, D]  kv_dtype   past values  row c, or c % window when window > 0)
 *   out    [B, H,   M, D]  io_dtype   rows >= query are written as exact +0
 * Row r attends to logical columns c with c <= past + r and (window == 0 or
 * past + r - c < window); kv plane of (b, h) is floor((b*H + h) / (H/Hkv)).
 * `half_scale` multiplies q AND k (IR attr `scale`; sqrt(1/sqrt(D)) for the usual 1/sqrt(D)).
 * Rejected before launch: H % Hkv != 0, query < 1 or > M, window > C, window == 0 with
 * past + query > C (packages/runtime/src/kernels/state-attention.ts:588-636,
 * packages/runtime/src/runtime/recipe.ts:273-280).
 * `workspace` holds split-K partials; ask krm_attention_state_workspace for its size. */
int32_t krm_attention_state_workspace(uint32_t batch, uint32_t heads, uint32_t kv_heads,
                                      uint32_t chunk_rows, uint32_t depth, uint32_t window,
                                      uint32_t max_past, uint32_t max_query, size_t* bytes);
int32_t krm_attention_state(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                            krm_buf slot_k, krm_buf slot_v, krm_buf out, uint32_t batch,
                            uint32_t heads, uint32_t kv_heads, uint32_t chunk_rows,
                            uint32_t depth, uint32_t capacity, uint32_t window,
                            float half_scale, uint32_t past, uint32_t query, int32_t io_dtype,
                            int32_t kv_dtype, krm_buf workspace, size_t workspace_bytes);

/* krm_attention_state for callers that cannot allocate device memory or hand in a workspace:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  Same arguments, checks and results (bit for bit) as
 * krm_attention_state, minus the workspace: split partials and arrival counters live in a
 * 4 MiB array that is part of the library's device code (every GPU the library runs on holds
 * its copy until the process ends).  It calls no allocating routine.  Limits: the call's split
 * partials (krm_attention_state_workspace bytes) must fit 4 MiB - 64 KiB and it may use at most
 * 512 arrival counters (B * Hkv * head groups); beyond that it returns KRM_ERR_VALIDATION and
 * krm_attention_state with a workspace is the call to make.  All calls on one GPU share the
 * array, whatever their context: calls that overlap on one GPU race. */
int32_t krm_attention_state_noalloc(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                                    krm_buf slot_k, krm_buf slot_v, krm_buf out, uint32_t batch,
                                    uint32_t heads, uint32_t kv_heads, uint32_t chunk_rows,
                                    uint32_t depth, uint32_t capacity, uint32_t window,
                                    float half_scale, uint32_t past, uint32_t query,
                                    int32_t io_dtype, int32_t kv_dtype);

/* The attention of a chunk of rows (a prefill step) with what a decoder layer does around it
 * folded in; D = 64, 128 or 256 and 16-byte aligned buffers, anything else is rejected (the three
 * separate calls remain).  Arguments as krm_attention_state; `lengths` != 0 reads past / query
 * on the device as krm_attention_state_lengths does.  No workspace.
 *   KRM_CHUNK_OUT_ROW_MAJOR : `out` is [B, M, H, D] (what the o-projection reads) instead of
 *                             [B, H, M, D] — the permute + reshape nodes behind the attention
 *   KRM_CHUNK_APPEND        : the first `query` rows of ins_k / ins_v are also appended to the
 *                             slots (krm_state_append's result, same roundings).  window == 0
 *                             only: slot rows past.. are read by nobody in this launch, while a
 *                             ring would overwrite rows it still reads (docs/ir-v1.md:345-348).
 *   KRM_CHUNK_OUT_F16       : `out` is fp16 whatever io_dtype is: the f32 result rounded once,
 *                             i.e. what a KRM_COMPUTE_F16 product would round it to when it
 *                             reads it (see x_dtype of krm_linear_i4_rows)
 * Fuses packages/runtime/src/kernels/state-attention.ts:169-552 with
 * packages/runtime/src/kernels/state-append.ts:47-96 and the permute of
 * tools/export-recipes/minicpm5/export_decode.py:14-35. */
#define KRM_CHUNK_OUT_ROW_MAJOR 1u
#define KRM_CHUNK_APPEND 2u
#define KRM_CHUNK_OUT_F16 4u
int32_t krm_attention_chunk(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v, krm_buf slot_k,
                            krm_buf slot_v, krm_buf out, uint32_t batch, uint32_t heads,
                            uint32_t kv_heads, uint32_t chunk_rows, uint32_t depth,
                            uint32_t capacity, uint32_t window, float half_scale, uint32_t past,
                            uint32_t query, krm_buf lengths, int32_t io_dtype, int32_t kv_dtype,
                            uint32_t flags);

/* ---- state_append (packages/runtime/src/kernels/state-append.ts:47-96,120-173;
 *      builder packages/runtime/src/runtime/recipe-builder.ts:2011-2048) --------------------
 * Copies the first `query` rows of x[kv_planes, M, D] (x_dtype) into
 * slot[kv_planes, C, D] (slot_dtype) at physical row (past+row) or (past+row) % window.
 * Rows >= query are never written.  With window > 0 and query > window only the last
 * logical row mapping to a physical row is written.  f32 -> f16 rounds to nearest even.
 * Must be issued after every reader of the slot in the same step (docs/ir-v1.md:345-348). */
int32_t krm_state_append(krm_ctx* ctx, krm_buf x, krm_buf slot, uint32_t kv_planes,
                         uint32_t chunk_rows, uint32_t depth, uint32_t capacity,
                         uint32_t window, uint32_t past, uint32_t query, int32_t x_dtype,
                         int32_t slot_dtype);

/* ---- run-time lengths on the device ---------------------------------------------------------
 * The reference carries (pastLength, queryLength) in an 8-byte uniform owned by the generation
 * context and rewritten every run, so that a baked plan can be replayed
 * (packages/runtime/src/kernels/state-attention.ts:190-193,
 * packages/runtime/src/runtime/generation-context.ts:559-591).  `lengths` below is the same
 * idea: 16 bytes of device memory {u32 past, u32 query, u32 fault, u32 reserved}.  The
 * `_lengths` forms of attention and append read past/query from it on the device, which lets
 * a recorded decode step (krm_graph_*) be replayed while the sequence grows.  A step whose
 * lengths break the run contract (query outside 1..M, past + query > C on a full slot) writes
 * nothing and raises `fault`; krm_lengths_advance then leaves `past` unchanged. */
int32_t krm_lengths_set(krm_ctx* ctx, krm_buf lengths, uint32_t past, uint32_t query);
/* past += query (only when no fault is raised). */
int32_t krm_lengths_advance(krm_ctx* ctx, krm_buf lengths);
/* positions[i] = past + i for i < rows (the decode graph's position_ids input). */
int32_t krm_lengths_positions(krm_ctx* ctx, krm_buf lengths, krm_buf positions_i32,
                              uint32_t rows);
/* history[lengths.reserved++] = token[0] (when in range): keeps the tokens of a replayed
 * greedy loop on the device until the host reads them in one go, instead of one read-back per
 * step (packages/models/src/generation/greedy.ts:245-252 reads back every step). */
int32_t krm_lengths_log_token(krm_ctx* ctx, krm_buf lengths, krm_buf token_i32,
                              krm_buf history_i32, uint32_t history_len);
/* krm_lengths_log_token, krm_lengths_advance and krm_lengths_positions (one row) in one launch:
 * the end of a recorded one-row decode step, which leaves the next step's position behind. */
int32_t krm_lengths_step_end(krm_ctx* ctx, krm_buf lengths, krm_buf token_i32,
                             krm_buf history_i32, uint32_t history_len, krm_buf positions_i32);
/* The exit of a one-row decode step in two launches instead of four (final rms_norm + lm_head
 * `linear`, `argmax`, the step's bookkeeping, the next step's `embedding`; graph order
 * tools/export-recipes/minicpm5/export_decode.py:14-35, loop
 * packages/models/src/generation/greedy.ts:245-252).
 * krm_decode_head: krm_linear_i4_fused for one row (optional rms_norm in front, logits [n]
 * written in full) whose workgroups also leave the argmax of the rows they stored in
 * `partials` ({f32 value bits, u32 row} pairs, 8 bytes per 4 rows of n at most);
 * *partial_count = how many pairs this launch writes (a function of the shape only).
 * krm_decode_tail: the argmax over those pairs with krm_argmax's order (NaN is the maximum,
 * ties go to the smallest index), then krm_lengths_step_end (token written to token_i32 and
 * logged, lengths advanced, next position written) and krm_embedding of that token into
 * `next_row` [hidden], in one launch.  The token equals krm_argmax of the logits bit for bit. */
int32_t krm_decode_head(krm_ctx* ctx, krm_buf x, krm_buf norm_weight_f32, float norm_eps,
                        krm_buf w, krm_buf scales, krm_buf bias, krm_buf logits, krm_buf partials,
                        size_t partials_bytes, uint32_t* partial_count, uint32_t n, uint32_t k,
                        uint32_t group, int32_t io_dtype, int32_t scale_dtype);
int32_t krm_decode_tail(krm_ctx* ctx, krm_buf partials, uint32_t partial_count, krm_buf token_i32,
                        krm_buf lengths, krm_buf history_i32, uint32_t history_len,
                        krm_buf positions_i32, krm_buf table, uint32_t vocab, uint32_t hidden,
                        krm_buf next_row, int32_t table_dtype, int32_t out_dtype);
/* krm_attention_state with device lengths; `max_past` sizes the launch and the workspace.  A
 * replay whose device-side pastLength needs more column splits than `max_past` did raises the
 * fault word and writes nothing (neither `out` nor the workspace nor the arrival counters). */
int32_t krm_attention_state_lengths(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                                    krm_buf slot_k, krm_buf slot_v, krm_buf out, uint32_t batch,
                                    uint32_t heads, uint32_t kv_heads, uint32_t chunk_rows,
                                    uint32_t depth, uint32_t capacity, uint32_t window,
                                    float half_scale, krm_buf lengths, uint32_t max_past,
                                    int32_t io_dtype, int32_t kv_dtype, krm_buf workspace,
                                    size_t workspace_bytes);
/* krm_state_append with device lengths. */
int32_t krm_state_append_lengths(krm_ctx* ctx, krm_buf x, krm_buf slot, uint32_t kv_planes,
                                 uint32_t chunk_rows, uint32_t depth, uint32_t capacity,
                                 uint32_t window, krm_buf lengths, int32_t x_dtype,
                                 int32_t slot_dtype);

/* ---- ragged decode batch (no counterpart in the reference, which runs one sequence at a
 *      time: docs/decisions/0066-generation-context-state-slots.md:130-135) -----------------
 * `nseq` sequences, one query row each, packed along the slot's row axis:
 *   q      [nseq, H, D]            io_dtype
 *   ins_k  [nseq, Hkv, D]          io_dtype   this step's key per sequence
 *   ins_v  [nseq, Hkv, D]          io_dtype
 *   slot_k [Hkv, total_rows, D]    kv_dtype   sequence i owns rows [cu_seqlens[i], cu_seqlens[i+1])
 *   slot_v [Hkv, total_rows, D]    kv_dtype
 *   out    [nseq, H, D]            io_dtype
 * `cu_seqlens` is a HOST array of nseq+1 ascending row offsets (cu_seqlens[0] >= 0,
 * cu_seqlens[nseq] <= total_rows); sequence i has past_i = cu[i+1]-cu[i] rows in the slot and
 * attends to those plus its own ins row (window = 0).  Each sequence's result is
 * bit-identical to krm_attention_state run on that sequence alone. */
int32_t krm_attention_varlen_workspace(uint32_t nseq, uint32_t heads, uint32_t kv_heads,
                                       uint32_t depth, uint64_t total_rows, size_t* bytes);
int32_t krm_attention_varlen(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                             krm_buf slot_k, krm_buf slot_v, krm_buf out,
                             const int32_t* cu_seqlens, uint32_t nseq, uint32_t heads,
                             uint32_t kv_heads, uint32_t depth, uint64_t total_rows,
                             float half_scale, int32_t io_dtype, int32_t kv_dtype,
                             krm_buf workspace, size_t workspace_bytes);

/* The same ragged step with its tables built on the device, so that the whole step can be
 * recorded (krm_graph_*) and replayed while the sequences grow (no counterpart in the
 * reference, as above).  `cu_seqlens_i32` is a DEVICE array of nseq+1 row offsets.
 * krm_attention_varlen_plan turns it into the launch tables in `plan`
 * (krm_attention_varlen_plan_bytes bytes: cu_rows[nseq+1], split_prefix[nseq+1], fault); one
 * plan serves every layer of a step.  Offsets that are negative, not ascending, beyond
 * total_rows, or that need more than `max_splits` column splits set plan's fault word (the
 * last int32 of the tables, index 2*(nseq+1)) to 1 and make the attention launch a no-op.
 * krm_attention_varlen_planned launches `max_splits` column splits (the bound
 * krm_attention_varlen_max_splits returns: total_rows / split columns + nseq) and reads the
 * tables on the device; results are bit-identical to krm_attention_varlen and to
 * krm_attention_state on each sequence alone.  `workspace` as for krm_attention_varlen. */
int32_t krm_attention_varlen_plan_bytes(uint32_t nseq, size_t* bytes);
int32_t krm_attention_varlen_max_splits(uint32_t nseq, uint32_t depth, int32_t kv_dtype,
                                        uint64_t total_rows, uint32_t* max_splits);
int32_t krm_attention_varlen_plan(krm_ctx* ctx, krm_buf cu_seqlens_i32, krm_buf plan,
                                  uint32_t nseq, uint32_t depth, int32_t kv_dtype,
                                  uint64_t total_rows, uint32_t max_splits);
int32_t krm_attention_varlen_planned(krm_ctx* ctx, krm_buf q, krm_buf ins_k, krm_buf ins_v,
                                     krm_buf slot_k, krm_buf slot_v, krm_buf out, krm_buf plan,
                                     uint32_t nseq, uint32_t heads, uint32_t kv_heads,
                                     uint32_t depth, uint64_t total_rows, uint32_t max_splits,
                                     float half_scale, int32_t io_dtype, int32_t kv_dtype,
                                     krm_buf workspace, size_t workspace_bytes);

/* ---- decoder-layer glue ops (f32 arithmetic; activations f32 or fp16) ------------------------
 * The ops a Llama-style layer runs around the linears and the attention in the decode graph
 * (tools/export-recipes/minicpm5/export_decode.py:14-35).  Each one follows the reference
 * kernel of the same name. */

/* out[r, i] = x[r, i] * rsqrt(mean_i(x[r]^2) + eps) * weight[i]; weight is f32.
 * packages/runtime/src/kernels/rms-norm.ts:35-91 */
int32_t krm_rms_norm(krm_ctx* ctx, krm_buf x, krm_buf weight_f32, krm_buf out, uint32_t rows,
                     uint32_t dim, float eps, int32_t io_dtype);
/* The same with the result stored as out_dtype: io_dtype, or KRM_F16 for f32 rows (the f32
 * result rounded once — the copy a KRM_COMPUTE_F16 product reads through x_dtype; no
 * counterpart in the reference, which has no mixed-type activations). */
int32_t krm_rms_norm_cast(krm_ctx* ctx, krm_buf x, krm_buf weight_f32, krm_buf out, uint32_t rows,
                          uint32_t dim, float eps, int32_t io_dtype, int32_t out_dtype);
/* Half-split RoPE: out = x*cos[pos] + rotate_half(x)*sin[pos] with cos/sin rows [table_rows, D]
 * (f32) looked up by positions[row] (i32, device); both products are rounded before the add
 * (packages/runtime/src/kernels/rope.ts:5-20,52-80).  x is [rows, heads, D]; out is
 * [heads, rows, D] when to_head_major != 0 (what the attention reads), else [rows, heads, D].
 * A position outside the table yields NaN (the reference's out-of-range gather does too). */
int32_t krm_rope_half(krm_ctx* ctx, krm_buf x, krm_buf positions_i32, krm_buf cos_table_f32,
                      krm_buf sin_table_f32, krm_buf out, uint32_t rows, uint32_t heads,
                      uint32_t head_dim, uint32_t table_rows, int32_t to_head_major,
                      int32_t io_dtype);
/* One decode row in one launch: RoPE (as krm_rope_half) of the H + Hkv leading heads of the
 * [q; k; v] row `qkv` ([H + 2*Hkv, D], what a fused qkv linear writes) into qk_out
 * ([H + Hkv, D]), plus the state_append (as krm_state_append with M = Q = 1) of the roped k row
 * into slot_k and of the v row into slot_v.  `lengths` == 0: `past` is this run's pastLength;
 * otherwise it is read on the device (and a violated run contract sets the fault word and
 * appends nothing).  May be issued BEFORE the attention of the same step: a one-row step's
 * attention never reads the slot row this writes.
 * Fuses packages/runtime/src/kernels/rope.ts:5-20,52-80 and
 * packages/runtime/src/kernels/state-append.ts:47-96. */
int32_t krm_decode_rope_append(krm_ctx* ctx, krm_buf qkv, krm_buf positions_i32,
                               krm_buf cos_table_f32, krm_buf sin_table_f32, krm_buf qk_out,
                               krm_buf slot_k, krm_buf slot_v, uint32_t heads, uint32_t kv_heads,
                               uint32_t depth, uint32_t table_rows, uint32_t capacity,
                               uint32_t window, uint32_t past, krm_buf lengths, int32_t io_dtype,
                               int32_t kv_dtype);
/* A whole decode row's attention inputs in one launch: (optional rms_norm) -> the fused
 * [q; k; v] projection (n = (H + 2*Hkv) * D rows, M = 1) -> half-split RoPE of q and k ->
 * state_append of the roped k row and of the v row.  `out` receives [q_rot; k_rot; v] as
 * [H + 2*Hkv, D].  The weight (and bias) rows of the q and k sections must be interleaved per
 * head as (0, D/2, 1, D/2 + 1, ...), so that one lane finishes both halves of a rotation pair;
 * the v section keeps its natural order.  Roundings are those of the separate ops
 * (krm_linear_i4_fused, krm_rope_half, krm_state_append); `lengths` / `past` as in
 * krm_decode_rope_append, and like it this may precede the step's attention.
 * kv_heads = 0 with both slots 0: a layer that attends over another layer's K / V (KV-sharing
 * layers, tools/export-recipes/gemma4/export_decode.py:59-70) projects and rotates q alone,
 * `out` = [q_rot], and nothing is appended.
 * Fuses packages/runtime/src/kernels/linear.ts:34-64, packages/runtime/src/kernels/rope.ts:5-20,
 * 52-80 and packages/runtime/src/kernels/state-append.ts:47-96. */
int32_t krm_decode_qkv(krm_ctx* ctx, krm_buf x, krm_buf norm_weight_f32, float norm_eps,
                       krm_buf w, krm_buf scales, krm_buf bias, krm_buf positions_i32,
                       krm_buf cos_table_f32, krm_buf sin_table_f32, krm_buf out, krm_buf slot_k,
                       krm_buf slot_v, uint32_t heads, uint32_t kv_heads, uint32_t depth,
                       uint32_t k, uint32_t group, uint32_t table_rows, uint32_t capacity,
                       uint32_t window, uint32_t past, krm_buf lengths, int32_t io_dtype,
                       int32_t scale_dtype, int32_t kv_dtype);
/* The attention inputs of a chunk of m rows in one launch: the fused [q; k; v] projection
 * (weights laid out as for krm_decode_qkv: q and k rows interleaved per head as
 * (0, D/2, 1, D/2 + 1, ...), v natural; arithmetic of krm_linear_i4_rows), each value rounded
 * to io_dtype as a separate linear would store it, half-split RoPE of q and k by
 * positions[row] (roundings of krm_rope_half; a position outside the table gives NaN), and the
 * head-major layouts the attention reads:
 *   q_out [H, m, D]   k_out [Hkv, m, D]   v_out [Hkv, m, D]      (io_dtype)
 * The state appends stay separate calls (after the attention, as docs/ir-v1.md:345-348 orders
 * them).  Same coverage limits and the same x_dtype rule as krm_linear_i4_rows.
 * Fuses packages/runtime/src/kernels/linear.ts:34-64, packages/runtime/src/kernels/rope.ts:5-20,
 * 52-80 and the permute nodes of tools/export-recipes/minicpm5/export_decode.py:14-35. */
int32_t krm_prefill_qkv(krm_ctx* ctx, krm_buf x, krm_buf w, krm_buf scales, krm_buf bias,
                        krm_buf positions_i32, krm_buf cos_table_f32, krm_buf sin_table_f32,
                        krm_buf q_out, krm_buf k_out, krm_buf v_out, uint32_t m, uint32_t heads,
                        uint32_t kv_heads, uint32_t depth, uint32_t k, uint32_t group,
                        uint32_t table_rows, int32_t io_dtype, int32_t scale_dtype,
                        int32_t compute, int32_t x_dtype);
/* ---- w4a8: `linear` with int4 weights on integer dot products (the reference's opt-in
 *      SessionOptions.linearCompute "i8a8" with int4-resident weights,
 *      packages/runtime/src/runtime/recipe-builder.ts:1320-1341,1407-1488;
 *      contract docs/decisions/0076-w4a8-linear-execution.md:40-60) --------------------------
 * Step 1, the activation quantiser (params {rows, dim} + bindings x, xq, xs:
 * packages/runtime/src/kernels/quantize-rows.ts:89-146):
 *   xs[row] = max(f32(max|x[row, :]| * f32(1/127)), f32 tiny); a NaN in the row makes it NaN
 *   xq[row, i] = clamp(round-half-even(x[row, i] / xs[row]), -127, 127), int8, row-major
 * x / xs is the correctly rounded division (the reference's WGSL division is not, and its
 * codes may differ by one next to a tie; these never do).  A NaN quotient stores 0.
 * Requires dim >= 1 and dim % 4 == 0 (quantize-rows.ts:160-173), x 16-byte aligned. */
int32_t krm_quantize_rows(krm_ctx* ctx, krm_buf x_f32, krm_buf xq_i8, krm_buf xs_f32,
                          uint32_t rows, uint32_t dim);
/* Step 2, the product (params {m, n, k} + bindings xq, w, bias, out, scales, xs:
 * packages/runtime/src/kernels/linear-i8a8.ts:47-72,376-510,589-625):
 *   accf = 0; for each group gi ascending: accf = fma(f32(sum_group xq * wq), scales[col, gi], accf)
 *   out[row, col] = fma(accf, xs[row], bias[col])
 * the group sums are exact int32, every fma is fused and correctly rounded, so the result is
 * bit-identical to packages/runtime/src/reference/i8a8.ts:209-231 evaluated with a fused
 * multiply-add, for every tiling.
 *   xq [m, k] int8, xs [m] f32 (from krm_quantize_rows), w [n, k] packed int4,
 *   scales [n, k/group] scale_dtype, bias [n] f32 or 0 (= zeros), out [m, n] f32.
 * Requires k > 0, k % 4 == 0 (recipe-builder.ts:1336-1338), group a power of two >= 16
 * dividing k, group <= 2113664 (the int32 gate LINEAR_W4A8_MAX_GROUP, linear-i8a8.ts:124-132). */
int32_t krm_linear_w4a8(krm_ctx* ctx, krm_buf xq_i8, krm_buf xs_f32, krm_buf w, krm_buf scales,
                        krm_buf bias_f32, krm_buf out_f32, uint32_t m, uint32_t n, uint32_t k,
                        uint32_t group, int32_t scale_dtype);
/* Steps 1 and 2 behind one call for f32 activations x [m, k] (the reference's builder emits
 * the pair back to back with node-local xq / xs, recipe-builder.ts:1407-1488): the same result
 * bit for bit.  For up to 8 rows with 32 <= group <= 2048 and rows-per-block * k <= 16384
 * (blocks of 1, 2 or 4 rows: m = 1 up to k = 16384, m <= 2 up to 8192, else 4096) it is ONE
 * launch — every workgroup quantises the block of x rows it multiplies, in LDS, while its
 * weights are on their way — and xq / xs are not touched (0 is allowed).  Every other shape runs
 * krm_quantize_rows + krm_linear_w4a8 through xq [m, k] int8 and xs [m] f32, which must then be
 * given.  Argument rules are those of the two steps. */
int32_t krm_linear_w4a8_fused(krm_ctx* ctx, krm_buf x_f32, krm_buf xq_i8, krm_buf xs_f32,
                              krm_buf w, krm_buf scales, krm_buf bias_f32, krm_buf out_f32,
                              uint32_t m, uint32_t n, uint32_t k, uint32_t group,
                              int32_t scale_dtype);
/* [a, b, d] -> [b, a, d] (the reshape + permute between linears and attention). */
int32_t krm_transpose_01(krm_ctx* ctx, krm_buf x, krm_buf out, uint32_t a, uint32_t b, uint32_t d,
                         int32_t io_dtype);
/* out = (gate * sigmoid(gate)) * up, the sigmoid and both products rounded to f32 in turn
 * (packages/runtime/src/kernels/silu.ts:47-93). */
int32_t krm_silu_mul(krm_ctx* ctx, krm_buf gate, krm_buf up, krm_buf out, uint64_t count,
                     int32_t io_dtype);
/* out = a + b (packages/runtime/src/codegen/elementwise.ts). */
int32_t krm_add(krm_ctx* ctx, krm_buf a, krm_buf b, krm_buf out, uint64_t count,
                int32_t io_dtype);
/* out[r, :] = table[index[r], :]; an index outside [0, vocab) fills the row with NaN, it is
 * never clamped (packages/runtime/src/kernels/embedding.ts:1-43). */
int32_t krm_embedding(krm_ctx* ctx, krm_buf table, krm_buf index_i32, krm_buf out, uint32_t rows,
                      uint32_t vocab, uint32_t hidden, int32_t table_dtype, int32_t out_dtype);
/* out[r] = argmax_i x[r, i]: ties -> smallest index, NaN is the maximum, all -inf -> 0
 * (packages/runtime/src/kernels/argmax.ts:16-34). */
int32_t krm_argmax(krm_ctx* ctx, krm_buf x, krm_buf out_i32, uint32_t rows, uint32_t dim,
                   int32_t io_dtype);

/* ==== DIAGNOSTICS ============================================================================
 * Not ops of the runtime: measurement probes that bench.py uses to state what a launch and a
 * read of a given size cost on this machine.  A host binds them only if it wants those floors
 * (include/karume_hip.ffi.ts lists them in a table of their own, KARUME_HIP_DIAGNOSTIC_SYMBOLS).
 * ============================================================================================ */
/* Measurement floors for a launch of `grid` workgroups of `block` threads on the context's
 * stream (diagnostics like the timestamp queries above; no op of the reference):
 *   KRM_PROBE_EMPTY — a kernel that does nothing (what a launch of that grid costs);
 *   KRM_PROBE_READ  — every thread streams its share of `bytes` at `src` with 16-byte loads
 *                     and stores nothing (what reading that much costs); up to eight loads a
 *                     thread are requested before any is used, so a grid that covers `bytes`
 *                     in one pass pays one memory round trip. */
#define KRM_PROBE_EMPTY 0
#define KRM_PROBE_READ 1
int32_t krm_probe_launch(krm_ctx* ctx, int32_t kind, krm_buf src, size_t bytes, uint32_t grid,
                         uint32_t block);

/* What an all-to-all hand-over of a vector of `entries` floats (2048, 4096 or 8192) costs
 * between the 256 workgroups of ONE persistent launch, `phases` times in a row: flags polled
 * and the vector read with agent-scope loads, results written with agent-scope stores (the
 * step a single-launch decode would pay at every op boundary).  `work` is scratch of at least
 * 2 * entries * 4 + 1040 bytes that the call clears; its last word written (offset
 * 2 * entries * 4 + 1024) is a fault flag: 1 if a poll exceeded `spin_limit` rounds (every wait
 * is bounded; the launch always ends).  Time it with events; no op of the reference. */
int32_t krm_probe_exchange(krm_ctx* ctx, krm_buf work, size_t work_bytes, uint32_t entries,
                           uint32_t phases, uint32_t spin_limit);
/* `count` launches of krm_linear_i4 (m rows, m <= 16) in a row from one call, launch i on the
 * weights w_list[i % copies] / scales_list[i % copies] (host arrays of `copies` device
 * addresses): what a host loop of krm_linear_i4 calls does, without the host's time per call
 * between the launches, so that a kernel trace of plain launches sees them back to back the way
 * a recorded run replays them.  Rejected while recording. */
int32_t krm_probe_linear_series(krm_ctx* ctx, krm_buf x, const krm_buf* w_list,
                                const krm_buf* scales_list, uint32_t copies, krm_buf out,
                                uint32_t count, uint32_t m, uint32_t n, uint32_t k,
                                uint32_t group, int32_t io_dtype, int32_t scale_dtype);

#ifdef __cplusplus
}
#endif
#endif /* KARUME_HIP_H */
