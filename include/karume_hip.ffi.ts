// Deno FFI symbol table of libkarume_hip.so: one entry per function declared in
// include/karume_hip.h, in the header's order.  Device addresses (krm_buf) are u64 (bigint on
// the Deno side), opaque handles (krm_ctx*, krm_event*, krm_graph*, hipStream_t) are
// "pointer", host arrays and out-parameters are TypedArrays ("buffer"), every status is i32.
//
//   const lib = Deno.dlopen("karume_amd/lib/libkarume_hip.so", KARUME_HIP_SYMBOLS);
//
// tests/test_ffi_table.py checks this table against the header (names, arity, types).

export const KARUME_HIP_SYMBOLS = {
  krm_ctx_create: { parameters: ["i32", "buffer"], result: "i32" },
  krm_ctx_create_on_stream: { parameters: ["i32", "pointer", "buffer"], result: "i32" },
  krm_ctx_destroy: { parameters: ["pointer"], result: "i32" },
  krm_last_error: { parameters: ["pointer"], result: "pointer" },
  krm_sync: { parameters: ["pointer"], result: "i32" },
  krm_version: { parameters: [], result: "pointer" },
  krm_buf_alloc: { parameters: ["pointer", "usize", "buffer"], result: "i32" },
  krm_buf_free: { parameters: ["pointer", "u64"], result: "i32" },
  krm_buf_upload: { parameters: ["pointer", "u64", "usize", "buffer", "usize"], result: "i32" },
  krm_buf_download: { parameters: ["pointer", "u64", "usize", "buffer", "usize"], result: "i32" },
  krm_buf_zero: { parameters: ["pointer", "u64", "usize", "usize"], result: "i32" },
  krm_buf_copy: { parameters: ["pointer", "u64", "u64", "usize"], result: "i32" },
  krm_event_create: { parameters: ["pointer", "buffer"], result: "i32" },
  krm_event_record: { parameters: ["pointer", "pointer"], result: "i32" },
  krm_event_elapsed_ms: { parameters: ["pointer", "pointer", "pointer", "buffer"], result: "i32" },
  krm_event_destroy: { parameters: ["pointer", "pointer"], result: "i32" },
  krm_graph_begin: { parameters: ["pointer"], result: "i32" },
  krm_graph_branch: { parameters: ["pointer", "u32"], result: "i32" },
  krm_graph_end: { parameters: ["pointer", "buffer"], result: "i32" },
  krm_graph_launch: { parameters: ["pointer", "pointer"], result: "i32" },
  krm_graph_destroy: { parameters: ["pointer", "pointer"], result: "i32" },
  krm_dequant_i4: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u32", "i32"
    ],
    result: "i32",
  },
  krm_linear_i4: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32", "i32", "i32",
      "i32"
    ],
    result: "i32",
  },
  krm_linear_i4_fused: {
    parameters: [
      "pointer", "u64", "u64", "f32", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32",
      "u32", "i32", "i32", "i32"
    ],
    result: "i32",
  },
  krm_linear_i4_rows: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32", "i32",
      "i32", "i32", "i32", "i32"
    ],
    result: "i32",
  },
  krm_attention_state_workspace: {
    parameters: [
      "u32", "u32", "u32", "u32", "u32", "u32", "u32", "u32", "buffer"
    ],
    result: "i32",
  },
  krm_attention_state: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32", "u32",
      "u32", "u32", "f32", "u32", "u32", "i32", "i32", "u64", "usize"
    ],
    result: "i32",
  },
  krm_attention_chunk: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32", "u32",
      "u32", "u32", "f32", "u32", "u32", "u64", "i32", "i32", "u32"
    ],
    result: "i32",
  },
  krm_attention_state_noalloc: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32", "u32",
      "u32", "u32", "f32", "u32", "u32", "i32", "i32"
    ],
    result: "i32",
  },
  krm_state_append: {
    parameters: [
      "pointer", "u64", "u64", "u32", "u32", "u32", "u32", "u32", "u32", "u32", "i32", "i32"
    ],
    result: "i32",
  },
  krm_lengths_set: { parameters: ["pointer", "u64", "u32", "u32"], result: "i32" },
  krm_lengths_advance: { parameters: ["pointer", "u64"], result: "i32" },
  krm_lengths_positions: { parameters: ["pointer", "u64", "u64", "u32"], result: "i32" },
  krm_lengths_log_token: { parameters: ["pointer", "u64", "u64", "u64", "u32"], result: "i32" },
  krm_lengths_step_end: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u32", "u64"
    ],
    result: "i32",
  },
  krm_decode_head: {
    parameters: [
      "pointer", "u64", "u64", "f32", "u64", "u64", "u64", "u64", "u64", "usize", "buffer", "u32",
      "u32", "u32", "i32", "i32"
    ],
    result: "i32",
  },
  krm_decode_tail: {
    parameters: [
      "pointer", "u64", "u32", "u64", "u64", "u64", "u32", "u64", "u64", "u32", "u32", "u64",
      "i32", "i32"
    ],
    result: "i32",
  },
  krm_attention_state_lengths: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32", "u32",
      "u32", "u32", "f32", "u64", "u32", "i32", "i32", "u64", "usize"
    ],
    result: "i32",
  },
  krm_state_append_lengths: {
    parameters: [
      "pointer", "u64", "u64", "u32", "u32", "u32", "u32", "u32", "u64", "i32", "i32"
    ],
    result: "i32",
  },
  krm_attention_varlen_workspace: {
    parameters: [
      "u32", "u32", "u32", "u32", "u64", "buffer"
    ],
    result: "i32",
  },
  krm_attention_varlen: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "buffer", "u32", "u32", "u32",
      "u32", "u64", "f32", "i32", "i32", "u64", "usize"
    ],
    result: "i32",
  },
  krm_attention_varlen_plan_bytes: { parameters: ["u32", "buffer"], result: "i32" },
  krm_attention_varlen_max_splits: {
    parameters: [
      "u32", "u32", "i32", "u64", "buffer"
    ],
    result: "i32",
  },
  krm_attention_varlen_plan: {
    parameters: [
      "pointer", "u64", "u64", "u32", "u32", "i32", "u64", "u32"
    ],
    result: "i32",
  },
  krm_attention_varlen_planned: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32",
      "u64", "u32", "f32", "i32", "i32", "u64", "usize"
    ],
    result: "i32",
  },
  krm_rms_norm: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u32", "u32", "f32", "i32"
    ],
    result: "i32",
  },
  krm_rms_norm_cast: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u32", "u32", "f32", "i32", "i32"
    ],
    result: "i32",
  },
  krm_rope_half: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32", "i32", "i32"
    ],
    result: "i32",
  },
  krm_decode_rope_append: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32",
      "u32", "u32", "u32", "u64", "i32", "i32"
    ],
    result: "i32",
  },
  krm_prefill_qkv: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u64", "u64", "u64", "u64", "u32",
      "u32", "u32", "u32", "u32", "u32", "u32", "i32", "i32", "i32", "i32"
    ],
    result: "i32",
  },
  krm_decode_qkv: {
    parameters: [
      "pointer", "u64", "u64", "f32", "u64", "u64", "u64", "u64", "u64", "u64", "u64", "u64",
      "u64", "u32", "u32", "u32", "u32", "u32", "u32", "u32", "u32", "u32", "u64", "i32",
      "i32", "i32"
    ],
    result: "i32",
  },
  krm_quantize_rows: { parameters: ["pointer", "u64", "u64", "u64", "u32", "u32"], result: "i32" },
  krm_linear_w4a8: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32", "i32"
    ],
    result: "i32",
  },
  krm_linear_w4a8_fused: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u64", "u64", "u64", "u64", "u32", "u32", "u32", "u32", "i32"
    ],
    result: "i32",
  },
  krm_transpose_01: {
    parameters: [
      "pointer", "u64", "u64", "u32", "u32", "u32", "i32"
    ],
    result: "i32",
  },
  krm_silu_mul: { parameters: ["pointer", "u64", "u64", "u64", "u64", "i32"], result: "i32" },
  krm_add: { parameters: ["pointer", "u64", "u64", "u64", "u64", "i32"], result: "i32" },
  krm_embedding: {
    parameters: [
      "pointer", "u64", "u64", "u64", "u32", "u32", "u32", "i32", "i32"
    ],
    result: "i32",
  },
  krm_argmax: { parameters: ["pointer", "u64", "u64", "u32", "u32", "i32"], result: "i32" },
} as const;

export type KarumeHipLibrary = Deno.DynamicLibrary<typeof KARUME_HIP_SYMBOLS>;

// Measurement probes (the DIAGNOSTICS section of the header): not ops of the runtime; bind them
// only to reproduce bench.py's launch and read floors.
export const KARUME_HIP_DIAGNOSTIC_SYMBOLS = {
  krm_probe_launch: { parameters: ["pointer", "i32", "u64", "usize", "u32", "u32"], result: "i32" },
  krm_probe_exchange: {
    parameters: [
      "pointer", "u64", "usize", "u32", "u32", "u32"
    ],
    result: "i32",
  },
  krm_probe_linear_series: {
    parameters: [
      "pointer", "u64", "buffer", "buffer", "u32", "u64", "u32", "u32", "u32", "u32", "u32", "i32",
      "i32"
    ],
    result: "i32",
  },
} as const;
