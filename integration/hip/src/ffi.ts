/**
 * bun:ffi binding of libalpha_hip.so: one entry per declaration of include/alpha_hip.h.
 *
 * The symbol table and the struct layouts below are written by ../gen_ffi_table.py from the ctypes table the parity
 * tests call through; a CPU test parses this file and compares names, argument counts, argument and return types and
 * every struct offset with that table and with the header.
 *
 * Replaces the N-API addon seam of the Vulkan backend (packages/helios/src/device.ts:17-39, export table
 * packages/helios/native/helios_vk.c:4403-4432).
 */
import { dlopen, FFIType, ptr as addressOf } from "bun:ffi";

const { i32, i64, u64, f32, f64, ptr, cstring } = FFIType;

export const lib = dlopen(process.env.ALPHA_HIP_LIB ?? "libalpha_hip.so", {
  // GENERATED SYMBOLS BEGIN
  ah_adafactor_2d:                 { args: [u64, u64, u64, u64, i64, i64, ptr], returns: i32 },
  ah_adafactor_flat:               { args: [u64, u64, u64, u64, ptr], returns: i32 },
  ah_adamw:                        { args: [u64, u64, u64, u64, u64, ptr, u64, u64, u64], returns: i32 },
  ah_adamw_list:                   { args: [ptr, i32, ptr, u64, u64], returns: i32 },
  ah_add_bf16:                     { args: [u64, u64, u64, u64], returns: i32 },
  ah_add_inplace:                  { args: [u64, u64, u64], returns: i32 },
  ah_alloc:                        { args: [u64, ptr], returns: i32 },
  ah_argmax:                       { args: [u64, u64, i64, i64, i64], returns: i32 },
  ah_axpy_inplace:                 { args: [u64, u64, f32, u64], returns: i32 },
  ah_binary:                       { args: [i32, u64, u64, u64, u64], returns: i32 },
  ah_binary_broadcast:             { args: [i32, u64, u64, u64, i32, ptr, ptr, ptr], returns: i32 },
  ah_broadcast:                    { args: [u64, u64, i32, ptr, ptr], returns: i32 },
  ah_cast:                         { args: [u64, i32, u64, i32, u64], returns: i32 },
  ah_cat_part:                     { args: [u64, u64, i32, ptr, ptr, i32, i64], returns: i32 },
  ah_causal_mask:                  { args: [u64, i64], returns: i32 },
  ah_channel_act:                  { args: [i32, u64, ptr, i32, u64, i64, i64], returns: i32 },
  ah_channel_act_bwd:              { args: [i32, u64, ptr, i32, u64, u64, ptr, i32, i64, i64], returns: i32 },
  ah_check_finite:                 { args: [u64, u64, u64], returns: i32 },
  ah_clip_coef:                    { args: [u64, f32, f32, u64], returns: i32 },
  ah_copy:                         { args: [u64, u64, u64], returns: i32 },
  ah_cross_entropy:                { args: [u64, i32, u64, u64, u64, i64, i64], returns: i32 },
  ah_cross_entropy_bwd:            { args: [u64, i32, u64, u64, u64, f32, u64, i64, i64], returns: i32 },
  ah_cross_entropy_fwd_bwd:        { args: [u64, i32, u64, u64, u64, u64, f32, u64, i64, i64], returns: i32 },
  ah_device_info:                  { args: [ptr], returns: i32 },
  ah_download:                     { args: [ptr, u64, u64], returns: i32 },
  ah_download_begin:               { args: [u64, u64, ptr], returns: i32 },
  ah_download_end:                 { args: [u64, ptr, u64], returns: i32 },
  ah_dropout_apply:                { args: [u64, i32, u64, u64, i32, u64, u64, i32, f64], returns: i32 },
  ah_dropout_mask:                 { args: [u64, u64, i32, i32, f64], returns: i32 },
  ah_embedding:                    { args: [u64, u64, u64, i64, i64, i64, i32], returns: i32 },
  ah_embedding_bwd:                { args: [u64, u64, u64, i64, i64, i64, i32], returns: i32 },
  ah_embedding_bwd_indexed:        { args: [u64, u64, u64, i64, i64, i64, i32], returns: i32 },
  ah_embedding_index:              { args: [u64, i64, i64, u64], returns: i32 },
  ah_embedding_index_bytes:        { args: [i64, i64], returns: i64 },
  ah_embedding_tok_pos:            { args: [u64, u64, u64, u64, i64, i64, i64, i64, i32], returns: i32 },
  ah_event_create:                 { args: [ptr], returns: i32 },
  ah_event_destroy:                { args: [u64], returns: i32 },
  ah_event_elapsed_ms:             { args: [u64, u64, ptr], returns: i32 },
  ah_event_record:                 { args: [u64], returns: i32 },
  ah_fill_f32:                     { args: [u64, f32, u64], returns: i32 },
  ah_fill_i32:                     { args: [u64, i32, u64], returns: i32 },
  ah_flash_bwd:                    { args: [ptr], returns: i32 },
  ah_flash_fwd:                    { args: [ptr], returns: i32 },
  ah_free:                         { args: [u64], returns: i32 },
  ah_gemm:                         { args: [ptr], returns: i32 },
  ah_gemm_grouped_destroy:         { args: [u64], returns: i32 },
  ah_gemm_grouped_plan:            { args: [ptr, i32, ptr], returns: i32 },
  ah_gemm_grouped_run:             { args: [u64, i32], returns: i32 },
  ah_gemm_grouped_run_sumsq:       { args: [u64, i32, u64], returns: i32 },
  ah_gemm_grouped_update:          { args: [u64, ptr, i32], returns: i32 },
  ah_gemm_last_kernel:             { args: [ptr, i32, ptr], returns: i32 },
  ah_gemm_planes:                  { args: [ptr, i64, i64, i64, i64, i32], returns: i32 },
  ah_graph_begin:                  { args: [], returns: i32 },
  ah_graph_destroy:                { args: [u64], returns: i32 },
  ah_graph_end:                    { args: [ptr], returns: i32 },
  ah_graph_launch:                 { args: [u64], returns: i32 },
  ah_init:                         { args: [i32], returns: i32 },
  ah_last_error:                   { args: [], returns: cstring },
  ah_layernorm:                    { args: [u64, u64, u64, u64, i64, i64, f32, i32, i32], returns: i32 },
  ah_layernorm_bwd:                { args: [u64, u64, u64, i32, u64, u64, u64, u64, u64, i64, i64, f32, i32, i32], returns: i32 },
  ah_layernorm_bwd_deferred:       { args: [u64, u64, u64, i32, u64, u64, u64, u64, i64, i64, f32, i32], returns: i32 },
  ah_layernorm_bwd_partials_bytes: { args: [i64, i64], returns: i64 },
  ah_layernorm_colsums:            { args: [ptr, i32], returns: i32 },
  ah_lion:                         { args: [u64, u64, u64, u64, ptr], returns: i32 },
  ah_masked_fill:                  { args: [u64, u64, u64, u64, u64, f32], returns: i32 },
  ah_pos_embedding_bwd:            { args: [u64, u64, i64, i64, i64, i32], returns: i32 },
  ah_probe_issue:                  { args: [i32, i32, i32, ptr], returns: i32 },
  ah_probe_mfma_bf16:              { args: [i32, i32, i32, ptr], returns: i32 },
  ah_reset_op_count:               { args: [], returns: i32 },
  ah_residual_dropout_add:         { args: [u64, u64, u64, u64, u64], returns: i32 },
  ah_rng_fill_gauss_f32:           { args: [ptr, ptr, u64, f64], returns: i32 },
  ah_rng_fill_uniform_f64:         { args: [ptr, ptr, u64], returns: i32 },
  ah_rng_next:                     { args: [ptr, ptr], returns: i32 },
  ah_rng_next_gauss:               { args: [ptr, ptr], returns: i32 },
  ah_rng_seed:                     { args: [ptr, i32], returns: i32 },
  ah_scale_inplace:                { args: [u64, f32, u64], returns: i32 },
  ah_scatter_slice:                { args: [u64, u64, i32, ptr, ptr, ptr], returns: i32 },
  ah_sgd:                          { args: [u64, u64, u64, f64, f64], returns: i32 },
  ah_shutdown:                     { args: [], returns: i32 },
  ah_side_begin:                   { args: [], returns: i32 },
  ah_side_end:                     { args: [], returns: i32 },
  ah_side_join:                    { args: [], returns: i32 },
  ah_silu_mul:                     { args: [u64, u64, u64, u64], returns: i32 },
  ah_silu_mul_bwd:                 { args: [u64, u64, u64, u64, u64, u64], returns: i32 },
  ah_slice:                        { args: [u64, u64, i32, ptr, ptr, ptr], returns: i32 },
  ah_slice_qkv:                    { args: [u64, u64, u64, u64, i64, i64], returns: i32 },
  ah_softmax:                      { args: [u64, u64, i64, i64, i64, i32], returns: i32 },
  ah_softmax_bwd:                  { args: [u64, u64, u64, i64, i64], returns: i32 },
  ah_stats:                        { args: [ptr], returns: i32 },
  ah_step_begin:                   { args: [u64], returns: i32 },
  ah_step_end:                     { args: [ptr], returns: i32 },
  ah_step_guard:                   { args: [u64, u64, f32, f32, f64, f64, u64, u64, u64], returns: i32 },
  ah_step_kick:                    { args: [], returns: i32 },
  ah_step_note:                    { args: [], returns: cstring },
  ah_step_reset:                   { args: [u64], returns: i32 },
  ah_sum_all:                      { args: [u64, u64, u64, i32], returns: i32 },
  ah_sum_axis:                     { args: [u64, u64, i64, i64, i64, i32], returns: i32 },
  ah_sum_sq:                       { args: [u64, u64, u64], returns: i32 },
  ah_sum_sq_list:                  { args: [ptr, ptr, i32, u64], returns: i32 },
  ah_sum_sq_static:                { args: [u64, u64, u64], returns: i32 },
  ah_swiglu:                       { args: [i32, u64, u64, i64, i64], returns: i32 },
  ah_swiglu_bwd:                   { args: [i32, u64, u64, u64, i64, i64], returns: i32 },
  ah_sync:                         { args: [], returns: i32 },
  ah_token_windows:                { args: [u64, i64, u64, i64, i64, u64, u64], returns: i32 },
  ah_transpose:                    { args: [u64, u64, i32, ptr, i32, i32], returns: i32 },
  ah_trim_pool:                    { args: [], returns: i32 },
  ah_unary:                        { args: [i32, u64, u64, u64, f32, f32], returns: i32 },
  ah_unary_bwd:                    { args: [i32, u64, u64, u64, u64, f32, f32], returns: i32 },
  ah_upload:                       { args: [u64, ptr, u64], returns: i32 },
  // GENERATED SYMBOLS END
}).symbols;

/** Byte offsets of the plain structs of include/alpha_hip.h (natural C alignment, little endian). */
export const LAYOUT = {
  // GENERATED LAYOUTS BEGIN
  AhGemm: { size: 128, layout: 0, in_dtype: 4, out_dtype: 8, epilogue: 12, m: 16, n: 24, k: 32, lda: 40, ldb: 48, ldc: 56, batch: 64, stride_a: 72, stride_b: 80, stride_c: 88, a: 96, b: 104, c: 112, aux: 120 },
  AhFlash: { size: 208, dtype: 0, batch: 4, heads: 8, seq: 12, head_dim: 16, q_sb: 24, q_sh: 32, q_st: 40, k_sb: 48, k_sh: 56, k_st: 64, v_sb: 72, v_sh: 80, v_st: 88, o_sb: 96, o_sh: 104, o_st: 112, scale: 120, soft_cap: 124, q: 128, k: 136, v: 144, o: 152, lse: 160, d_o: 168, dq: 176, dk: 184, dv: 192, bwd_variant: 200, reserved: 204 },
  AhAdamW: { size: 32, lr: 0, beta1: 4, beta2: 8, eps: 12, weight_decay: 16, bc1: 20, bc2: 24, grad_scale: 28 },
  AhAdamWItem: { size: 56, p: 0, g: 8, m: 16, v: 24, shadow: 32, n: 40, weight_decay: 48, reserved: 52 },
  AhStats: { size: 88, live_allocs: 0, live_bytes: 8, pool_blocks: 16, pool_bytes: 24, device_mallocs: 32, ops_launched: 40, graphs_live: 48, steps_recorded: 56, steps_replayed: 64, steps_fallback: 72, step_node_updates: 80 },
  AhDeviceInfo: { size: 184, name: 0, arch: 128, compute_units: 160, wavefront: 164, clock_khz: 168, lds_bytes_per_block: 172, hbm_bytes: 176 },
  AhColsumJob: { size: 48, partials: 0, dw: 8, db: 16, rows: 24, dim: 32, accumulate: 40, reserved: 44 },
  AhLion: { size: 40, lr: 0, beta1: 8, beta2: 16, weight_decay: 24, grad_scale: 32 },
  AhAdafactor: { size: 48, lr: 0, beta2: 8, eps: 16, clip_threshold: 24, weight_decay: 32, grad_scale: 40 },
  AhRng: { size: 24, s0: 0, s1: 4, has_spare: 8, _pad: 12, spare: 16 },
  // GENERATED LAYOUTS END
} as const;

export const enum Dt { F32 = 0, BF16 = 1, I32 = 2, F16 = 3 }
export const enum Bin { ADD = 0, SUB = 1, MUL = 2, DIV = 3 }
export const enum Un { NEG = 0, EXP, LOG, SQRT, POW, SCALE, CLAMP, GELU, RELU, SILU, SOFTCAP }
export const enum UnBwd { GELU = 0, RELU, SILU, CLAMP, SOFTCAP }
export const enum Layout { NN = 0, NT = 1, TN = 2 }
export const enum Epi { NONE = 0, ACCUM, GELU, RESIDUAL, GELU_BWD, GELU_GRAD, MUL_AUX }

/** Every export returns a status; a non-zero one becomes a thrown Error with the library's message, which is where the
 *  reference's backends throw (packages/tensor/src/cpu_ref.ts:172-182). */
export function check(rc: number): void {
  if (rc !== 0) throw new Error(`alpha_hip error ${rc}: ${lib.ah_last_error()}`);
}

/** A reusable little-endian struct buffer; `p` is what an FFI call takes for a `const AhX *`. */
export class Struct<K extends keyof typeof LAYOUT> {
  readonly bytes: ArrayBuffer;
  readonly view: DataView;
  readonly p: ReturnType<typeof addressOf>;
  constructor(readonly kind: K, count = 1) {
    this.bytes = new ArrayBuffer(LAYOUT[kind].size * count);
    this.view = new DataView(this.bytes);
    this.p = addressOf(this.bytes);
  }
  private at(field: string, index: number): number {
    return LAYOUT[this.kind].size * index + (LAYOUT[this.kind] as Record<string, number>)[field];
  }
  i32(field: string, v: number, index = 0): this { this.view.setInt32(this.at(field, index), v, true); return this; }
  f32(field: string, v: number, index = 0): this { this.view.setFloat32(this.at(field, index), v, true); return this; }
  f64(field: string, v: number, index = 0): this { this.view.setFloat64(this.at(field, index), v, true); return this; }
  i64(field: string, v: number | bigint, index = 0): this { this.view.setBigInt64(this.at(field, index), BigInt(v), true); return this; }
  u64(field: string, v: number | bigint, index = 0): this { this.view.setBigUint64(this.at(field, index), BigInt(v), true); return this; }
  getU64(field: string, index = 0): bigint { return this.view.getBigUint64(this.at(field, index), true); }
  getI32(field: string, index = 0): number { return this.view.getInt32(this.at(field, index), true); }
  getString(field: string, max: number): string {
    const raw = new Uint8Array(this.bytes, this.at(field, 0), max);
    const end = raw.indexOf(0);
    return new TextDecoder().decode(raw.subarray(0, end < 0 ? max : end));
  }
}

/** int64 arrays (shapes, strides, starts) as the `const int64_t *` arguments want them. */
export function i64s(values: readonly number[]): BigInt64Array {
  const a = new BigInt64Array(Math.max(1, values.length));
  values.forEach((v, i) => (a[i] = BigInt(v)));
  return a;
}

export { addressOf };
