// Shared between the GEMM translation units: argument block and the fused epilogues.
#pragma once
#include "common.h"

namespace ah {

// One problem of a grouped launch (device-resident table; see ah_gemm_grouped_plan).
struct GemmGroupEntry {
  const void *a, *b;
  void *c;
  int M, N, K, tile_start;      // tile_start: first block id of this problem
  int64_t lda, ldb, ldc;
};

// Records which kernel ah_gemm launched last (read back by ah_gemm_last_kernel).
void note_gemm_kernel(const char *fmt, ...);
void note_gemm_split(int nsplit);

struct GemmArgs {
  const void *a, *b;
  void *c;
  const void *aux;     // EPI_RESIDUAL: f32 [M,N]; EPI_GELU_BWD: pre-activation (C dtype)
  void *aux_out;       // EPI_GELU: pre-activation out (C dtype)
  int M, N, K;
  int64_t lda, ldb, ldc;
  int64_t sa, sb, sc;  // batch strides (elements)
  int epi;
  int ksplit, nsplit;  // split-K (bf16 direct kernel only): K elements per split, number of splits (1 = off)
};

// Epilogue for 4 consecutive columns (col..col+3) of one row: the MFMA operands are swapped (acc = B-frag x A-frag)
// so that an accumulator's 4 consecutive registers are 4 consecutive COLUMNS of C; a lane then moves 16 bytes (f32)
// or 8 bytes (bf16) per access and the 2 half-waves of a row group fill 32 contiguous bytes.
template <int EPI, class OUT>
__device__ __forceinline__ void epilogue4(const GemmArgs &g, int64_t cbase, int row, int col, float v0, float v1, float v2, float v3, bool vec) {
  if (row >= g.M || col >= g.N) return;
  int64_t idx = cbase + (int64_t)row * g.ldc + col;
  OUT *c = (OUT *)g.c;
  float v[4] = {v0, v1, v2, v3};
  if (vec && col + 3 < g.N) {
    if (EPI == AH_EPI_ACCUM) {
      if (sizeof(OUT) == 4) { float4 o = *reinterpret_cast<const float4 *>((const float *)g.c + idx); v[0] += o.x; v[1] += o.y; v[2] += o.z; v[3] += o.w; }
      else { uint2 o = *reinterpret_cast<const uint2 *>((const uint16_t *)g.c + idx);
             v[0] += bf16_bits_to_f32(o.x & 0xffff); v[1] += bf16_bits_to_f32(o.x >> 16); v[2] += bf16_bits_to_f32(o.y & 0xffff); v[3] += bf16_bits_to_f32(o.y >> 16); }
    } else if (EPI == AH_EPI_RESIDUAL) {
      float4 o = *reinterpret_cast<const float4 *>((const float *)g.aux + idx);
      v[0] += o.x; v[1] += o.y; v[2] += o.z; v[3] += o.w;
    } else if (EPI == AH_EPI_GELU_BWD) {
      float x[4];
      if (sizeof(OUT) == 4) { float4 o = *reinterpret_cast<const float4 *>((const float *)g.aux + idx); x[0] = o.x; x[1] = o.y; x[2] = o.z; x[3] = o.w; }
      else { uint2 o = *reinterpret_cast<const uint2 *>((const uint16_t *)g.aux + idx);
             x[0] = bf16_bits_to_f32(o.x & 0xffff); x[1] = bf16_bits_to_f32(o.x >> 16); x[2] = bf16_bits_to_f32(o.y & 0xffff); x[3] = bf16_bits_to_f32(o.y >> 16); }
#pragma unroll
      for (int i = 0; i < 4; i++) v[i] *= gelu_grad_f(x[i]);
    } else if (EPI == AH_EPI_MUL_AUX) {
      float x[4];
      if (sizeof(OUT) == 4) { float4 o = *reinterpret_cast<const float4 *>((const float *)g.aux + idx); x[0] = o.x; x[1] = o.y; x[2] = o.z; x[3] = o.w; }
      else { uint2 o = *reinterpret_cast<const uint2 *>((const uint16_t *)g.aux + idx);
             x[0] = bf16_bits_to_f32(o.x & 0xffff); x[1] = bf16_bits_to_f32(o.x >> 16); x[2] = bf16_bits_to_f32(o.y & 0xffff); x[3] = bf16_bits_to_f32(o.y >> 16); }
#pragma unroll
      for (int i = 0; i < 4; i++) v[i] *= x[i];
    } else if (EPI == AH_EPI_GELU_GRAD) {
      float d[4];
#pragma unroll
      for (int i = 0; i < 4; i++) gelu_both_f(v[i], v[i], d[i]);
      if (sizeof(OUT) == 4) *reinterpret_cast<float4 *>((float *)g.aux_out + idx) = make_float4(d[0], d[1], d[2], d[3]);
      else *reinterpret_cast<uint2 *>((uint16_t *)g.aux_out + idx) = make_uint2(pack_bf16x2(d[0], d[1]), pack_bf16x2(d[2], d[3]));
    } else if (EPI == AH_EPI_GELU) {
      if (sizeof(OUT) == 4) *reinterpret_cast<float4 *>((float *)g.aux_out + idx) = make_float4(v[0], v[1], v[2], v[3]);
      else *reinterpret_cast<uint2 *>((uint16_t *)g.aux_out + idx) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
#pragma unroll
      for (int i = 0; i < 4; i++) v[i] = gelu_f(v[i]);
    }
    if (sizeof(OUT) == 4) *reinterpret_cast<float4 *>((float *)g.c + idx) = make_float4(v[0], v[1], v[2], v[3]);
    else *reinterpret_cast<uint2 *>((uint16_t *)g.c + idx) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (col + i < g.N) {
      float a = v[i];
      if (EPI == AH_EPI_ACCUM) a += Io<OUT>::ld(c, idx + i);
      else if (EPI == AH_EPI_RESIDUAL) a += ((const float *)g.aux)[idx + i];
      else if (EPI == AH_EPI_GELU_BWD) a *= gelu_grad_f(Io<OUT>::ld((const OUT *)g.aux, idx + i));
      else if (EPI == AH_EPI_GELU) { Io<OUT>::st((OUT *)g.aux_out, idx + i, a); a = gelu_f(a); }
      else if (EPI == AH_EPI_MUL_AUX) a *= Io<OUT>::ld((const OUT *)g.aux, idx + i);
      else if (EPI == AH_EPI_GELU_GRAD) { float d; gelu_both_f(a, a, d); Io<OUT>::st((OUT *)g.aux_out, idx + i, d); }
      Io<OUT>::st(c, idx + i, a);
    }
  }
}

// Stores a wave's TM x TN grid of 32x32 accumulators (C^T orientation: 4 consecutive registers = 4 consecutive columns).
template <int EPI, class OUT, int TM, int TN>
__device__ __forceinline__ void store_tiles(const GemmArgs &g, int64_t cbase, int row0, int col0, int lane, const f32x16 (&acc)[TM][TN]) {
  int lr = lane & 31, lk = lane >> 5;
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
      for (int q = 0; q < 4; q++)
        epilogue4<EPI, OUT>(g, cbase, row0 + 32 * i + lr, col0 + 32 * j + 8 * q + 4 * lk, acc[i][j][4 * q], acc[i][j][4 * q + 1],
                            acc[i][j][4 * q + 2], acc[i][j][4 * q + 3], true);
      __builtin_amdgcn_sched_barrier(0);      // drain one 32x32 tile at a time: the accumulators leave AGPRs 16 at a time
    }
}


// gemm_bf16.hip
int32_t gemm_bf16_direct(const GemmArgs &ga, int layout, int batch, int out_dtype);
// gemm_bf16_dma_{nt,nn,tn}.hip: 256 x bn tiles (bn = 256 or 192) fed by direct global->LDS loads (same preconditions as the
// direct kernel)
int32_t gemm_bf16_dma_nt(const GemmArgs &ga, int batch, int out_dtype, int bn);
int32_t gemm_bf16_dma_nn(const GemmArgs &ga, int batch, int out_dtype, int bn);
int32_t gemm_bf16_dma_tn(const GemmArgs &ga, int batch, int out_dtype, int bn);
int32_t gemm_bf16_dma_nt_grouped(const GemmGroupEntry *tab, int count, int blocks, int epi, int out_dtype);
int32_t gemm_bf16_dma_nn_grouped(const GemmGroupEntry *tab, int count, int blocks, int epi, int out_dtype);
int32_t gemm_bf16_dma_tn_grouped(const GemmGroupEntry *tab, int count, int blocks, int epi, int out_dtype);

}  // namespace ah
