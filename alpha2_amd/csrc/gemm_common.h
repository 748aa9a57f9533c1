// Shared between the GEMM translation units: argument block and the fused epilogues.
#pragma once
#include <type_traits>
#include "common.h"

namespace ah {

// One problem of a grouped launch (device-resident table; see ah_gemm_grouped_plan).
struct GemmGroupEntry {
  const void *a, *b;
  void *c;
  int M, N, K, tile_start;      // tile_start: first block id of this problem
  int partial, pad_;            // partial: what the entry stores is one half of a k-split product, not the final C
  int64_t lda, ldb, ldc;
};

// Records which kernel ah_gemm launched last (read back by ah_gemm_last_kernel).
void note_gemm_kernel(const char *fmt, ...);
void note_gemm_split(int nsplit);

struct GemmArgs {
  const void *a, *b;
  void *c;
  const void *aux;     // EPI_RESIDUAL: [M,N] of C's dtype; EPI_GELU_BWD: pre-activation (C dtype)
  void *aux_out;       // EPI_GELU: pre-activation out (C dtype)
  int M, N, K;
  int64_t lda, ldb, ldc;
  int64_t sa, sb, sc;  // batch strides (elements)
  int epi;
  int ksplit, nsplit;  // split-K (bf16 direct kernel only): K elements per split, number of splits (1 = off)
  float *sumsq;        // grouped launches that also sum the squares of what they store: the block's four slots (one per wave)
  // Planes (the large-tile bf16 kernel with a k-contiguous A only; off by default).  C: columns [p n, (p + 1) n) with
  // n = c_plane_n live c_plane_adj ELEMENTS further per p than in one [M, ldc] matrix.  A: k-tiles [p t, (p + 1) t) with
  // t = a_plane_tiles live a_plane_adj BYTES further per p than in one [M, lda] matrix (p <= 2).
  int c_plane_n = 0, a_plane_tiles = 1 << 28;
  int64_t c_plane_adj = 0, a_plane_adj = 0;
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
      if (sizeof(OUT) == 4) { float4 o = *reinterpret_cast<const float4 *>((const float *)g.aux + idx); v[0] += o.x; v[1] += o.y; v[2] += o.z; v[3] += o.w; }
      else { uint2 o = *reinterpret_cast<const uint2 *>((const uint16_t *)g.aux + idx);
             v[0] += bf16_bits_to_f32(o.x & 0xffff); v[1] += bf16_bits_to_f32(o.x >> 16); v[2] += bf16_bits_to_f32(o.y & 0xffff); v[3] += bf16_bits_to_f32(o.y >> 16); }
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
      else if (EPI == AH_EPI_RESIDUAL) a += Io<OUT>::ld((const OUT *)g.aux, idx + i);
      else if (EPI == AH_EPI_GELU_BWD) a *= gelu_grad_f(Io<OUT>::ld((const OUT *)g.aux, idx + i));
      else if (EPI == AH_EPI_GELU) { Io<OUT>::st((OUT *)g.aux_out, idx + i, a); a = gelu_f(a); }
      else if (EPI == AH_EPI_MUL_AUX) a *= Io<OUT>::ld((const OUT *)g.aux, idx + i);
      else if (EPI == AH_EPI_GELU_GRAD) { float d; gelu_both_f(a, a, d); Io<OUT>::st((OUT *)g.aux_out, idx + i, d); }
      Io<OUT>::st(c, idx + i, a);
    }
  }
}

// The values an epilogue reads beside the accumulators, 4 consecutive columns at a time, as the buffer load delivers them.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <bool F32> struct AuxVec;
template <> struct AuxVec<true> {
  typedef u32x4 T;
  static __device__ __forceinline__ T load(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0); }
  static __device__ __forceinline__ void unpack(const T &o, float (&x)[4]) {
    x[0] = __uint_as_float(o.x); x[1] = __uint_as_float(o.y); x[2] = __uint_as_float(o.z); x[3] = __uint_as_float(o.w);
  }
};
template <> struct AuxVec<false> {
  typedef u32x2 T;
  static __device__ __forceinline__ T load(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0); }
  static __device__ __forceinline__ void unpack(const T &o, float (&x)[4]) {
    x[0] = bf16_bits_to_f32(o.x & 0xffff); x[1] = bf16_bits_to_f32(o.x >> 16); x[2] = bf16_bits_to_f32(o.y & 0xffff); x[3] = bf16_bits_to_f32(o.y >> 16);
  }
};
// Descriptor of the `bytes` bytes at p (none if bytes <= 0): a lane whose byte offset reaches past them has its store
// dropped and its load answered with zeros by the address unit, so edge tiles need neither clamped addresses nor a
// masked-off branch around every access.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_window(const void *p, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, max(bytes, 0), 0x00020000);
}
// A plain epilogue whose stores carry the non-temporal hint: for an output far larger than the caches (the logits), whose
// lines would otherwise push the operand panels the same XCD needs again out of its L2.  Internal to the dispatcher.
constexpr int EPI_PLAIN_STREAMED = 7;
template <int POLICY>
__device__ __forceinline__ void buffer_store4(float v0, float v1, float v2, float v3, float *, __amdgpu_buffer_rsrc_t r, uint32_t off) {
  u32x4 d = {__float_as_uint(v0), __float_as_uint(v1), __float_as_uint(v2), __float_as_uint(v3)};
  __builtin_amdgcn_raw_buffer_store_b128(d, r, off, 0, POLICY);
}
template <int POLICY>
__device__ __forceinline__ void buffer_store4(float v0, float v1, float v2, float v3, uint16_t *, __amdgpu_buffer_rsrc_t r, uint32_t off) {
  u32x2 d = {pack_bf16x2(v0, v1), pack_bf16x2(v2, v3)};
  __builtin_amdgcn_raw_buffer_store_b64(d, r, off, 0, POLICY);
}

// Four 4 KB pieces of LDS that belong to the calling wave alone (nobody else reads or writes them until the next
// workgroup barrier).
struct EpiStage { char *p[4]; };

// Epilogue of a wave tile through LDS.  In the accumulator layout a lane owns 4 consecutive
// columns of ONE row, so a store instruction written straight from the accumulators scatters 16-byte pieces over 32
// rows: 32 partial cache lines per instruction (measured: the stores of a K = 768 product then take a third of its time).
// Instead each 32 x 32 accumulator goes to LDS as f32 (row r at r * 128 bytes, 16-byte chunk c at position c ^ (r & 7):
// conflict-free both ways) and comes back row-major: 8 (f32 output) or 16 (bf16 output, two tiles side by side) lanes
// cover one row's 128 contiguous bytes, and everything an epilogue reads (residual, accumulate, saved gelu') is loaded in
// that same coalesced layout.
// Addressing: every access goes through a buffer descriptor whose base is moved, with scalar arithmetic, to the first
// row and column of the group of rows being written, and whose size is what is left of the wave tile's rows inside C
// from there; the per-lane part of the address is one of two constants (row in the group x ldc + column).  A lane in a
// row past the end of C is then out of the descriptor's range, a lane in a column past the end is given an offset that
// always is.  The loads run ahead: vmcnt retires in issue order, stores included, so the reads of pass p + DEPTH are issued
// before the stores of pass p.  Requires N % 4 == 0 and 128 rows of C to span less than 2 GiB.
// With SUMSQ the lane also adds up the squares of the values it stores (those the address unit drops count as zero) and
// returns the sum.
template <int EPI, class OUT, int TM, int TN, bool SUMSQ = false>
__device__ __forceinline__ float store_tiles_lds(const GemmArgs &g, int64_t cbase, int row0, int col0, int lane, const f32x16 (&acc)[TM][TN],
                                                 const EpiStage &st) {
  constexpr bool F32OUT = sizeof(OUT) == 4;
  constexpr int JP = F32OUT ? 1 : 2;                  // 32 x 32 tiles per pass: a row of the pass is 128 bytes of output
  constexpr int NJP = (TN + JP - 1) / JP, NPASS = TM * NJP;
  constexpr bool READS = EPI == AH_EPI_ACCUM || EPI == AH_EPI_RESIDUAL || EPI == AH_EPI_GELU_BWD || EPI == AH_EPI_MUL_AUX;
  constexpr bool AUX_F32 = F32OUT;                    // what an epilogue reads has the type of C
  constexpr int DEPTH = 4 < NPASS ? 4 : NPASS;        // passes of reads in flight: 4 x 16 registers
  constexpr int ES = sizeof(OUT), AES = AUX_F32 ? 4 : 2;
  constexpr uint32_t OUTSIDE = 0x80000000u;           // a byte offset no descriptor here reaches (they are shorter than 2 GiB)
  typedef AuxVec<AUX_F32> AV;
  typedef typename AV::T AuxT;
  const int lr = lane & 31, lk = lane >> 5;
  const int64_t origin = cbase + (int64_t)row0 * g.ldc + col0;
  const char *c = (const char *)g.c + origin * ES;
  const char *aux = (const char *)(EPI == AH_EPI_ACCUM ? (const void *)g.c : g.aux) + origin * AES;
  const char *aux_out = (const char *)g.aux_out + origin * ES;
  // a pass of NS tiles side by side comes back in 4 NS iterations of 8 / NS rows: lane -> (row in the group, chunk)
  const int rr1 = lane >> 3, cc1 = lane & 7, rr2 = lane >> 4, cc2 = lane & 15;
  const int rows_here = min(g.M - row0, 32 * TM), cols_left = g.N - col0;       // rows / columns of the wave tile inside C
  const int ldc = (int)g.ldc, span = rows_here * ldc;       // span: elements from the origin to the end of the last row inside C (< 2^29)
  const uint32_t lane_el1 = (uint32_t)(rr1 * ldc + 4 * cc1), lane_el2 = (uint32_t)(rr2 * ldc + 4 * cc2);
  int wofs[4];
#pragma unroll
  for (int q = 0; q < 4; q++) wofs[q] = lr * 128 + (((2 * q + lk) ^ (lr & 7)) << 4);

  AuxT pre[DEPTH][8];
  float ss = 0.f;
  // element offset (uniform) of the first row and column of iteration `it` of pass p, and this lane's part for the pass
  auto group_el = [&](int p, int it) -> int {
    const int i = p / NJP, j0 = (p % NJP) * JP, ns = TN - j0 < JP ? TN - j0 : JP;
    return (32 * i + it * (8 / ns)) * ldc + 32 * j0;
  };
  auto lane_bytes = [&](int p, int esize) -> uint32_t {
    const int j0 = (p % NJP) * JP, ns = TN - j0 < JP ? TN - j0 : JP;
    const bool col_inside = 32 * j0 + 4 * (ns == 2 ? cc2 : cc1) < cols_left;
    return col_inside ? (ns == 2 ? lane_el2 : lane_el1) * (uint32_t)esize : OUTSIDE;
  };
  auto issue_reads = [&](int p) {
    const int j0 = (p % NJP) * JP, ns = TN - j0 < JP ? TN - j0 : JP;
    const uint32_t le = lane_bytes(p, AES);
#pragma unroll
    for (int it = 0; it < 4 * ns; it++) {
      const int ge = group_el(p, it);
      pre[p % DEPTH][it] = AV::load(buffer_window(aux + ge * AES, (span - ge) * AES), le);
    }
  };
  if (READS) {
#pragma unroll
    for (int p = 0; p < DEPTH; p++) issue_reads(p);
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int p = 0; p < NPASS; p++) {
    const int i = p / NJP, j0 = (p % NJP) * JP, ns = TN - j0 < JP ? TN - j0 : JP;
    char *piece0 = st.p[JP == 2 ? 2 * (p & 1) : p & 3], *piece1 = st.p[JP == 2 ? 2 * (p & 1) + 1 : p & 3];
#pragma unroll
    for (int jj = 0; jj < ns; jj++)
#pragma unroll
      for (int q = 0; q < 4; q++)
        *reinterpret_cast<float4 *>((jj ? piece1 : piece0) + wofs[q]) =
            make_float4(acc[i][j0 + jj][4 * q], acc[i][j0 + jj][4 * q + 1], acc[i][j0 + jj][4 * q + 2], acc[i][j0 + jj][4 * q + 3]);
    const uint32_t le = lane_bytes(p, ES);
#pragma unroll
    for (int it = 0; it < 4 * ns; it++) {
      const int r = it * (8 / ns) + (ns == 2 ? rr2 : rr1), ch = ns == 2 ? cc2 & 7 : cc1;
      const char *src = (ns == 2 && cc2 >= 8 ? piece1 : piece0) + r * 128 + ((ch ^ (r & 7)) << 4);
      const float4 t = *reinterpret_cast<const float4 *>(src);
      float v[4] = {t.x, t.y, t.z, t.w};
      const int ge = group_el(p, it);
      if (READS) {
        float x[4];
        AV::unpack(pre[p % DEPTH][it], x);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          if (EPI == AH_EPI_ACCUM || EPI == AH_EPI_RESIDUAL) v[e] += x[e];
          else if (EPI == AH_EPI_MUL_AUX) v[e] *= x[e];
          else v[e] *= gelu_grad_f(x[e]);
        }
      } else if (EPI == AH_EPI_GELU_GRAD) {
        float d[4];
#pragma unroll
        for (int e = 0; e < 4; e++) gelu_both_f(v[e], v[e], d[e]);
        buffer_store4<2>(d[0], d[1], d[2], d[3], (OUT *)nullptr, buffer_window(aux_out + ge * ES, (span - ge) * ES), le);   // kept for backward: streamed past the caches
      } else if (EPI == AH_EPI_GELU) {
        buffer_store4<0>(v[0], v[1], v[2], v[3], (OUT *)nullptr, buffer_window(aux_out + ge * ES, (span - ge) * ES), le);
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = gelu_f(v[e]);
      }
      buffer_store4<EPI == EPI_PLAIN_STREAMED ? 2 : 0>(v[0], v[1], v[2], v[3], (OUT *)nullptr, buffer_window(c + ge * ES, (span - ge) * ES), le);
      if (SUMSQ) {      // the address unit's own test: the lane's 4 elements end inside the window
        const bool stored = le != OUTSIDE && (int)(ns == 2 ? lane_el2 : lane_el1) + 4 <= span - ge;
        const float q = v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
        ss += stored ? q : 0.f;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (READS && p + DEPTH < NPASS) {
      issue_reads(p + DEPTH);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  return ss;
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
bool gemm_bf16_takes_large_tile(const GemmArgs &ga, int layout);       // would gemm_bf16_direct run it on the 256-row tile kernel (batch 1)
// c[M][N] (leading dimension ldc) = (accumulate ? c : 0) + sum over the nsplit slices of ws[nsplit][M][N], in fixed order; M N % 4 == 0
int32_t splitk_reduce(const float *ws, float *c, int nsplit, int M, int N, int64_t ldc, bool accumulate);
// gemm_bf16_dma_{nt,nn,tn}.hip: 256 x bn tiles (bn = 256 or 192) fed by direct global->LDS loads (same preconditions as the
// direct kernel)
int32_t gemm_bf16_dma_nt(const GemmArgs &ga, int batch, int out_dtype, int bn);
int32_t gemm_bf16_dma_nn(const GemmArgs &ga, int batch, int out_dtype, int bn);
int32_t gemm_bf16_dma_tn(const GemmArgs &ga, int batch, int out_dtype, int bn);
// sumsq (f32 outputs only, or null): 4 floats per block, the sums of the squares of what each wave stored as final values of C
int32_t gemm_bf16_dma_nt_grouped(const GemmGroupEntry *tab, int count, int blocks, int epi, int out_dtype, float *sumsq);
int32_t gemm_bf16_dma_nn_grouped(const GemmGroupEntry *tab, int count, int blocks, int epi, int out_dtype, float *sumsq);
int32_t gemm_bf16_dma_tn_grouped(const GemmGroupEntry *tab, int count, int blocks, int epi, int out_dtype, float *sumsq);

}  // namespace ah
