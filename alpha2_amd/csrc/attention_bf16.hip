// bf16 causal flash attention (fp32 accumulation) on v_mfma_f32_32x32x16_bf16, forward and backward.
//
// Same arrangement as the fp32 kernels: the index a wave owns (32 queries in forward / dQ, 32 keys in dK/dV) is
// the accumulator COLUMN, so softmax statistics are per-lane scalars and the probabilities feed the second product
// straight from registers.  A 32x32 accumulator holds rows 8j + 4h + r (j = 0..3, r = 0..3, h = lane/32); as the B
// operand of a 16-deep MFMA, half h supplies 8 k-slots, and slot i of MFMA m is taken to mean streamed row
// 16m + 8(i/4) + 4h + i%4 -- exactly the rows that half holds in accumulator registers 8m..8m+7.  The other operand
// must use the same slot order; it is read from the [row][d] LDS tile with ds_read_b64_tr_b16, whose 16-lane groups
// may address any four rows, so no transposed copy of V (or K, Q, dO in the backward kernels) is ever made.
//
// One block = 4 waves = 128 owned rows; the streamed operand moves in 64-row tiles, register-prefetched one tile
// ahead and double-buffered in LDS (one barrier per 64 rows).
//
// The kernels are bound by the per-score VALU work (exp and rcp are quarter rate), not by the MFMAs, so the score
// path is pared down to the instructions that cannot be avoided:
//   * everything runs in base-2: constants carry log2(e), exp is the bare v_exp_f32;
//   * with a soft cap c the capped score is c*tanh(u) = c - 2c*r, r = 1/(exp(2u) + 1), which is bounded by c.  For
//     c <= 40 the running maximum of the online softmax is replaced by the constant c: p = exp(-2c*r) needs no max
//     pass, no rescale of the output accumulators and no cross-lane traffic until the row sum is finished; the smallest
//     possible p, exp(-80), is far inside fp32 / bf16 range.  tanh' = 4r(1 - r) reuses r in the backward kernels;
//   * masking code runs only for tiles that touch the diagonal or the end of the sequence (a wave-uniform branch);
//   * constant factors (scale, the 4 of tanh') are applied once to the accumulators, not per score.
#include "attention_common.h"
#include <cstdlib>
#include <cstring>

using namespace ah;

namespace {

constexpr int ST = 64;       // streamed rows per LDS tile
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) bf16x4 lds_v4;

template <int D> struct Geo {
  static constexpr int PITCH = D + 16;                 // bf16 elements; (D+16)*2 bytes = 32 mod 128 for D in {32,64,128}... see tile_frag_t
  static constexpr int ELEMS = ST * PITCH;
  static constexpr int CHUNKS = ST * D / 8 / 256;      // 16-byte chunks per thread per tile (D=32: 1, 64: 2, 128: 4)
};

constexpr float LOG2E = 1.4426950408889634f;
constexpr float FIXED_MAX_CAP = 40.f;      // soft caps up to this use the constant-maximum softmax
// AH_FLASH_BWD=onepass makes variant 1 of the backward pass the default of a process (measurement aid)
bool flash_bwd_one_pass() {
  static const bool on = [] { const char *e = getenv("AH_FLASH_BWD"); return e && strcmp(e, "onepass") == 0; }();
  return on;
}

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float rcp_fast(float x) { return __builtin_amdgcn_rcpf(x); }
// First statement of a block that only the tiles on the diagonal need (masking): with it the compiler keeps the block behind a
// branch the other tiles skip, where it would otherwise turn a cheap block into selects that every tile executes.
__device__ __forceinline__ void keep_branch() { asm volatile("; rare path" ::: "memory"); }

// global -> registers: rows [row0, row0+64) of a [T][D] operand with row stride st (elements); rows >= T read as zero
// (PAD: the tensors' head size hd is smaller than D; features hd .. D - 1 read as zero)
template <int D, bool PAD = false>
__device__ __forceinline__ void tile_load(const uint16_t *__restrict__ base, int64_t st, int row0, int T, u32x4 (&v)[Geo<D>::CHUNKS], int hd = D) {
#pragma unroll
  for (int i = 0; i < Geo<D>::CHUNKS; i++) {
    int c = threadIdx.x + 256 * i, r = c / (D / 8), c8 = c % (D / 8);
    u32x4 x = {0u, 0u, 0u, 0u};
    if (row0 + r < T && (!PAD || c8 * 8 < hd)) x = *reinterpret_cast<const u32x4 *>(base + (int64_t)(row0 + r) * st + c8 * 8);
    v[i] = x;
  }
}
template <int D>
__device__ __forceinline__ void tile_store(uint16_t *s, const u32x4 (&v)[Geo<D>::CHUNKS]) {
#pragma unroll
  for (int i = 0; i < Geo<D>::CHUNKS; i++) {
    int c = threadIdx.x + 256 * i, r = c / (D / 8), c8 = c % (D / 8);
    *reinterpret_cast<u32x4 *>(s + r * Geo<D>::PITCH + c8 * 8) = v[i];
  }
}
// A/B fragment with the tile ROW as the MFMA row/column (k = feature d): rows r0 + lane%32, d = 16*ks + 8*(lane/32)..
template <int D>
__device__ __forceinline__ bf16x8 tile_frag(const uint16_t *s, int r0, int ks, int lane) {
  return *reinterpret_cast<const bf16x8 *>(s + (r0 + (lane & 31)) * Geo<D>::PITCH + ks * 16 + (lane >> 5) * 8);
}
// A fragment with the feature d as the MFMA row (k = tile row, in the accumulator's slot order): features
// 32*db + lane%32, k-slot i of this half = tile row r0 + 16m + 8(i/4) + 4(lane/32) + i%4.
template <int D>
__device__ __forceinline__ bf16x8 tile_frag_t(const uint16_t *s, int r0, int m, int db, int lane) {
  int j = lane & 15, g = lane >> 4, lk = g >> 1;
  const uint16_t *p = s + (r0 + 16 * m + 4 * lk + (j >> 2)) * Geo<D>::PITCH + 32 * db + 16 * (g & 1) + 4 * (j & 3);
  bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4 *)p);
  bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4 *)(p + 8 * Geo<D>::PITCH));
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
// accumulator registers 8m..8m+7 -> bf16 B operand of MFMA m
__device__ __forceinline__ bf16x8 acc_to_b(const f32x16 &s, int m) {
  bf16x8 r;
#pragma unroll
  for (int i = 0; i < 8; i++) r[i] = (__bf16)s[8 * m + i];
  return r;
}
// this lane's row of a [T][D] operand as B fragments (k = d): one 16-byte global load per 16 features
template <int D, bool PAD = false>
__device__ __forceinline__ void row_frags(const uint16_t *__restrict__ base, int64_t st, int row, bool live, int lane, bf16x8 (&f)[D / 16], int hd = D) {
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++) {
    u32x4 x = {0u, 0u, 0u, 0u};
    if (live && (!PAD || ks * 16 + (lane >> 5) * 8 < hd)) x = *reinterpret_cast<const u32x4 *>(base + (int64_t)row * st + ks * 16 + (lane >> 5) * 8);
    f[ks] = __builtin_bit_cast(bf16x8, x);
  }
}
// O^T-style accumulators (rows = features 32db + 8j + 4h + r, column = owned row) -> bf16 row-major store
template <int D, bool PAD = false>
__device__ __forceinline__ void store_rows(uint16_t *__restrict__ dst, const f32x16 (&acc)[D / 32], float mul, int lane, int hd = D) {
  int lk = lane >> 5;
#pragma unroll
  for (int db = 0; db < D / 32; db++)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      uint2 w = make_uint2(pack_bf16x2(acc[db][4 * j] * mul, acc[db][4 * j + 1] * mul), pack_bf16x2(acc[db][4 * j + 2] * mul, acc[db][4 * j + 3] * mul));
      if (!PAD || 32 * db + 8 * j + 4 * lk < hd) *reinterpret_cast<uint2 *>(dst + 32 * db + 8 * j + 4 * lk) = w;
    }
}

// ------------------------------------------------------------------------------------------ forward
// Launch bounds ask for at least two (three) waves per SIMD at head sizes up to 64: besides the occupancy this keeps the
// register budget at 256 (170), where the compiler uses the VGPR form of MFMA and no accumulator ever has to be copied
// between AGPRs and VGPRs for the softmax arithmetic.
template <int D, bool CAPPED, bool PAD>
__device__ __forceinline__ void flash_fwd_bf16_body(const FlashArgs &a) {
  constexpr int DB = D / 32, KS = D / 16;
  __shared__ __attribute__((aligned(16))) uint16_t Ks[2][Geo<D>::ELEMS], Vs[2][Geo<D>::ELEMS];
  int bh, xblk;
  flash_block(bh, xblk, flash_head_group(a.T, D, 2));
  int b = bh / a.H, h = bh % a.H;
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 31, lk = lane >> 5;
  int qblk = gridDim.x - 1 - xblk;                                 // longest (latest) query blocks are scheduled first
  int q0 = qblk * 128 + wave * 32, qi = q0 + lr;
  const uint16_t *Q = (const uint16_t *)a.q + b * a.q_sb + h * a.q_sh;
  const uint16_t *K = (const uint16_t *)a.k + b * a.k_sb + h * a.k_sh;
  const uint16_t *V = (const uint16_t *)a.v + b * a.v_sb + h * a.v_sh;
  // CAPPED: u2 = s*c1 = 2*score/cap in base 2; p = 2^(c2*r).  Otherwise x = s*c1 = score in base 2.
  const float c1 = CAPPED ? 2.0f * a.scale * LOG2E / a.cap : a.scale * LOG2E;
  const float ic2 = CAPPED ? -1.0f / (2.0f * a.cap * LOG2E) : 0.f;      // 1 / c2, c2 = -2 cap log2(e): p = 2^(c2 r)

  bf16x8 qf[KS];
  row_frags<D, PAD>(Q, a.q_st, qi, qi < a.T, lane, qf, a.hd);
  f32x16 o[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int e = 0; e < 16; e++) o[d][e] = 0.f;
  // CAPPED: l is this half-wave's partial row sum of the probabilities as computed (for LSE, from which the backward
  // kernels rebuild them); lacc accumulates the row sum of the probabilities as rounded to bf16 (for normalising O); m is unused
  float m = -INFINITY, l = 0.f, l_rnd = 0.f;
  f32x16 lacc;
  bf16x8 ones;
#pragma unroll
  for (int e = 0; e < 16; e++) lacc[e] = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) ones[i] = (__bf16)1.0f;

  int kv_end = min(a.T, (qblk + 1) * 128);                         // causal: keys < kv_end
  int ntile = (kv_end + ST - 1) / ST;
  u32x4 rk[Geo<D>::CHUNKS], rv[Geo<D>::CHUNKS];
  tile_load<D, PAD>(K, a.k_st, 0, a.T, rk, a.hd);
  tile_load<D, PAD>(V, a.v_st, 0, a.T, rv, a.hd);
  tile_store<D>(Ks[0], rk);
  tile_store<D>(Vs[0], rv);
  __syncthreads();
  for (int it = 0; it < ntile; it++) {
    int cur = it & 1;
    if (it + 1 < ntile) {
      tile_load<D, PAD>(K, a.k_st, (it + 1) * ST, a.T, rk, a.hd);
      tile_load<D, PAD>(V, a.v_st, (it + 1) * ST, a.T, rv, a.hd);
    }
    if (CAPPED && it * ST + ST - 1 <= q0) {
      // Both 32-key halves of the tile lie entirely below this wave's diagonal (no masking, which is most tiles): run
      // them as two independent MFMA chains so the softmax arithmetic of one overlaps the matrix work of the other.
      f32x16 s0, s1;
#pragma unroll
      for (int e = 0; e < 16; e++) { s0[e] = 0.f; s1[e] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag<D>(Ks[cur], 0, ks, lane), qf[ks], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag<D>(Ks[cur], 32, ks, lane), qf[ks], s1, 0, 0, 0);
      }
#pragma unroll
      for (int e = 0; e < 16; e++) { s0[e] = exp2_fast(rcp_fast(fmaf(exp2_fast(s0[e] * c1), ic2, ic2))); l += s0[e]; }
      bf16x8 pa0 = acc_to_b(s0, 0), pa1 = acc_to_b(s0, 1);
      lacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pa0, lacc, 0, 0, 0);
      lacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pa1, lacc, 0, 0, 0);
#pragma unroll
      for (int d = 0; d < DB; d++) {
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Vs[cur], 0, 0, d, lane), pa0, o[d], 0, 0, 0);
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Vs[cur], 0, 1, d, lane), pa1, o[d], 0, 0, 0);
      }
#pragma unroll
      for (int e = 0; e < 16; e++) { s1[e] = exp2_fast(rcp_fast(fmaf(exp2_fast(s1[e] * c1), ic2, ic2))); l += s1[e]; }
      bf16x8 pc0 = acc_to_b(s1, 0), pc1 = acc_to_b(s1, 1);
      lacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pc0, lacc, 0, 0, 0);
      lacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pc1, lacc, 0, 0, 0);
#pragma unroll
      for (int d = 0; d < DB; d++) {
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Vs[cur], 32, 0, d, lane), pc0, o[d], 0, 0, 0);
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Vs[cur], 32, 1, d, lane), pc1, o[d], 0, 0, 0);
      }
    } else
#pragma unroll
    for (int sub = 0; sub < ST / 32; sub++) {
      int kv0 = it * ST + sub * 32;
      if (kv0 <= q0 + 31) {                                        // otherwise the sub-tile is in this wave's future
        f32x16 s;
#pragma unroll
        for (int e = 0; e < 16; e++) s[e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
          s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag<D>(Ks[cur], sub * 32, ks, lane), qf[ks], s, 0, 0, 0);   // S^T[kv, q]
        const bool edge = kv0 + 31 > q0 || kv0 + 32 > a.T;         // wave-uniform: some score of the tile is masked
        if (CAPPED) {
#pragma unroll
          for (int e = 0; e < 16; e++)        // c2 r = c2 / (e + 1) = 1 / (e / c2 + 1 / c2): one fma feeds the reciprocal
            s[e] = exp2_fast(rcp_fast(fmaf(exp2_fast(s[e] * c1), ic2, ic2)));
          if (edge) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
              int kv = kv0 + 8 * (e >> 2) + 4 * lk + (e & 3);
              s[e] = (kv > qi || kv >= a.T) ? 0.f : s[e];
            }
          }
#pragma unroll
          for (int e = 0; e < 16; e++) l += s[e];
        } else {
          float tmax = -INFINITY;
#pragma unroll
          for (int e = 0; e < 16; e++) s[e] *= c1;
          if (edge) {
            keep_branch();
#pragma unroll
            for (int e = 0; e < 16; e++) {
              int kv = kv0 + 8 * (e >> 2) + 4 * lk + (e & 3);
              s[e] = (kv > qi || kv >= a.T) ? -INFINITY : s[e];
            }
          }
#pragma unroll
          for (int e = 0; e < 16; e++) tmax = fmaxf(tmax, s[e]);
          tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
          float m_new = fmaxf(m, tmax);
          float m_use = m_new == -INFINITY ? 0.f : m_new;
          float alpha = exp2_fast(m - m_use);
          float psum = 0.f;
#pragma unroll
          for (int e = 0; e < 16; e++) { float p = exp2_fast(s[e] - m_use); s[e] = p; psum += p; }
          psum += __shfl_xor(psum, 32, 64);
          l = l * alpha + psum;
          m = m_new;
#pragma unroll
          for (int d = 0; d < DB; d++)
#pragma unroll
            for (int e = 0; e < 16; e++) o[d][e] *= alpha;
        }
        bf16x8 pb0 = acc_to_b(s, 0), pb1 = acc_to_b(s, 1);
        if (CAPPED) {
          // O is normalised by the sum of the bf16-rounded probabilities the MFMA sees (a row with a single key
          // returns that key's V exactly).  That sum is taken by the idle matrix pipe: a ones operand in place of V
          // leaves sum_kv p[kv][q] in every row of the accumulator.
          lacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb0, lacc, 0, 0, 0);
          lacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb1, lacc, 0, 0, 0);
        }
#pragma unroll
        for (int d = 0; d < DB; d++) {
          o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Vs[cur], sub * 32, 0, d, lane), pb0, o[d], 0, 0, 0);   // O^T[d, q]
          o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Vs[cur], sub * 32, 1, d, lane), pb1, o[d], 0, 0, 0);
        }
      }
    }
    if (it + 1 < ntile) {
      tile_store<D>(Ks[cur ^ 1], rk);
      tile_store<D>(Vs[cur ^ 1], rv);
    }
    __syncthreads();
  }
  if (CAPPED) { l += __shfl_xor(l, 32, 64); l_rnd = lacc[0]; } else l_rnd = l;
  if (qi < a.T) {
    float inv_l = l_rnd > 0.f ? 1.0f / l_rnd : 0.f;
    store_rows<D, PAD>((uint16_t *)a.o + b * a.o_sb + h * a.o_sh + (int64_t)qi * a.o_st, o, inv_l, lane, a.hd);
    // natural-log LSE: the constant maximum is the cap itself; the running maximum is held in base 2
    if (lk == 0) a.lse[((int64_t)b * a.H + h) * a.T + qi] = (CAPPED ? a.cap : m * (1.0f / LOG2E)) + __logf(l);
  }
}
template <int D, bool CAPPED>
__global__ __launch_bounds__(256, D <= 64 ? 3 : 1) void k_flash_fwd_bf16(FlashArgs a) { flash_fwd_bf16_body<D, CAPPED, false>(a); }
// the same for tensors whose head size is smaller than D
template <int D, bool CAPPED>
__global__ __launch_bounds__(256, D <= 64 ? 3 : 1) void k_flash_fwd_bf16_padded(FlashArgs a) { flash_fwd_bf16_body<D, CAPPED, true>(a); }

// Per-score backward arithmetic shared by the dQ and dK/dV kernels.  s = raw q.k, dpd = dO.v - delta with delta =
// rowsum(dO*O) (in dK/dV the dP accumulator starts at -delta, so the subtraction rides on the MFMA; dQ subtracts it per score),
// krow = (max - lse) in base 2 (max = cap when CAPPED, else 0).  Returns p and writes ds WITHOUT the constant factor (scale,
// and 4 for tanh' when CAPPED), which the caller applies to its accumulators once.
template <bool CAPPED>
__device__ __forceinline__ float score_bwd(float s, float dpd, float krow, float c1, float c2, float &ds) {
  float p;
  if (CAPPED) {
    float r = rcp_fast(exp2_fast(s * c1) + 1.0f);
    p = exp2_fast(fmaf(r, c2, krow));
    ds = p * dpd * fmaf(-r, r, r);                                 // tanh' / 4 = r (1 - r)
  } else {
    p = exp2_fast(fmaf(s, c1, krow));
    ds = p * dpd;
  }
  return p;
}

// ------------------------------------------------------------------------------------------ dQ (and delta)
template <int D, bool CAPPED, bool PAD>
__device__ __forceinline__ void flash_dq_bf16_body(const FlashArgs &a) {
  constexpr int DB = D / 32, KS = D / 16;
  __shared__ __attribute__((aligned(16))) uint16_t Ks[2][Geo<D>::ELEMS], Vs[2][Geo<D>::ELEMS];
  int bh, xblk;
  flash_block(bh, xblk, flash_head_group(a.T, D, 2));
  int b = bh / a.H, h = bh % a.H;
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 31, lk = lane >> 5;
  int qblk = gridDim.x - 1 - xblk;
  int q0 = qblk * 128 + wave * 32, qi = q0 + lr;
  const uint16_t *Q = (const uint16_t *)a.q + b * a.q_sb + h * a.q_sh;
  const uint16_t *K = (const uint16_t *)a.k + b * a.k_sb + h * a.k_sh;
  const uint16_t *V = (const uint16_t *)a.v + b * a.v_sb + h * a.v_sh;
  const uint16_t *O = (const uint16_t *)a.o + b * a.o_sb + h * a.o_sh;
  const uint16_t *dO = (const uint16_t *)a.d_o + b * a.o_sb + h * a.o_sh;
  const float c1 = CAPPED ? 2.0f * a.scale * LOG2E / a.cap : a.scale * LOG2E;
  const float c2 = -2.0f * a.cap * LOG2E;
  bool live = qi < a.T;
  bf16x8 qf[KS], dof[KS];
  row_frags<D, PAD>(Q, a.q_st, qi, live, lane, qf, a.hd);
  row_frags<D, PAD>(dO, a.o_st, qi, live, lane, dof, a.hd);
  // the first key tile is asked for before delta is worked out, so that the two waits for memory are one
  u32x4 rk[Geo<D>::CHUNKS], rv[Geo<D>::CHUNKS];
  tile_load<D, PAD>(K, a.k_st, 0, a.T, rk, a.hd);
  tile_load<D, PAD>(V, a.v_st, 0, a.T, rv, a.hd);
  int64_t srow = ((int64_t)b * a.H + h) * a.T + qi;
  // delta = rowsum(dO * O): each half-wave holds half of the row's features; also published for the dK/dV kernel
  float delta = 0.f;
  {
    bf16x8 of[KS];
    row_frags<D, PAD>(O, a.o_st, qi, live, lane, of, a.hd);
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
      for (int i = 0; i < 8; i++) delta += (float)dof[ks][i] * (float)of[ks][i];
    delta += __shfl_xor(delta, 32, 64);
    if (live && lk == 0) a.delta[srow] = delta;
  }
  float krow = live ? ((CAPPED ? a.cap : 0.f) - a.lse[srow]) * LOG2E : 0.f;
  f32x16 dq[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int e = 0; e < 16; e++) dq[d][e] = 0.f;

  int kv_end = min(a.T, (qblk + 1) * 128);
  int ntile = (kv_end + ST - 1) / ST;
  tile_store<D>(Ks[0], rk);
  tile_store<D>(Vs[0], rv);
  __syncthreads();
  for (int it = 0; it < ntile; it++) {
    int cur = it & 1;
    if (it + 1 < ntile) {
      tile_load<D, PAD>(K, a.k_st, (it + 1) * ST, a.T, rk, a.hd);
      tile_load<D, PAD>(V, a.v_st, (it + 1) * ST, a.T, rv, a.hd);
    }
#pragma unroll
    for (int sub = 0; sub < ST / 32; sub++) {
      int kv0 = it * ST + sub * 32;
      if (kv0 <= q0 + 31) {
        f32x16 s, dp;
#pragma unroll
        for (int e = 0; e < 16; e++) { s[e] = 0.f; dp[e] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag<D>(Ks[cur], sub * 32, ks, lane), qf[ks], s, 0, 0, 0);     // S^T[kv, q]
          dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag<D>(Vs[cur], sub * 32, ks, lane), dof[ks], dp, 0, 0, 0);  // dP^T[kv, q]
        }
        const bool edge = kv0 + 31 > q0 || kv0 + 32 > a.T;
#pragma unroll
        for (int e = 0; e < 16; e++) {
          float ds;
          score_bwd<CAPPED>(s[e], dp[e] - delta, krow, c1, c2, ds);       // this lane's column is one query
          s[e] = ds;
        }
        if (edge) {
#pragma unroll
          for (int e = 0; e < 16; e++) {
            int kv = kv0 + 8 * (e >> 2) + 4 * lk + (e & 3);
            s[e] = (kv > qi || kv >= a.T) ? 0.f : s[e];
          }
        }
        bf16x8 b0 = acc_to_b(s, 0), b1 = acc_to_b(s, 1);
#pragma unroll
        for (int d = 0; d < DB; d++) {                             // dQ^T[d, q] += K^T[d, kv] dS^T[kv, q]
          dq[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Ks[cur], sub * 32, 0, d, lane), b0, dq[d], 0, 0, 0);
          dq[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Ks[cur], sub * 32, 1, d, lane), b1, dq[d], 0, 0, 0);
        }
      }
    }
    if (it + 1 < ntile) {
      tile_store<D>(Ks[cur ^ 1], rk);
      tile_store<D>(Vs[cur ^ 1], rv);
    }
    __syncthreads();
  }
  if (live) store_rows<D, PAD>((uint16_t *)a.dq + b * a.q_sb + h * a.q_sh + (int64_t)qi * a.q_st, dq, CAPPED ? 4.0f * a.scale : a.scale, lane, a.hd);
}
// Three waves per SIMD at head sizes up to 64 (170 registers): these kernels are bound by what the vector unit issues, and a
// third wave keeps it fed while another waits for memory, a barrier or an MFMA chain.  That is why delta is subtracted per
// score above instead of riding on the dP product as its starting value: the 16 registers that held it bought the third wave
// (two waves with the products of the next sub-tile pipelined between the scores of the current one: 170 against 166 us for
// the backward pass of a layer at B = 16, H = 12, T = 1024; 174 before either).
template <int D, bool CAPPED>
__global__ __launch_bounds__(256, D <= 64 ? 3 : 1) void k_flash_dq_bf16(FlashArgs a) { flash_dq_bf16_body<D, CAPPED, false>(a); }
// the same for tensors whose head size is smaller than D
template <int D, bool CAPPED>
__global__ __launch_bounds__(256, D <= 64 ? 3 : 1) void k_flash_dq_bf16_padded(FlashArgs a) { flash_dq_bf16_body<D, CAPPED, true>(a); }

// ------------------------------------------------------------------------------------------ dK, dV
template <int D, bool CAPPED, bool PAD>
__device__ __forceinline__ void flash_dkv_bf16_body(const FlashArgs &a) {
  constexpr int DB = D / 32, KS = D / 16;
  __shared__ __attribute__((aligned(16))) uint16_t Qs[2][Geo<D>::ELEMS], dOs[2][Geo<D>::ELEMS];
  __shared__ __attribute__((aligned(16))) float Ls[2][ST], Ds[2][ST];      // per streamed query: (max - lse) in base 2; -delta
  int bh, xblk;
  flash_block(bh, xblk, flash_head_group(a.T, D, 2));
  int b = bh / a.H, h = bh % a.H;
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 31, lk = lane >> 5;
  int kv_blk0 = xblk * 128, kv0 = kv_blk0 + wave * 32, kvi = kv0 + lr;
  const uint16_t *Q = (const uint16_t *)a.q + b * a.q_sb + h * a.q_sh;
  const uint16_t *K = (const uint16_t *)a.k + b * a.k_sb + h * a.k_sh;
  const uint16_t *V = (const uint16_t *)a.v + b * a.v_sb + h * a.v_sh;
  const uint16_t *dO = (const uint16_t *)a.d_o + b * a.o_sb + h * a.o_sh;
  const float c1 = CAPPED ? 2.0f * a.scale * LOG2E / a.cap : a.scale * LOG2E;
  const float c2 = -2.0f * a.cap * LOG2E;
  const float lse_max = CAPPED ? a.cap : 0.f;
  bool live = kvi < a.T;
  bf16x8 kf[KS], vf[KS];
  row_frags<D, PAD>(K, a.k_st, kvi, live, lane, kf, a.hd);
  row_frags<D, PAD>(V, a.v_st, kvi, live, lane, vf, a.hd);
  f32x16 dk[DB], dv[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int e = 0; e < 16; e++) { dk[d][e] = 0.f; dv[d][e] = 0.f; }

  int64_t srow0 = ((int64_t)b * a.H + h) * a.T;
  int q_first = (kv_blk0 / ST) * ST;                               // causal: queries at or after this block's first key
  int ntile = (a.T - q_first + ST - 1) / ST;
  u32x4 rq[Geo<D>::CHUNKS], rdo[Geo<D>::CHUNKS];
  float rl = 0.f, rd = 0.f;
  // rows past the end of the sequence carry zero Q / dO and finite statistics, so they contribute exact zeros
  auto load_stats = [&](int q_base) {
    if (threadIdx.x < ST) {
      int qi = q_base + threadIdx.x;
      rl = qi < a.T ? (lse_max - a.lse[srow0 + qi]) * LOG2E : 0.f;
      rd = qi < a.T ? -a.delta[srow0 + qi] : 0.f;
    }
  };
  tile_load<D, PAD>(Q, a.q_st, q_first, a.T, rq, a.hd);
  tile_load<D, PAD>(dO, a.o_st, q_first, a.T, rdo, a.hd);
  load_stats(q_first);
  tile_store<D>(Qs[0], rq);
  tile_store<D>(dOs[0], rdo);
  if (threadIdx.x < ST) { Ls[0][threadIdx.x] = rl; Ds[0][threadIdx.x] = rd; }
  __syncthreads();
  for (int it = 0; it < ntile; it++) {
    int cur = it & 1;
    if (it + 1 < ntile) {
      tile_load<D, PAD>(Q, a.q_st, q_first + (it + 1) * ST, a.T, rq, a.hd);
      tile_load<D, PAD>(dO, a.o_st, q_first + (it + 1) * ST, a.T, rdo, a.hd);
      load_stats(q_first + (it + 1) * ST);
    }
#pragma unroll
    for (int sub = 0; sub < ST / 32; sub++) {
      int qs = q_first + it * ST + sub * 32;
      if (qs + 31 >= kv0 && qs < a.T) {                            // otherwise every query of the sub-tile precedes this wave's keys
        f32x16 s, dp;
#pragma unroll
        for (int j = 0; j < 4; j++) {                              // accumulator rows are queries: dP starts at -delta[query]
          float4 de = *reinterpret_cast<const float4 *>(&Ds[cur][sub * 32 + 8 * j + 4 * lk]);
          s[4 * j] = 0.f; s[4 * j + 1] = 0.f; s[4 * j + 2] = 0.f; s[4 * j + 3] = 0.f;
          dp[4 * j] = de.x; dp[4 * j + 1] = de.y; dp[4 * j + 2] = de.z; dp[4 * j + 3] = de.w;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {                          // rows = queries, columns = this wave's keys
          s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag<D>(Qs[cur], sub * 32, ks, lane), kf[ks], s, 0, 0, 0);
          dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag<D>(dOs[cur], sub * 32, ks, lane), vf[ks], dp, 0, 0, 0);
        }
        const bool edge = qs < kv0 + 31;                           // wave-uniform: some query of the tile precedes some key
#pragma unroll
        for (int j = 0; j < 4; j++) {
          float4 kr = *reinterpret_cast<const float4 *>(&Ls[cur][sub * 32 + 8 * j + 4 * lk]);
          float krv[4] = {kr.x, kr.y, kr.z, kr.w};
#pragma unroll
          for (int r = 0; r < 4; r++) {
            int e = 4 * j + r;
            float ds;
            float p = score_bwd<CAPPED>(s[e], dp[e], krv[r], c1, c2, ds);
            dp[e] = p;
            s[e] = ds;
          }
        }
        if (edge) {
#pragma unroll
          for (int e = 0; e < 16; e++) {
            int qi = qs + 8 * (e >> 2) + 4 * lk + (e & 3);
            bool dead = kvi > qi;
            dp[e] = dead ? 0.f : dp[e];
            s[e] = dead ? 0.f : s[e];
          }
        }
        bf16x8 p0 = acc_to_b(dp, 0), p1 = acc_to_b(dp, 1), d0 = acc_to_b(s, 0), d1 = acc_to_b(s, 1);
#pragma unroll
        for (int d = 0; d < DB; d++) {
          dv[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(dOs[cur], sub * 32, 0, d, lane), p0, dv[d], 0, 0, 0);   // dV^T[d, kv]
          dv[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(dOs[cur], sub * 32, 1, d, lane), p1, dv[d], 0, 0, 0);
          dk[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Qs[cur], sub * 32, 0, d, lane), d0, dk[d], 0, 0, 0);    // dK^T[d, kv]
          dk[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Qs[cur], sub * 32, 1, d, lane), d1, dk[d], 0, 0, 0);
        }
      }
    }
    if (it + 1 < ntile) {
      tile_store<D>(Qs[cur ^ 1], rq);
      tile_store<D>(dOs[cur ^ 1], rdo);
      if (threadIdx.x < ST) { Ls[cur ^ 1][threadIdx.x] = rl; Ds[cur ^ 1][threadIdx.x] = rd; }
    }
    __syncthreads();
  }
  if (live) {
    store_rows<D, PAD>((uint16_t *)a.dk + b * a.k_sb + h * a.k_sh + (int64_t)kvi * a.k_st, dk, CAPPED ? 4.0f * a.scale : a.scale, lane, a.hd);
    store_rows<D, PAD>((uint16_t *)a.dv + b * a.v_sb + h * a.v_sh + (int64_t)kvi * a.v_st, dv, 1.0f, lane, a.hd);
  }
}
// (two waves per SIMD at head size 64: 212 registers, of which the two output accumulators are 64; three at head size 32)
template <int D, bool CAPPED>
__global__ __launch_bounds__(256, D <= 32 ? 3 : D <= 64 ? 2 : 1) void k_flash_dkv_bf16(FlashArgs a) { flash_dkv_bf16_body<D, CAPPED, false>(a); }
// the same for tensors whose head size is smaller than D
template <int D, bool CAPPED>
__global__ __launch_bounds__(256, D <= 32 ? 3 : D <= 64 ? 2 : 1) void k_flash_dkv_bf16_padded(FlashArgs a) { flash_dkv_bf16_body<D, CAPPED, true>(a); }

// ------------------------------------------------------------------------------------------ backward, one pass over the scores
// The dQ / dK,dV pair above evaluates every probability and every score gradient twice, and that per-score arithmetic is what
// bounds both kernels.  Here a workgroup of 8 waves owns 256 keys of one head (a wave 32 of them, as in k_flash_dkv_bf16) and
// streams the queries at or after them once: P and dS are computed once, dV and dK accumulate in registers as before, and dS
// also feeds dQ:
//   * each wave leaves its 32 keys x 32 queries of dS (bf16, the operand the dK product has just consumed) in LDS as
//     [key][query]; a transposing read of that tile is exactly the B operand (column = query, k-slots = keys) of
//     dQ^T[d, q] += K^T[d, kv] dS^T[kv, q];
//   * for every 32-query sub-tile ONE wave contracts over all 256 keys of the workgroup (K^T fragments from the workgroup's K
//     block in LDS, dS^T fragments from the 8 waves' tiles): no sum across waves is needed, and the order of the additions is
//     fixed.  That duty moves between the two halves of the workgroup from tile to tile and runs one tile behind, while the
//     other waves are already in the score arithmetic of the next tile;
//   * what a workgroup gets is the part of dQ that comes from its 256 keys: it goes to dq_part[head][key block][query][d]
//     (f32), and k_flash_dq_reduce adds the parts of a query in key-block order, applies the constant factor and rounds to
//     bf16.  No atomics anywhere: the result is the same from run to run.
// delta = rowsum(dO * O) is taken from the O tile as it is streamed in.
constexpr int FW = 8;                   // waves per workgroup
constexpr int FKB = FW * 32;            // keys per workgroup
constexpr int FSP = Geo<32>::PITCH;     // pitch of a dS tile [32 keys][32 queries]

template <int D, bool CAPPED>
__global__ __launch_bounds__(512, 1) void k_flash_bwd_fused_bf16(FlashArgs a, float *__restrict__ dq_part) {
  constexpr int DB = D / 32, KS = D / 16, CPR = D / 8;             // CPR: 16-byte chunks per row
  constexpr int TCH = ST * CPR, TPT = (TCH + 511) / 512;           // chunks per streamed tile, per thread
  constexpr int ND = 2 * DB;                                       // dQ duties per tile: (sub-tile, block of 32 features)
  static_assert(ND <= FW, "one duty per wave at most");
  __shared__ __attribute__((aligned(16))) uint16_t Qs[2][Geo<D>::ELEMS], dOs[2][Geo<D>::ELEMS];
  __shared__ __attribute__((aligned(16))) float Ls[2][ST], Ds[2][ST];
  __shared__ __attribute__((aligned(16))) uint16_t Kb[FKB * Geo<D>::PITCH];
  __shared__ __attribute__((aligned(16))) uint16_t dSs[2][FW][32 * FSP];
  int bh, kb;
  flash_block(bh, kb, flash_head_group(a.T, D, 2));
  const int nkb = gridDim.x;
  const int b = bh / a.H, h = bh % a.H;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 31, lk = lane >> 5;
  const int kv_blk0 = kb * FKB, kv0 = kv_blk0 + wave * 32, kvi = kv0 + lr;
  const uint16_t *Q = (const uint16_t *)a.q + b * a.q_sb + h * a.q_sh;
  const uint16_t *K = (const uint16_t *)a.k + b * a.k_sb + h * a.k_sh;
  const uint16_t *V = (const uint16_t *)a.v + b * a.v_sb + h * a.v_sh;
  const uint16_t *O = (const uint16_t *)a.o + b * a.o_sb + h * a.o_sh;
  const uint16_t *dO = (const uint16_t *)a.d_o + b * a.o_sb + h * a.o_sh;
  const float c1 = CAPPED ? 2.0f * a.scale * LOG2E / a.cap : a.scale * LOG2E;
  const float c2 = -2.0f * a.cap * LOG2E;
  const float lse_max = CAPPED ? a.cap : 0.f;
  const bool live = kvi < a.T;
  bf16x8 kf[KS], vf[KS];
  row_frags<D>(K, a.k_st, kvi, live, lane, kf);
  row_frags<D>(V, a.v_st, kvi, live, lane, vf);
  // the workgroup's K block as it lies, for the K^T fragments of the dQ product (keys past the end of the sequence are zero)
  for (int c = threadIdx.x; c < FKB * CPR; c += 512) {
    int r = c / CPR, c8 = c % CPR;
    u32x4 x = {0u, 0u, 0u, 0u};
    if (kv_blk0 + r < a.T) x = *reinterpret_cast<const u32x4 *>(K + (int64_t)(kv_blk0 + r) * a.k_st + c8 * 8);
    *reinterpret_cast<u32x4 *>(Kb + r * Geo<D>::PITCH + c8 * 8) = x;
  }
  f32x16 dk[DB], dv[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int e = 0; e < 16; e++) { dk[d][e] = 0.f; dv[d][e] = 0.f; }

  const int64_t srow0 = ((int64_t)b * a.H + h) * a.T;
  const int q_first = kv_blk0;                                     // a multiple of the streamed tile: causal start
  const int ntile = (a.T - q_first + ST - 1) / ST;
  float *part = dq_part + ((int64_t)bh * nkb + kb) * a.T * D;
  u32x4 rq[TPT], rdo[TPT], ro[TPT];
  float rl = 0.f;
  auto load_tile = [&](int q_base) {
#pragma unroll
    for (int i = 0; i < TPT; i++) {
      int c = threadIdx.x + 512 * i, r = c / CPR, c8 = c % CPR;
      u32x4 z = {0u, 0u, 0u, 0u};
      rq[i] = z; rdo[i] = z; ro[i] = z;
      if (c < TCH && q_base + r < a.T) {
        rq[i] = *reinterpret_cast<const u32x4 *>(Q + (int64_t)(q_base + r) * a.q_st + c8 * 8);
        rdo[i] = *reinterpret_cast<const u32x4 *>(dO + (int64_t)(q_base + r) * a.o_st + c8 * 8);
        ro[i] = *reinterpret_cast<const u32x4 *>(O + (int64_t)(q_base + r) * a.o_st + c8 * 8);
      }
    }
    if (threadIdx.x < ST) {
      int qi = q_base + threadIdx.x;
      rl = qi < a.T ? (lse_max - a.lse[srow0 + qi]) * LOG2E : 0.f;
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TPT; i++) {
      int c = threadIdx.x + 512 * i, r = c / CPR, c8 = c % CPR;
      // delta of the row: the CPR lanes that hold its chunks are neighbours
      bf16x8 vo = __builtin_bit_cast(bf16x8, ro[i]), vd = __builtin_bit_cast(bf16x8, rdo[i]);
      float dsum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) dsum += (float)vd[e] * (float)vo[e];
#pragma unroll
      for (int o = 1; o < CPR; o <<= 1) dsum += __shfl_xor(dsum, o, 64);
      if (c < TCH) {
        *reinterpret_cast<u32x4 *>(&Qs[buf][r * Geo<D>::PITCH + c8 * 8]) = rq[i];
        *reinterpret_cast<u32x4 *>(&dOs[buf][r * Geo<D>::PITCH + c8 * 8]) = rdo[i];
        if (c8 == 0) Ds[buf][r] = -dsum;
      }
    }
    if (threadIdx.x < ST) Ls[buf][threadIdx.x] = rl;
  };
  // scores of one 32-query sub-tile against this wave's keys: P and dS as bf16 MFMA operands.  false: nothing to do
  auto scores = [&](int cur, int sub, int qs, bf16x8 &p0, bf16x8 &p1, bf16x8 &d0, bf16x8 &d1) -> bool {
    if (!(qs + 31 >= kv0 && qs < a.T)) return false;
    f32x16 s, dp;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      float4 de = *reinterpret_cast<const float4 *>(&Ds[cur][sub * 32 + 8 * j + 4 * lk]);
      s[4 * j] = 0.f; s[4 * j + 1] = 0.f; s[4 * j + 2] = 0.f; s[4 * j + 3] = 0.f;
      dp[4 * j] = de.x; dp[4 * j + 1] = de.y; dp[4 * j + 2] = de.z; dp[4 * j + 3] = de.w;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag<D>(Qs[cur], sub * 32, ks, lane), kf[ks], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag<D>(dOs[cur], sub * 32, ks, lane), vf[ks], dp, 0, 0, 0);
    }
    const bool edge = qs < kv0 + 31 || kv0 + 32 > a.T;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      float4 kr = *reinterpret_cast<const float4 *>(&Ls[cur][sub * 32 + 8 * j + 4 * lk]);
      float krv[4] = {kr.x, kr.y, kr.z, kr.w};
#pragma unroll
      for (int r = 0; r < 4; r++) {
        int e = 4 * j + r;
        float ds;
        float p = score_bwd<CAPPED>(s[e], dp[e], krv[r], c1, c2, ds);
        dp[e] = p;
        s[e] = ds;
      }
    }
    if (edge) {
#pragma unroll
      for (int e = 0; e < 16; e++) {
        int qi = qs + 8 * (e >> 2) + 4 * lk + (e & 3);
        bool dead = kvi > qi || kvi >= a.T;                        // dS of a key past the end must not reach dQ
        dp[e] = dead ? 0.f : dp[e];
        s[e] = dead ? 0.f : s[e];
      }
    }
    p0 = acc_to_b(dp, 0); p1 = acc_to_b(dp, 1); d0 = acc_to_b(s, 0); d1 = acc_to_b(s, 1);
    return true;
  };
  // dV, dK from the operands, and dS into this wave's LDS tile as [key][query]
  auto accumulate = [&](int cur, int sub, const bf16x8 &p0, const bf16x8 &p1, const bf16x8 &d0, const bf16x8 &d1) {
    uint16_t *t = dSs[sub][wave] + lr * FSP + 4 * lk;
    const uint2 *w0 = reinterpret_cast<const uint2 *>(&d0), *w1 = reinterpret_cast<const uint2 *>(&d1);
    *reinterpret_cast<uint2 *>(t) = w0[0];                         // queries 4 lk .. +3
    *reinterpret_cast<uint2 *>(t + 8) = w0[1];                     // 8 + 4 lk ..
    *reinterpret_cast<uint2 *>(t + 16) = w1[0];
    *reinterpret_cast<uint2 *>(t + 24) = w1[1];
#pragma unroll
    for (int d = 0; d < DB; d++) {
      dv[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(dOs[cur], sub * 32, 0, d, lane), p0, dv[d], 0, 0, 0);
      dv[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(dOs[cur], sub * 32, 1, d, lane), p1, dv[d], 0, 0, 0);
      dk[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Qs[cur], sub * 32, 0, d, lane), d0, dk[d], 0, 0, 0);
      dk[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Qs[cur], sub * 32, 1, d, lane), d1, dk[d], 0, 0, 0);
    }
  };
  // the dQ duty of tile t: this wave's (sub-tile, feature block) over all keys of the workgroup
  auto dq_duty = [&](int t) {
    const int di = (wave + ((t & 1) ? FW / 2 : 0)) % FW;
    if (di >= ND) return;
    const int sub = di / DB, db = di % DB;
    const int qs = q_first + t * ST + sub * 32;
    if (qs >= a.T) return;
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
#pragma unroll
    for (int wv = 0; wv < FW; wv++) {
      if (qs + 31 >= kv_blk0 + wv * 32) {                          // the waves that wrote a tile for this sub-tile
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Kb, wv * 32, 0, db, lane), tile_frag_t<32>(dSs[sub][wv], 0, 0, 0, lane), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tile_frag_t<D>(Kb, wv * 32, 1, db, lane), tile_frag_t<32>(dSs[sub][wv], 0, 1, 0, lane), acc, 0, 0, 0);
      }
    }
    const int qi = qs + lr;                                        // accumulator column = query, rows = features 32 db + 8 j + 4 lk + r
    if (qi < a.T) {
      float *dst = part + (int64_t)qi * D + 32 * db + 4 * lk;
#pragma unroll
      for (int j = 0; j < 4; j++)
        *reinterpret_cast<float4 *>(dst + 8 * j) = make_float4(acc[4 * j], acc[4 * j + 1], acc[4 * j + 2], acc[4 * j + 3]);
    }
  };

  load_tile(q_first);
  store_tile(0);
  __syncthreads();
  for (int it = 0; it < ntile; it++) {
    const int cur = it & 1;
    const int qs0 = q_first + it * ST;
    if (it + 1 < ntile) load_tile(q_first + (it + 1) * ST);
    if (it > 0) dq_duty(it - 1);                                   // reads the dS tiles of the previous query tile
    bf16x8 p0, p1, d0, d1;
    const bool on0 = scores(cur, 0, qs0, p0, p1, d0, d1);
    __syncthreads();                                               // every duty has read: the dS tiles may be overwritten
    if (on0) accumulate(cur, 0, p0, p1, d0, d1);
    if (scores(cur, 1, qs0 + 32, p0, p1, d0, d1)) accumulate(cur, 1, p0, p1, d0, d1);
    if (it + 1 < ntile) store_tile(cur ^ 1);
    __syncthreads();                                               // dS tiles of this query tile and the next Q / dO tile are in place
  }
  dq_duty(ntile - 1);
  if (live) {
    store_rows<D>((uint16_t *)a.dk + b * a.k_sb + h * a.k_sh + (int64_t)kvi * a.k_st, dk, CAPPED ? 4.0f * a.scale : a.scale, lane);
    store_rows<D>((uint16_t *)a.dv + b * a.v_sb + h * a.v_sh + (int64_t)kvi * a.v_st, dv, 1.0f, lane);
  }
}

// dq[q] = factor * sum over the key blocks at or before q of dq_part[key block][q], in key-block order, rounded to bf16
template <int D>
__global__ __launch_bounds__(256) void k_flash_dq_reduce(FlashArgs a, const float *__restrict__ dq_part, int nkb, float factor) {
  constexpr int TPR = D / 4;                                       // threads per query row
  const int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t row = idx / TPR;
  const int d4 = (int)(idx % TPR) * 4;
  if (row >= (int64_t)a.B * a.H * a.T) return;
  const int q = (int)(row % a.T), bh = (int)(row / a.T), b = bh / a.H, h = bh % a.H;
  const float *src = dq_part + ((int64_t)bh * nkb * a.T + q) * D + d4;
  float4 acc = *reinterpret_cast<const float4 *>(src);
  const int last = q / FKB;
  for (int kb = 1; kb <= last; kb++) {
    float4 x = *reinterpret_cast<const float4 *>(src + (int64_t)kb * a.T * D);
    acc.x += x.x; acc.y += x.y; acc.z += x.z; acc.w += x.w;
  }
  uint2 w = make_uint2(pack_bf16x2(acc.x * factor, acc.y * factor), pack_bf16x2(acc.z * factor, acc.w * factor));
  *reinterpret_cast<uint2 *>((uint16_t *)a.dq + b * a.q_sb + h * a.q_sh + (int64_t)q * a.q_st + d4) = w;
}

template <int D, bool CAPPED>
int32_t run_fwd(const FlashArgs &a) {
  dim3 grid((unsigned)cdiv(a.T, 128), (unsigned)(a.B * a.H));
  if (a.hd == D) ah::launch_kernel((k_flash_fwd_bf16<D, CAPPED>), grid, dim3(256), 0, a);
  else ah::launch_kernel((k_flash_fwd_bf16_padded<D, CAPPED>), grid, dim3(256), 0, a);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
template <int D, bool CAPPED>
int32_t run_bwd_fused(FlashArgs &a) {
  const int nkb = (int)cdiv(a.T, FKB);
  const int64_t rows = (int64_t)a.B * a.H * a.T;
  ah_ptr part = 0;
  int32_t rc = ah_alloc((uint64_t)rows * nkb * D * 4, &part);
  if (rc) return rc;
  ah::launch_kernel(k_flash_bwd_fused_bf16<D, CAPPED>, dim3((unsigned)nkb, (unsigned)(a.B * a.H)), dim3(512), 0, a, dp<float>(part));
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_flash_dq_reduce<D>, dim3((unsigned)cdiv(rows * (D / 4), 256)), dim3(256), 0, a, dp<const float>(part), nkb,
                    CAPPED ? 4.0f * a.scale : a.scale);
  AH_LAUNCH_CHECK();
  return ah_free(part);
}
// AhFlash::bwd_variant = 1 selects the one-pass kernel (head sizes up to 64) instead of the dQ + dK/dV pair; both give the same
// results to bf16 rounding.  The pair is the default: at B = 16, H = 12, T = 1024 it takes 192-208 us against 196-210 us.
template <int D, bool CAPPED>
int32_t run_bwd(FlashArgs &a) {
  if constexpr (D <= 64) {
    if (a.hd == D && (a.variant == 1 || flash_bwd_one_pass())) return run_bwd_fused<D, CAPPED>(a);      // (the one-pass kernel takes whole head sizes only)
  }
  int64_t rows = (int64_t)a.B * a.H * a.T;
  ah_ptr delta = 0;
  int32_t rc = ah_alloc((uint64_t)rows * 4, &delta);
  if (rc) return rc;
  a.delta = dp<float>(delta);
  dim3 grid((unsigned)cdiv(a.T, 128), (unsigned)(a.B * a.H));
  if (a.hd == D) ah::launch_kernel((k_flash_dq_bf16<D, CAPPED>), grid, dim3(256), 0, a);      // also writes delta
  else ah::launch_kernel((k_flash_dq_bf16_padded<D, CAPPED>), grid, dim3(256), 0, a);
  AH_LAUNCH_CHECK();
  if (a.hd == D) ah::launch_kernel((k_flash_dkv_bf16<D, CAPPED>), grid, dim3(256), 0, a);
  else ah::launch_kernel((k_flash_dkv_bf16_padded<D, CAPPED>), grid, dim3(256), 0, a);
  AH_LAUNCH_CHECK();
  return ah_free(delta);
}
template <int D>
int32_t run_fwd_d(const FlashArgs &a) {
  return a.cap > 0.f && a.cap <= FIXED_MAX_CAP ? run_fwd<D, true>(a) : run_fwd<D, false>(a);
}
template <int D>
int32_t run_bwd_d(FlashArgs &a) {
  return a.cap > 0.f && a.cap <= FIXED_MAX_CAP ? run_bwd<D, true>(a) : run_bwd<D, false>(a);
}

}  // namespace

namespace ah {

int32_t flash_fwd_bf16(const FlashArgs &a, int head_dim) {
  switch (head_dim) {
    case 32: return run_fwd_d<32>(a);
    case 64: return run_fwd_d<64>(a);
    default: return run_fwd_d<128>(a);
  }
}
int32_t flash_bwd_bf16(FlashArgs &a, int head_dim) {
  switch (head_dim) {
    case 32: return run_bwd_d<32>(a);
    case 64: return run_bwd_d<64>(a);
    default: return run_bwd_d<128>(a);
  }
}

}  // namespace ah
