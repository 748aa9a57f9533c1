// Fused causal flash attention, forward and backward, on the gfx950 matrix cores.
//
// Semantics (packages/helios/src/kernels/attention.ts:1-586; CPU chain packages/model/src/gpt.ts:255-279):
//   s = scale * q.k;  s = cap * tanh(s / cap) when cap > 0;  keys after the query are masked;
//   P = softmax(s);  O = P V;  LSE = max + log(sum exp).
//
// fp32 path: v_mfma_f32_32x32x2_f32.  One wave owns 32 query rows (forward, dQ) or 32 key rows (dK/dV)
// and the products are arranged so that the owned index is the accumulator COLUMN (= lane % 32):
//   forward / dQ : S^T[kv, q] = K Q^T, so a lane holds 16 kv entries of one query row and the running
//                  max / sum / rescale are per-lane scalars (one cross-half shuffle per tile);
//                  O^T[d, q] += V^T[d, kv] P^T[kv, q] takes P^T straight from the accumulator registers.
//   dK / dV      : S[q, kv] = Q K^T with the key as column; dV^T += dO^T P and dK^T += Q^T dS likewise.
// An accumulator element e of a 32x32 tile sits at row 8*(e/4) + 4*(lane/32) + e%4, column lane%32, and
// MFMA number (j, r) of a 32-deep contraction contracts rows {8j + r, 8j + 4 + r}: half lane/32 = h owns
// row 8j + 4h + r in the accumulator and must supply exactly that row as operand -> no data movement.
#include "attention_common.h"

using namespace ah;

namespace {

constexpr int BC = 32;     // rows of the streamed tile per iteration
constexpr int WAVES = 4;   // 4 waves x 32 owned rows = 128 rows per block

__device__ __forceinline__ float softcap_fwd(float s, float cap, float inv_cap) { return cap > 0.f ? tanhf(s * inv_cap) * cap : s; }

// cooperative load of a [32 x D] f32 tile (rows row0.., zero beyond `rows` and beyond feature hd) into LDS with pitch D+1
template <int D>
__device__ __forceinline__ void load_tile_f32(float *s, const float *__restrict__ base, int64_t st, int row0, int rows, float mul, int hd) {
  constexpr int P = D + 1, V4 = D / 4;
  for (int c = threadIdx.x; c < BC * V4; c += blockDim.x) {
    int r = c / V4, d4 = c % V4;
    float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row0 + r < rows && d4 * 4 < hd) x = *reinterpret_cast<const float4 *>(base + (int64_t)(row0 + r) * st + d4 * 4);
    float *p = s + r * P + d4 * 4;
    p[0] = x.x * mul; p[1] = x.y * mul; p[2] = x.z * mul; p[3] = x.w * mul;
  }
}

// ------------------------------------------------------------------------------------------ forward
template <int D>
__global__ __launch_bounds__(256) void k_flash_fwd_f32(FlashArgs a) {
  constexpr int P = D + 1, DB = D / 32;
  __shared__ float Ks[BC * P], Vs[BC * P];
  int bh, xblk;
  flash_block(bh, xblk, flash_head_group(a.T, D, 4));
  xblk = gridDim.x - 1 - xblk;                                     // longest (latest) query blocks are scheduled first
  int b = bh / a.H, h = bh % a.H;
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 31, lk = lane >> 5;
  int q0 = xblk * (WAVES * 32) + wave * 32, qi = q0 + lr;
  const float *Q = (const float *)a.q + b * a.q_sb + h * a.q_sh;
  const float *K = (const float *)a.k + b * a.k_sb + h * a.k_sh;
  const float *V = (const float *)a.v + b * a.v_sb + h * a.v_sh;
  float inv_cap = a.cap > 0.f ? 1.0f / a.cap : 0.f;

  float qreg[D / 2];                                  // Q[qi][2i + lk] * scale
#pragma unroll
  for (int i = 0; i < D / 2; i++) qreg[i] = qi < a.T && 2 * i + lk < a.hd ? Q[(int64_t)qi * a.q_st + 2 * i + lk] * a.scale : 0.f;

  f32x16 o[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int e = 0; e < 16; e++) o[d][e] = 0.f;
  float m = -INFINITY, l = 0.f;

  int q_block_end = min(a.T, (xblk + 1) * (WAVES * 32));   // causal: keys < q_block_end
  for (int kv0 = 0; kv0 < q_block_end; kv0 += BC) {
    __syncthreads();
    load_tile_f32<D>(Ks, K, a.k_st, kv0, a.T, 1.0f, a.hd);
    load_tile_f32<D>(Vs, V, a.v_st, kv0, a.T, 1.0f, a.hd);
    __syncthreads();
    if (kv0 > q0 + 31) continue;                      // whole tile is in this wave's future (uniform per wave)
    f32x16 s;
#pragma unroll
    for (int e = 0; e < 16; e++) s[e] = 0.f;
#pragma unroll
    for (int i = 0; i < D / 2; i++) s = __builtin_amdgcn_mfma_f32_32x32x2f32(Ks[lr * P + 2 * i + lk], qreg[i], s, 0, 0, 0);
    float tmax = -INFINITY;
#pragma unroll
    for (int e = 0; e < 16; e++) {
      int kv = kv0 + 8 * (e >> 2) + 4 * lk + (e & 3);
      float x = softcap_fwd(s[e], a.cap, inv_cap);
      x = (kv > qi || kv >= a.T) ? -INFINITY : x;
      s[e] = x;
      tmax = fmaxf(tmax, x);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    float m_new = fmaxf(m, tmax);
    float m_use = m_new == -INFINITY ? 0.f : m_new;   // rows with nothing visible yet stay at zero weight
    float alpha = expf(m - m_use);
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 16; e++) { float p = expf(s[e] - m_use); s[e] = p; psum += p; }
    psum += __shfl_xor(psum, 32, 64);
    l = l * alpha + psum;
    m = m_new;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int e = 0; e < 16; e++) o[d][e] *= alpha;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int e = 0; e < 16; e++) {                  // MFMA (j = e/4, r = e%4): this half supplies kv row 8j + 4lk + r
        int kvr = 8 * (e >> 2) + 4 * lk + (e & 3);
        o[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(Vs[kvr * P + 32 * d + lr], s[e], o[d], 0, 0, 0);
      }
  }
  if (qi < a.T) {
    float inv_l = l > 0.f ? 1.0f / l : 0.f;
    float *O = (float *)a.o + b * a.o_sb + h * a.o_sh + (int64_t)qi * a.o_st;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float4 w = make_float4(o[d][4 * j] * inv_l, o[d][4 * j + 1] * inv_l, o[d][4 * j + 2] * inv_l, o[d][4 * j + 3] * inv_l);
        if (32 * d + 8 * j + 4 * lk < a.hd) *reinterpret_cast<float4 *>(O + 32 * d + 8 * j + 4 * lk) = w;
      }
    if (lk == 0) a.lse[((int64_t)b * a.H + h) * a.T + qi] = m + logf(l);
  }
}

// delta[b,h,t] = sum_d dO[t,d] * O[t,d]
template <int D>
__global__ void k_flash_delta_f32(FlashArgs a) {
  int64_t row = blockIdx.x * (int64_t)(blockDim.x >> 6) + (threadIdx.x >> 6);
  int64_t total = (int64_t)a.B * a.H * a.T;
  if (row >= total) return;
  int lane = threadIdx.x & 63;
  int t = (int)(row % a.T), h = (int)((row / a.T) % a.H), b = (int)(row / ((int64_t)a.T * a.H));
  const float *O = (const float *)a.o + b * a.o_sb + h * a.o_sh + (int64_t)t * a.o_st;
  const float *dO = (const float *)a.d_o + b * a.o_sb + h * a.o_sh + (int64_t)t * a.o_st;
  float s = 0.f;
  for (int d = lane; d < a.hd; d += 64) s += O[d] * dO[d];
  s = wave_sum(s);
  if (lane == 0) a.delta[row] = s;
}

// ------------------------------------------------------------------------------------------ dQ
template <int D>
__global__ __launch_bounds__(256) void k_flash_dq_f32(FlashArgs a) {
  constexpr int P = D + 1, DB = D / 32;
  __shared__ float Ks[BC * P], Vs[BC * P];
  int bh, xblk;
  flash_block(bh, xblk, flash_head_group(a.T, D, 4));
  xblk = gridDim.x - 1 - xblk;                                     // longest (latest) query blocks are scheduled first
  int b = bh / a.H, h = bh % a.H;
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 31, lk = lane >> 5;
  int q0 = xblk * (WAVES * 32) + wave * 32, qi = q0 + lr;
  const float *Q = (const float *)a.q + b * a.q_sb + h * a.q_sh;
  const float *K = (const float *)a.k + b * a.k_sb + h * a.k_sh;
  const float *V = (const float *)a.v + b * a.v_sb + h * a.v_sh;
  const float *dO = (const float *)a.d_o + b * a.o_sb + h * a.o_sh;
  float inv_cap = a.cap > 0.f ? 1.0f / a.cap : 0.f;
  bool live = qi < a.T;
  float qreg[D / 2], doreg[D / 2];
#pragma unroll
  for (int i = 0; i < D / 2; i++) {
    qreg[i] = live && 2 * i + lk < a.hd ? Q[(int64_t)qi * a.q_st + 2 * i + lk] * a.scale : 0.f;
    doreg[i] = live && 2 * i + lk < a.hd ? dO[(int64_t)qi * a.o_st + 2 * i + lk] : 0.f;
  }
  int64_t srow = ((int64_t)b * a.H + h) * a.T + qi;
  float lse = live ? a.lse[srow] : 0.f, delta = live ? a.delta[srow] : 0.f;

  f32x16 dq[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int e = 0; e < 16; e++) dq[d][e] = 0.f;

  int q_block_end = min(a.T, (xblk + 1) * (WAVES * 32));
  for (int kv0 = 0; kv0 < q_block_end; kv0 += BC) {
    __syncthreads();
    load_tile_f32<D>(Ks, K, a.k_st, kv0, a.T, 1.0f, a.hd);
    load_tile_f32<D>(Vs, V, a.v_st, kv0, a.T, 1.0f, a.hd);
    __syncthreads();
    if (kv0 > q0 + 31) continue;
    f32x16 s, dp;
#pragma unroll
    for (int e = 0; e < 16; e++) { s[e] = 0.f; dp[e] = 0.f; }
#pragma unroll
    for (int i = 0; i < D / 2; i++) {
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(Ks[lr * P + 2 * i + lk], qreg[i], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(Vs[lr * P + 2 * i + lk], doreg[i], dp, 0, 0, 0);
    }
#pragma unroll
    for (int e = 0; e < 16; e++) {
      int kv = kv0 + 8 * (e >> 2) + 4 * lk + (e & 3);
      float sc = softcap_fwd(s[e], a.cap, inv_cap);
      float p = (kv > qi || kv >= a.T || !live) ? 0.f : expf(sc - lse);
      float ds = p * (dp[e] - delta);
      if (a.cap > 0.f) { float t = sc * inv_cap; ds *= (1.0f - t * t); }
      s[e] = ds * a.scale;
    }
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        int kvr = 8 * (e >> 2) + 4 * lk + (e & 3);
        dq[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(Ks[kvr * P + 32 * d + lr], s[e], dq[d], 0, 0, 0);
      }
  }
  if (live) {
    float *dQ = (float *)a.dq + b * a.q_sb + h * a.q_sh + (int64_t)qi * a.q_st;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (32 * d + 8 * j + 4 * lk < a.hd)
          *reinterpret_cast<float4 *>(dQ + 32 * d + 8 * j + 4 * lk) = make_float4(dq[d][4 * j], dq[d][4 * j + 1], dq[d][4 * j + 2], dq[d][4 * j + 3]);
  }
}

// ------------------------------------------------------------------------------------------ dK, dV
template <int D>
__global__ __launch_bounds__(256) void k_flash_dkv_f32(FlashArgs a) {
  constexpr int P = D + 1, DB = D / 32;
  __shared__ float Qs[BC * P], dOs[BC * P], Ls[BC], Ds[BC];
  int bh, xblk;
  flash_block(bh, xblk, flash_head_group(a.T, D, 4));
  int b = bh / a.H, h = bh % a.H;
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 31, lk = lane >> 5;
  int kv_blk0 = xblk * (WAVES * 32), kv0 = kv_blk0 + wave * 32, kvi = kv0 + lr;
  const float *Q = (const float *)a.q + b * a.q_sb + h * a.q_sh;
  const float *K = (const float *)a.k + b * a.k_sb + h * a.k_sh;
  const float *V = (const float *)a.v + b * a.v_sb + h * a.v_sh;
  const float *dO = (const float *)a.d_o + b * a.o_sb + h * a.o_sh;
  float inv_cap = a.cap > 0.f ? 1.0f / a.cap : 0.f;
  bool live = kvi < a.T;
  float kreg[D / 2], vreg[D / 2];
#pragma unroll
  for (int i = 0; i < D / 2; i++) {
    kreg[i] = live && 2 * i + lk < a.hd ? K[(int64_t)kvi * a.k_st + 2 * i + lk] : 0.f;
    vreg[i] = live && 2 * i + lk < a.hd ? V[(int64_t)kvi * a.v_st + 2 * i + lk] : 0.f;
  }
  f32x16 dk[DB], dv[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int e = 0; e < 16; e++) { dk[d][e] = 0.f; dv[d][e] = 0.f; }

  int64_t srow0 = ((int64_t)b * a.H + h) * a.T;
  for (int q0 = kv_blk0; q0 < a.T; q0 += BC) {        // causal: queries at or after this block's first key
    __syncthreads();
    load_tile_f32<D>(Qs, Q, a.q_st, q0, a.T, a.scale, a.hd);
    load_tile_f32<D>(dOs, dO, a.o_st, q0, a.T, 1.0f, a.hd);
    if (threadIdx.x < BC) {
      int qi = q0 + threadIdx.x;
      Ls[threadIdx.x] = qi < a.T ? a.lse[srow0 + qi] : 0.f;
      Ds[threadIdx.x] = qi < a.T ? a.delta[srow0 + qi] : 0.f;
    }
    __syncthreads();
    if (q0 + 31 < kv0) continue;                      // every query of the tile precedes this wave's keys
    f32x16 s, dp;
#pragma unroll
    for (int e = 0; e < 16; e++) { s[e] = 0.f; dp[e] = 0.f; }
#pragma unroll
    for (int i = 0; i < D / 2; i++) {                 // rows = queries, columns = this wave's keys
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(Qs[lr * P + 2 * i + lk], kreg[i], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(dOs[lr * P + 2 * i + lk], vreg[i], dp, 0, 0, 0);
    }
    f32x16 pm;
#pragma unroll
    for (int e = 0; e < 16; e++) {
      int qr = 8 * (e >> 2) + 4 * lk + (e & 3), qi = q0 + qr;
      float sc = softcap_fwd(s[e], a.cap, inv_cap);
      float p = (kvi > qi || qi >= a.T || !live) ? 0.f : expf(sc - Ls[qr]);
      float ds = p * (dp[e] - Ds[qr]);
      if (a.cap > 0.f) { float t = sc * inv_cap; ds *= (1.0f - t * t); }
      pm[e] = p;
      s[e] = ds;                                      // Qs already carries `scale`, so dK = dS^T (scale*Q)
    }
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        int qr = 8 * (e >> 2) + 4 * lk + (e & 3);
        dv[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(dOs[qr * P + 32 * d + lr], pm[e], dv[d], 0, 0, 0);
        dk[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(Qs[qr * P + 32 * d + lr], s[e], dk[d], 0, 0, 0);
      }
  }
  if (live) {
    float *dK = (float *)a.dk + b * a.k_sb + h * a.k_sh + (int64_t)kvi * a.k_st;
    float *dV = (float *)a.dv + b * a.v_sb + h * a.v_sh + (int64_t)kvi * a.v_st;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        if (32 * d + 8 * j + 4 * lk >= a.hd) continue;
        *reinterpret_cast<float4 *>(dK + 32 * d + 8 * j + 4 * lk) = make_float4(dk[d][4 * j], dk[d][4 * j + 1], dk[d][4 * j + 2], dk[d][4 * j + 3]);
        *reinterpret_cast<float4 *>(dV + 32 * d + 8 * j + 4 * lk) = make_float4(dv[d][4 * j], dv[d][4 * j + 1], dv[d][4 * j + 2], dv[d][4 * j + 3]);
      }
  }
}

int32_t check(const AhFlash *f, bool bwd, FlashArgs &a) {
  AH_ARG(f != nullptr, "flash attention: null descriptor");
  AH_ARG(f->dtype == AH_F32 || f->dtype == AH_BF16, "flash attention: dtype %d must be f32 or bf16", f->dtype);
  AH_ARG(f->head_dim >= 8 && f->head_dim <= 128 && f->head_dim % 8 == 0, "flash attention: head_dim %d is not a multiple of 8 from 8 to 128", f->head_dim);
  AH_ARG(f->batch >= 0 && f->heads >= 0 && f->seq >= 0, "flash attention: negative extent");
  AH_ARG((int64_t)f->batch * f->heads <= 65535, "flash attention: batch*heads %lld exceeds 65535", (long long)f->batch * f->heads);
  AH_ARG(f->q && f->k && f->v && f->o && f->lse, "flash attention: null operand");
  const int64_t st[] = {f->q_sb, f->q_sh, f->q_st, f->k_sb, f->k_sh, f->k_st, f->v_sb, f->v_sh, f->v_st, f->o_sb, f->o_sh, f->o_st};
  const int64_t sm = f->dtype == AH_BF16 ? 8 : 4;        // rows are moved in 16-byte pieces
  for (int64_t s : st) AH_ARG(s % sm == 0 && s >= 0, "flash attention: strides must be non-negative multiples of 16 bytes");
  AH_ARG(f->q_st >= f->head_dim && f->k_st >= f->head_dim && f->v_st >= f->head_dim && f->o_st >= f->head_dim,
         "flash attention: row stride smaller than head_dim");
  AH_ARG(aligned16(f->q) && aligned16(f->k) && aligned16(f->v) && aligned16(f->o), "flash attention: operands must be 16-byte aligned");
  if (bwd) {
    AH_ARG(f->d_o && f->dq && f->dk && f->dv, "flash attention backward: null gradient operand");
    AH_ARG(aligned16(f->d_o) && aligned16(f->dq) && aligned16(f->dk) && aligned16(f->dv), "flash attention backward: operands must be 16-byte aligned");
  }
  a.q = dp<const void>(f->q); a.k = dp<const void>(f->k); a.v = dp<const void>(f->v);
  a.o = dp<void>(f->o); a.lse = dp<float>(f->lse);
  a.d_o = dp<const void>(f->d_o); a.dq = dp<void>(f->dq); a.dk = dp<void>(f->dk); a.dv = dp<void>(f->dv);
  a.delta = nullptr; a.variant = f->bwd_variant;
  a.B = f->batch; a.H = f->heads; a.T = f->seq; a.hd = f->head_dim;
  a.q_sb = f->q_sb; a.q_sh = f->q_sh; a.q_st = f->q_st;
  a.k_sb = f->k_sb; a.k_sh = f->k_sh; a.k_st = f->k_st;
  a.v_sb = f->v_sb; a.v_sh = f->v_sh; a.v_st = f->v_st;
  a.o_sb = f->o_sb; a.o_sh = f->o_sh; a.o_st = f->o_st;
  a.scale = f->scale; a.cap = f->soft_cap;
  return AH_OK;
}

template <int D>
int32_t run_fwd(const FlashArgs &a) {
  dim3 grid((unsigned)cdiv(a.T, WAVES * 32), (unsigned)(a.B * a.H));
  ah::launch_kernel(k_flash_fwd_f32<D>, grid, dim3(256), 0, a);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
template <int D>
int32_t run_bwd(FlashArgs &a) {
  int64_t rows = (int64_t)a.B * a.H * a.T;
  ah_ptr delta = 0;
  int32_t rc = ah_alloc((uint64_t)rows * 4, &delta);
  if (rc) return rc;
  a.delta = dp<float>(delta);
  ah::launch_kernel(k_flash_delta_f32<D>, dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, a);
  AH_LAUNCH_CHECK();
  dim3 grid((unsigned)cdiv(a.T, WAVES * 32), (unsigned)(a.B * a.H));
  ah::launch_kernel(k_flash_dq_f32<D>, grid, dim3(256), 0, a);
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_flash_dkv_f32<D>, grid, dim3(256), 0, a);
  AH_LAUNCH_CHECK();
  return ah_free(delta);
}

}  // namespace

extern "C" {

int32_t ah_flash_fwd(const AhFlash *f) {
  AH_REQUIRE_READY();
  FlashArgs a;
  int32_t rc = check(f, false, a);
  if (rc) return rc;
  if (a.B * a.H == 0 || a.T == 0) return AH_OK;
  const int tile_d = f->head_dim <= 32 ? 32 : f->head_dim <= 64 ? 64 : 128;      // the kernels' head size: the features beyond head_dim are zeros
  if (f->dtype == AH_BF16) return flash_fwd_bf16(a, tile_d);
  switch (tile_d) {
    case 32: return run_fwd<32>(a);
    case 64: return run_fwd<64>(a);
    default: return run_fwd<128>(a);
  }
}

int32_t ah_flash_bwd(const AhFlash *f) {
  AH_REQUIRE_READY();
  FlashArgs a;
  int32_t rc = check(f, true, a);
  if (rc) return rc;
  if (a.B * a.H == 0 || a.T == 0) return AH_OK;
  const int tile_d = f->head_dim <= 32 ? 32 : f->head_dim <= 64 ? 64 : 128;
  if (f->dtype == AH_BF16) return flash_bwd_bf16(a, tile_d);
  switch (tile_d) {
    case 32: return run_bwd<32>(a);
    case 64: return run_bwd<64>(a);
    default: return run_bwd<128>(a);
  }
}

}  // extern "C"
