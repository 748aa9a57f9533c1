// Fused AdamW and the device-side clip coefficient (packages/train/src/optimizers.ts:76-92;
// packages/train/src/trainer.ts:1650-1656).  Single pass: 4 f32 reads + 3 f32 writes per element
// (+ one bf16 write when a shadow copy for the next step's MFMA operands is requested).
#include "common.h"

using namespace ah;

namespace {

constexpr int TPB = 256;

__device__ __forceinline__ void adam_one(float &p, float g, float &m, float &v, const AhAdamW &h, float gs) {
  g *= gs;
  if (h.weight_decay > 0.f) p -= h.lr * h.weight_decay * p;
  m = h.beta1 * m + (1.0f - h.beta1) * g;
  v = h.beta2 * v + (1.0f - h.beta2) * g * g;
  float mh = m / h.bc1, vh = v / h.bc2;
  p -= h.lr * mh / (sqrtf(vh) + h.eps);
}

__global__ void k_adamw(float *__restrict__ p, const float *__restrict__ g, float *__restrict__ m, float *__restrict__ v,
                        uint64_t n, AhAdamW h, const AhAdamW *__restrict__ dev_h, const float *__restrict__ dev_scale,
                        uint16_t *__restrict__ shadow, int vec) {
  if (dev_h) { float wd = h.weight_decay; h = *dev_h; h.weight_decay = wd; }   // weight decay stays per tensor
  float gs = h.grad_scale * (dev_scale ? dev_scale[0] : 1.0f);
  // A gradient scale that is not finite means "skip this step" (ah_step_guard writes NaN for a non-finite loss or gradient
  // norm, as the reference trainer skips the optimizer call, trainer.ts:1248-1262,1495-1522): p, m, v and the shadow stay.
  if (!(fabsf(gs) <= 3.4028234e38f)) return;
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  uint64_t start = 0;
  if (vec) {
    uint64_t n4 = n >> 2;
    for (uint64_t i = tid; i < n4; i += stride) {
      // every element is touched once per step: non-temporal loads and stores (measured 5.4 -> 5.7 TB/s)
      typedef float f4 __attribute__((ext_vector_type(4)));
      typedef unsigned u2 __attribute__((ext_vector_type(2)));
      f4 pp = __builtin_nontemporal_load(reinterpret_cast<f4 *>(p) + i), gg = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(g) + i);
      f4 mm = __builtin_nontemporal_load(reinterpret_cast<f4 *>(m) + i), vv = __builtin_nontemporal_load(reinterpret_cast<f4 *>(v) + i);
      float pa[4] = {pp.x, pp.y, pp.z, pp.w}, ma[4] = {mm.x, mm.y, mm.z, mm.w}, va[4] = {vv.x, vv.y, vv.z, vv.w};
      adam_one(pa[0], gg.x, ma[0], va[0], h, gs); adam_one(pa[1], gg.y, ma[1], va[1], h, gs);
      adam_one(pa[2], gg.z, ma[2], va[2], h, gs); adam_one(pa[3], gg.w, ma[3], va[3], h, gs);
      pp = f4{pa[0], pa[1], pa[2], pa[3]}; mm = f4{ma[0], ma[1], ma[2], ma[3]}; vv = f4{va[0], va[1], va[2], va[3]};
      __builtin_nontemporal_store(pp, reinterpret_cast<f4 *>(p) + i); __builtin_nontemporal_store(mm, reinterpret_cast<f4 *>(m) + i);
      __builtin_nontemporal_store(vv, reinterpret_cast<f4 *>(v) + i);
      if (shadow) {
        u2 s; s.x = pack_bf16x2(pp.x, pp.y); s.y = pack_bf16x2(pp.z, pp.w);
        __builtin_nontemporal_store(s, reinterpret_cast<u2 *>(shadow) + i);
      }
    }
    start = n4 << 2;
  }
  for (uint64_t i = start + tid; i < n; i += stride) {
    float pp = p[i], mm = m[i], vv = v[i];
    adam_one(pp, g[i], mm, vv, h, gs);
    p[i] = pp; m[i] = mm; v[i] = vv;
    if (shadow) shadow[i] = f32_to_bf16_bits(pp);
  }
}

// The same update for a LIST of tensors in one launch (the table is passed by value): block b works on one chunk of
// AL_CHUNK elements of one tensor, found by bisection of the chunk offsets.  Element arithmetic = k_adamw's.  One float4 per
// thread: measured on the 101 tensors of the 163 M-parameter model, 855 us per pass against 876 / 914 / 962 with 2 / 4 / 16
// iterations per thread (k_adamw on one contiguous array: 864).
constexpr int AL_MAX = 48;
#ifndef AL_CHUNK_LOG2
#define AL_CHUNK_LOG2 10
#endif
constexpr uint64_t AL_CHUNK = uint64_t(1) << AL_CHUNK_LOG2;
struct AdamList {
  float *p[AL_MAX];
  const float *g[AL_MAX];
  float *m[AL_MAX], *v[AL_MAX];
  uint16_t *shadow[AL_MAX];
  uint64_t n[AL_MAX];
  float wd[AL_MAX];
  uint32_t first[AL_MAX + 1];
  int count;
};
__global__ __launch_bounds__(TPB) void k_adamw_list(AdamList L, AhAdamW h, const AhAdamW *__restrict__ dev_h, const float *__restrict__ dev_scale) {
  const uint32_t b = blockIdx.x;
  int lo = 0, hi = L.count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (L.first[mid] <= b) lo = mid; else hi = mid - 1;
  }
  if (dev_h) h = *dev_h;
  h.weight_decay = L.wd[lo];
  const float gs = h.grad_scale * (dev_scale ? dev_scale[0] : 1.0f);
  if (!(fabsf(gs) <= 3.4028234e38f)) return;                      // "skip this step", as in k_adamw
  float *p = L.p[lo], *m = L.m[lo], *v = L.v[lo];
  const float *g = L.g[lo];
  uint16_t *shadow = L.shadow[lo];
  const uint64_t n = L.n[lo], c0 = (uint64_t)(b - L.first[lo]) * AL_CHUNK, c1 = c0 + AL_CHUNK < n ? c0 + AL_CHUNK : n;
  uint64_t start = c0;
  if (((((uintptr_t)p | (uintptr_t)g | (uintptr_t)m | (uintptr_t)v) & 15u) | ((uintptr_t)shadow & 7u)) == 0) {
    const uint64_t q0 = c0 >> 2, q1 = c1 >> 2;
    typedef float f4 __attribute__((ext_vector_type(4)));
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    for (uint64_t i = q0 + threadIdx.x; i < q1; i += TPB) {
      f4 pp = __builtin_nontemporal_load(reinterpret_cast<f4 *>(p) + i), gg = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(g) + i);
      f4 mm = __builtin_nontemporal_load(reinterpret_cast<f4 *>(m) + i), vv = __builtin_nontemporal_load(reinterpret_cast<f4 *>(v) + i);
      float pa[4] = {pp.x, pp.y, pp.z, pp.w}, ma[4] = {mm.x, mm.y, mm.z, mm.w}, va[4] = {vv.x, vv.y, vv.z, vv.w};
      adam_one(pa[0], gg.x, ma[0], va[0], h, gs); adam_one(pa[1], gg.y, ma[1], va[1], h, gs);
      adam_one(pa[2], gg.z, ma[2], va[2], h, gs); adam_one(pa[3], gg.w, ma[3], va[3], h, gs);
      pp = f4{pa[0], pa[1], pa[2], pa[3]}; mm = f4{ma[0], ma[1], ma[2], ma[3]}; vv = f4{va[0], va[1], va[2], va[3]};
      __builtin_nontemporal_store(pp, reinterpret_cast<f4 *>(p) + i); __builtin_nontemporal_store(mm, reinterpret_cast<f4 *>(m) + i);
      __builtin_nontemporal_store(vv, reinterpret_cast<f4 *>(v) + i);
      if (shadow) {
        u2 s; s.x = pack_bf16x2(pp.x, pp.y); s.y = pack_bf16x2(pp.z, pp.w);
        __builtin_nontemporal_store(s, reinterpret_cast<u2 *>(shadow) + i);
      }
    }
    start = q1 << 2;
  }
  for (uint64_t i = start + threadIdx.x; i < c1; i += TPB) {
    float pp = p[i], mm = m[i], vv = v[i];
    adam_one(pp, g[i], mm, vv, h, gs);
    p[i] = pp; m[i] = mm; v[i] = vv;
    if (shadow) shadow[i] = f32_to_bf16_bits(pp);
  }
}

__global__ void k_clip_coef(const float *__restrict__ sumsq, float grad_scale, float clip, float *__restrict__ out) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    float norm = sqrtf(sumsq[0]) * fabsf(grad_scale);
    out[0] = (clip > 0.f && norm > clip) ? clip / norm : 1.0f;
    out[1] = norm;
  }
}

// One thread: the clip coefficient of ah_clip_coef plus the decisions the reference trainer takes on the host between backward
// and the optimizer call.  state (doubles): [0] beta1^t, [1] beta2^t, [2] steps skipped so far.
__global__ void k_step_guard(const float *__restrict__ sumsq, const float *__restrict__ loss, float grad_scale, float clip,
                             double beta1, double beta2, double *__restrict__ state, AhAdamW *__restrict__ hyper,
                             float *__restrict__ out) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  float norm = sqrtf(sumsq[0]) * fabsf(grad_scale);
  bool ok = (fabsf(norm) <= 3.4028234e38f) && (!loss || fabsf(loss[0]) <= 3.4028234e38f);
  out[1] = norm;
  if (!ok) {
    out[0] = __int_as_float(0x7fc00000);
    out[2] = 1.0f;
    state[2] += 1.0;
    return;
  }
  out[0] = (clip > 0.f && norm > clip) ? clip / norm : 1.0f;
  out[2] = 0.0f;
  state[0] *= beta1;                       // running products of the betas advance with applied steps only (optimizers.ts:107-115)
  state[1] *= beta2;
  hyper->bc1 = (float)(1.0 - state[0]);
  hyper->bc2 = (float)(1.0 - state[1]);
}

// ---- Lion, SGD, Adafactor: the reference's host loops (double arithmetic, one rounding per Float32Array store) ----
// No contraction into fused multiply-adds from here on: JavaScript rounds every product.
#pragma clang fp contract(off)
__global__ void k_lion(float *__restrict__ p, const float *__restrict__ g, float *__restrict__ m, uint64_t n, AhLion h) {
  const double decay = h.weight_decay > 0 ? 1.0 - h.lr * h.weight_decay : 1.0;
  uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x;
  if (i >= n) return;
  double gi = (double)g[i] * h.grad_scale, mi = (double)m[i];
  float pi = p[i];
  if (h.weight_decay > 0) pi = (float)((double)pi * decay);
  double update = h.beta1 * mi + (1.0 - h.beta1) * gi;
  double sign = update > 0 ? 1.0 : update < 0 ? -1.0 : update;      // Math.sign keeps +-0 (and NaN)
  p[i] = (float)((double)pi - h.lr * sign);
  m[i] = (float)(h.beta2 * mi + (1.0 - h.beta2) * gi);
}

__global__ void k_sgd(float *__restrict__ p, const float *__restrict__ g, uint64_t n, double lr, double gs) {
  uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x;
  if (i < n) p[i] = (float)((double)p[i] - lr * ((double)g[i] * gs));
}

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
// block-wide sum (256 threads) of doubles; the result is valid in thread 0
__device__ __forceinline__ double block_sum_f64(double v, double *sh) {
  v = wave_sum_f64(v);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  double r = 0;
  if (threadIdx.x == 0) for (int w = 0; w < (int)(blockDim.x >> 6); w++) r += sh[w];
  __syncthreads();
  return r;
}

// one block per row: vr[r] = beta2 vr[r] + (1 - beta2) mean_c (g gs)^2 + eps
__global__ __launch_bounds__(256) void k_af_rows(const float *__restrict__ g, float *__restrict__ vr, int64_t cols, AhAdafactor h) {
  __shared__ double sh[4];
  const float *gr = g + blockIdx.x * cols;
  double s = 0;
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) { double x = (double)gr[c] * h.grad_scale; s += x * x; }
  s = block_sum_f64(s, sh);
  if (threadIdx.x == 0) vr[blockIdx.x] = (float)(h.beta2 * (double)vr[blockIdx.x] + (1.0 - h.beta2) * (s * (1.0 / (double)cols)) + h.eps);
}
// one thread per column, rows in order (the reference's own summation order): vc[c] likewise
__global__ void k_af_cols(const float *__restrict__ g, float *__restrict__ vc, int64_t rows, int64_t cols, AhAdafactor h) {
  int64_t c = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (c >= cols) return;
  double s = 0;
  for (int64_t r = 0; r < rows; r++) { double x = (double)g[r * cols + c] * h.grad_scale; s += x * x; }
  vc[c] = (float)(h.beta2 * (double)vc[c] + (1.0 - h.beta2) * (s * (1.0 / (double)rows)) + h.eps);
}
// ws[0] = 1 / max(mean(vr), eps)
__global__ __launch_bounds__(256) void k_af_vrmean(const float *__restrict__ vr, int64_t rows, double eps, double *__restrict__ ws) {
  __shared__ double sh[4];
  double s = 0;
  for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) s += (double)vr[r];
  s = block_sum_f64(s, sh);
  if (threadIdx.x == 0) { double mean = s * (1.0 / (double)rows); ws[0] = 1.0 / ((mean > eps || mean != mean) ? mean : eps); }      // Math.max(mean, eps): a NaN stays one (optimizers.ts:450)
}
__device__ __forceinline__ double af_denom(const float *vr, const float *vc, int64_t r, int64_t c, double inv_vr_mean, double eps) {
  double d = sqrt((double)vr[r] * inv_vr_mean) * sqrt((double)vc[c]);
  return eps > d ? eps : d;
}
// part[b] = sum over the block's elements of (g gs / denom)^2; FLAT: denom = sqrt(v), after v's own update
template <bool FLAT>
__global__ __launch_bounds__(256) void k_af_update_sq(const float *__restrict__ g, const float *__restrict__ vr, const float *__restrict__ vc,
                                                      float *__restrict__ v, uint64_t n, int64_t cols, AhAdafactor h, const double *__restrict__ ws,
                                                      double *__restrict__ part) {
  __shared__ double sh[4];
  double s = 0;
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    double x = (double)g[i] * h.grad_scale, d;
    if (FLAT) {
      float vi = (float)(h.beta2 * (double)v[i] + (1.0 - h.beta2) * (x * x) + h.eps);
      v[i] = vi;
      d = sqrt((double)vi);
    } else {
      d = af_denom(vr, vc, (int64_t)(i / (uint64_t)cols), (int64_t)(i % (uint64_t)cols), ws[0], h.eps);
    }
    double u = x / d;
    s += u * u;
  }
  s = block_sum_f64(s, sh);
  if (threadIdx.x == 0) part[blockIdx.x] = s;
}
// ws[1] = lr / max(1, rms / clip) with rms = sqrt(sum(part) / max(1, n))
__global__ void k_af_step_scale(const double *__restrict__ part, int nblk, uint64_t n, AhAdafactor h, double *__restrict__ ws) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    double s = 0;
    for (int b = 0; b < nblk; b++) s += part[b];
    double rms = sqrt(s / (double)(n > 1 ? n : 1));
    const double q = rms / h.clip_threshold;
    double den = h.clip_threshold > 0 ? ((q > 1.0 || q != q) ? q : 1.0) : 1.0;      // Math.max(1, rms / clip): a NaN stays one (optimizers.ts:466,499)
    ws[1] = h.lr / den;
  }
}
template <bool FLAT>
__global__ void k_af_apply(float *__restrict__ p, const float *__restrict__ g, const float *__restrict__ vr, const float *__restrict__ vc,
                           const float *__restrict__ v, uint64_t n, int64_t cols, AhAdafactor h, const double *__restrict__ ws) {
  uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x;
  if (i >= n) return;
  const double decay = h.weight_decay > 0 ? 1.0 - h.lr * h.weight_decay : 1.0;
  double x = (double)g[i] * h.grad_scale;
  double d = FLAT ? sqrt((double)v[i]) : af_denom(vr, vc, (int64_t)(i / (uint64_t)cols), (int64_t)(i % (uint64_t)cols), ws[0], h.eps);
  float pi = p[i];
  if (h.weight_decay > 0) pi = (float)((double)pi * decay);
  p[i] = (float)((double)pi - ws[1] * (x / d));
}

// the shared tail of the two Adafactor branches: RMS of the update -> step scale -> parameter update
template <bool FLAT>
int32_t adafactor_tail(ah_ptr p, ah_ptr g, ah_ptr vr, ah_ptr vc, ah_ptr v, uint64_t n, int64_t cols, const AhAdafactor &h, double *ws) {
  int nblk = (int)(cdiv((int64_t)n, TPB) < 1024 ? cdiv((int64_t)n, TPB) : 1024);
  double *part = ws + 2;
  ah::launch_kernel((k_af_update_sq<FLAT>), dim3(nblk), dim3(TPB), 0, dp<const float>(g), dp<const float>(vr), dp<const float>(vc),
                     dp<float>(v), n, cols, h, ws, part);
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_af_step_scale, dim3(1), dim3(64), 0, part, nblk, n, h, ws);
  AH_LAUNCH_CHECK();
  ah::launch_kernel((k_af_apply<FLAT>), dim3((unsigned)cdiv((int64_t)n, TPB)), dim3(TPB), 0, dp<float>(p), dp<const float>(g),
                     dp<const float>(vr), dp<const float>(vc), dp<const float>(v), n, cols, h, ws);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

}  // namespace

extern "C" {

int32_t ah_lion(ah_ptr p, ah_ptr g, ah_ptr m, uint64_t n, const AhLion *h) {
  AH_REQUIRE_READY();
  AH_ARG(h != nullptr, "ah_lion: null hyper-parameters");
  if (n == 0) return AH_OK;
  AH_ARG(p && g && m, "ah_lion: null operand");
  AH_ARG(n < ((uint64_t)1 << 39), "ah_lion: tensor too large");
  ah::launch_kernel(k_lion, dim3((unsigned)cdiv((int64_t)n, TPB)), dim3(TPB), 0, dp<float>(p), dp<const float>(g), dp<float>(m), n, *h);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_sgd(ah_ptr p, ah_ptr g, uint64_t n, double lr, double grad_scale) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(p && g, "ah_sgd: null operand");
  AH_ARG(n < ((uint64_t)1 << 39), "ah_sgd: tensor too large");
  ah::launch_kernel(k_sgd, dim3((unsigned)cdiv((int64_t)n, TPB)), dim3(TPB), 0, dp<float>(p), dp<const float>(g), n, lr, grad_scale);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_adafactor_2d(ah_ptr p, ah_ptr g, ah_ptr vr, ah_ptr vc, int64_t rows, int64_t cols, const AhAdafactor *h) {
  AH_REQUIRE_READY();
  AH_ARG(h != nullptr, "ah_adafactor_2d: null hyper-parameters");
  AH_ARG(rows >= 0 && cols >= 0, "ah_adafactor_2d: negative shape [%lld, %lld]", (long long)rows, (long long)cols);
  if (rows == 0 || cols == 0) return AH_OK;
  AH_ARG(p && g && vr && vc, "ah_adafactor_2d: null operand");
  AH_ARG(rows < ((int64_t)1 << 31) && cols < ((int64_t)1 << 31), "ah_adafactor_2d: shape too large");
  double *ws = (double *)scratch(sizeof(double) * (2 + 1024));
  if (!ws) return fail(AH_ERR_OOM, "ah_adafactor_2d: no scratch");
  ah::launch_kernel(k_af_rows, dim3((unsigned)rows), dim3(TPB), 0, dp<const float>(g), dp<float>(vr), cols, *h);
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_af_cols, dim3((unsigned)cdiv(cols, 64)), dim3(64), 0, dp<const float>(g), dp<float>(vc), rows, cols, *h);
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_af_vrmean, dim3(1), dim3(TPB), 0, dp<const float>(vr), rows, h->eps, ws);
  AH_LAUNCH_CHECK();
  return adafactor_tail<false>(p, g, vr, vc, 0, (uint64_t)rows * (uint64_t)cols, cols, *h, ws);
}

int32_t ah_adafactor_flat(ah_ptr p, ah_ptr g, ah_ptr v, uint64_t n, const AhAdafactor *h) {
  AH_REQUIRE_READY();
  AH_ARG(h != nullptr, "ah_adafactor_flat: null hyper-parameters");
  if (n == 0) return AH_OK;
  AH_ARG(p && g && v, "ah_adafactor_flat: null operand");
  AH_ARG(n < ((uint64_t)1 << 39), "ah_adafactor_flat: tensor too large");
  double *ws = (double *)scratch(sizeof(double) * (2 + 1024));
  if (!ws) return fail(AH_ERR_OOM, "ah_adafactor_flat: no scratch");
  return adafactor_tail<true>(p, g, 0, 0, v, n, 1, *h, ws);
}

int32_t ah_adamw(ah_ptr p, ah_ptr g, ah_ptr m, ah_ptr v, uint64_t n, const AhAdamW *h, ah_ptr dev_hyper, ah_ptr dev_scale,
                 ah_ptr bf16_shadow) {
  AH_REQUIRE_READY();
  AH_ARG(h != nullptr, "ah_adamw: null hyper-parameters");
  if (n == 0) return AH_OK;
  AH_ARG(p && g && m && v, "ah_adamw: null operand");
  int vec = aligned16(p) && aligned16(g) && aligned16(m) && aligned16(v) && ((bf16_shadow & 7u) == 0);
  int64_t blocks = cdiv((int64_t)(vec ? n / 4 + 1 : n), TPB);
  // one float4 group per thread: measured 5.4 TB/s against 4.3 TB/s for a grid of 16 blocks per CU striding over the array
  int64_t cap = (int64_t)1 << 22;
  if (blocks > cap) blocks = cap;
  ah::launch_kernel(k_adamw, dim3((unsigned)blocks), dim3(TPB), 0, dp<float>(p), dp<const float>(g), dp<float>(m),
                     dp<float>(v), n, *h, dp<const AhAdamW>(dev_hyper), dp<const float>(dev_scale), dp<uint16_t>(bf16_shadow), vec);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_adamw_list(const AhAdamWItem *items, int32_t count, const AhAdamW *h, ah_ptr dev_hyper, ah_ptr dev_scale) {
  AH_REQUIRE_READY();
  AH_ARG(h != nullptr, "ah_adamw_list: null hyper-parameters");
  AH_ARG(count >= 0 && (count == 0 || items != nullptr), "ah_adamw_list: bad list");
  for (int i = 0; i < count; i++)
    AH_ARG(items[i].n == 0 || (items[i].p && items[i].g && items[i].m && items[i].v), "ah_adamw_list: null operand in item %d", i);
  int i = 0;
  while (i < count) {
    AdamList L;
    L.count = 0;
    uint64_t nb = 0;
    for (; i < count && L.count < AL_MAX; i++) {
      const AhAdamWItem &it = items[i];
      if (it.n == 0) continue;
      const int k = L.count++;
      L.p[k] = dp<float>(it.p); L.g[k] = dp<const float>(it.g); L.m[k] = dp<float>(it.m); L.v[k] = dp<float>(it.v);
      L.shadow[k] = dp<uint16_t>(it.shadow); L.n[k] = it.n; L.wd[k] = it.weight_decay;
      L.first[k] = (uint32_t)nb;
      nb += (it.n + AL_CHUNK - 1) / AL_CHUNK;
    }
    if (L.count == 0) break;
    AH_ARG(nb < (uint64_t(1) << 31), "ah_adamw_list: too many elements in one launch");
    L.first[L.count] = (uint32_t)nb;
    for (int k = L.count; k < AL_MAX; k++) {
      L.p[k] = nullptr; L.g[k] = nullptr; L.m[k] = nullptr; L.v[k] = nullptr; L.shadow[k] = nullptr; L.n[k] = 0; L.wd[k] = 0.f;
      L.first[k + 1] = (uint32_t)nb;
    }
    ah::launch_kernel(k_adamw_list, dim3((unsigned)nb), dim3(TPB), 0, L, *h, dp<const AhAdamW>(dev_hyper), dp<const float>(dev_scale));
    AH_LAUNCH_CHECK();
  }
  return AH_OK;
}

int32_t ah_clip_coef(ah_ptr sumsq, float grad_scale, float clip, ah_ptr out2) {
  AH_REQUIRE_READY();
  AH_ARG(sumsq && out2, "ah_clip_coef: null operand");
  ah::launch_kernel(k_clip_coef, dim3(1), dim3(64), 0, dp<const float>(sumsq), grad_scale, clip, dp<float>(out2));
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_step_guard(ah_ptr sumsq, ah_ptr loss, float grad_scale, float clip, double beta1, double beta2, ah_ptr state_f64x3,
                      ah_ptr dev_hyper, ah_ptr out3) {
  AH_REQUIRE_READY();
  AH_ARG(sumsq && state_f64x3 && dev_hyper && out3, "ah_step_guard: null operand");
  AH_ARG((state_f64x3 & 7u) == 0, "ah_step_guard: state must be 8-byte aligned");
  ah::launch_kernel(k_step_guard, dim3(1), dim3(64), 0, dp<const float>(sumsq), dp<const float>(loss), grad_scale, clip,
                     beta1, beta2, dp<double>(state_f64x3), dp<AhAdamW>(dev_hyper), dp<float>(out3));
  AH_LAUNCH_CHECK();
  return AH_OK;
}

}  // extern "C"
