// Reductions: sum/mean over an axis or everything, softmax / log-softmax, first-index argmax,
// sum of squares.  All are HBM-bound; accumulation is f64 so results stay within f32 rounding of the
// reference's f64 loops (cpu_ref.ts:260-330, 437-541) at any length.
#include "common.h"

using namespace ah;

namespace {

constexpr int TPB = 256;

__device__ __forceinline__ double block_sum_d(double v, double *sh) {
  v = wave_sum_d(v);
  int w = threadIdx.x >> 6, l = threadIdx.x & 63;
  __syncthreads();
  if (l == 0) sh[w] = v;
  __syncthreads();
  double t = 0;
  for (int i = 0; i < (int)(blockDim.x >> 6); i++) t += sh[i];
  return t;
}
__device__ __forceinline__ float block_max_f(float v, float *sh) {
  v = wave_max(v);
  int w = threadIdx.x >> 6, l = threadIdx.x & 63;
  __syncthreads();
  if (l == 0) sh[w] = v;
  __syncthreads();
  float t = -INFINITY;
  for (int i = 0; i < (int)(blockDim.x >> 6); i++) t = fmaxf(t, sh[i]);
  return t;
}

// line (o, i) = { a[(o*dim + j)*inner + i] : j < dim }.  One block per line.
__global__ void k_sum_lines(const float *__restrict__ a, float *__restrict__ out, int64_t dim, int64_t inner, int mean) {
  __shared__ double sh[TPB / 64];
  int64_t line = blockIdx.x, o = line / inner, i = line % inner;
  const float *p = a + o * dim * inner + i;
  double s = 0;
  for (int64_t j = threadIdx.x; j < dim; j += blockDim.x) s += (double)p[j * inner];
  s = block_sum_d(s, sh);
  if (threadIdx.x == 0) {
    float sf = (float)s;
    out[line] = mean ? (float)((double)sf / (double)dim) : sf;     // mean divides the stored f32 sum (cpu_ref.ts:324-328)
  }
}
// inner > 1 and many lines: one thread per line, coalesced across i.
__global__ void k_sum_strided(const float *__restrict__ a, float *__restrict__ out, int64_t outer, int64_t dim, int64_t inner, int mean) {
  int64_t line = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (line >= outer * inner) return;
  int64_t o = line / inner, i = line % inner;
  const float *p = a + o * dim * inner + i;
  double s = 0;
  for (int64_t j = 0; j < dim; j++) s += (double)p[j * inner];
  float sf = (float)s;
  out[line] = mean ? (float)((double)sf / (double)dim) : sf;
}

// stage 1 of a full reduction: partial[b] = sum over a grid-stride slice; SQ squares first
template <int SQ>
__global__ void k_partial_sum(const float *__restrict__ a, uint64_t n, double *__restrict__ partial) {
  __shared__ double sh[TPB / 64];
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  double s = 0;
  if ((((uintptr_t)a) & 15u) == 0) {
    uint64_t n4 = n >> 2;
    for (uint64_t i = tid; i < n4; i += stride) {
      float4 v = reinterpret_cast<const float4 *>(a)[i];
      if (SQ) s += (double)v.x * v.x + (double)v.y * v.y + (double)v.z * v.z + (double)v.w * v.w;
      else s += ((double)v.x + (double)v.y) + ((double)v.z + (double)v.w);
    }
    for (uint64_t i = (n4 << 2) + tid; i < n; i += stride) { double v = a[i]; s += SQ ? v * v : v; }
  } else {
    for (uint64_t i = tid; i < n; i += stride) { double v = a[i]; s += SQ ? v * v : v; }
  }
  s = block_sum_d(s, sh);
  if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
// stage 1 for a LIST of tensors in one launch: block b sums the squares of one 64 K-element chunk of one tensor (the table is
// passed by value; a block finds its tensor by bisection of the chunk offsets).  The partition depends on the sizes only.
constexpr int SL_MAX = 120;
#ifndef SL_CHUNK_LOG2
#define SL_CHUNK_LOG2 14
#endif
constexpr uint64_t SL_CHUNK = uint64_t(1) << SL_CHUNK_LOG2;
struct SumList {
  const float *x[SL_MAX];
  uint64_t n[SL_MAX];
  uint32_t first[SL_MAX + 1];      // first block of tensor t; first[count] = number of blocks
  int count;
};
__global__ void k_sum_sq_list(SumList L, double *__restrict__ partial) {
  __shared__ double sh[TPB / 64];
  const uint32_t b = blockIdx.x;
  int lo = 0, hi = L.count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (L.first[mid] <= b) lo = mid; else hi = mid - 1;
  }
  const float *a = L.x[lo];
  const uint64_t n = L.n[lo], c0 = (uint64_t)(b - L.first[lo]) * SL_CHUNK, c1 = c0 + SL_CHUNK < n ? c0 + SL_CHUNK : n;
  double s = 0;
  if ((((uintptr_t)a) & 15u) == 0) {                 // chunk starts are multiples of SL_CHUNK elements: as aligned as the tensor
    const uint64_t q0 = c0 >> 2, q1 = c1 >> 2;
    for (uint64_t i = q0 + threadIdx.x; i < q1; i += blockDim.x) {
      float4 v = reinterpret_cast<const float4 *>(a)[i];
      s += (double)v.x * v.x + (double)v.y * v.y + (double)v.z * v.z + (double)v.w * v.w;
    }
    for (uint64_t i = (q1 << 2) + threadIdx.x; i < c1; i += blockDim.x) { double v = a[i]; s += v * v; }
  } else {
    for (uint64_t i = c0 + threadIdx.x; i < c1; i += blockDim.x) { double v = a[i]; s += v * v; }
  }
  s = block_sum_d(s, sh);
  if (threadIdx.x == 0) partial[b] = s;
}
// stage 2: fixed-order sum of the partials by one block
__global__ void k_final_sum(const double *__restrict__ partial, int nparts, float *__restrict__ out, double div) {
  __shared__ double sh[TPB / 64];
  double s = 0;
  for (int i = threadIdx.x; i < nparts; i += blockDim.x) s += partial[i];
  s = block_sum_d(s, sh);
  if (threadIdx.x == 0) out[0] = (float)(s / div);
}

__global__ void k_softmax(const float *__restrict__ a, float *__restrict__ out, int64_t dim, int64_t inner, int logsm) {
  __shared__ double shd[TPB / 64];
  __shared__ float shf[TPB / 64];
  int64_t line = blockIdx.x, o = line / inner, i = line % inner;
  const float *p = a + o * dim * inner + i;
  float *q = out + o * dim * inner + i;
  float m = -INFINITY;
  for (int64_t j = threadIdx.x; j < dim; j += blockDim.x) m = fmaxf(m, p[j * inner]);
  m = block_max_f(m, shf);
  double s = 0;
  for (int64_t j = threadIdx.x; j < dim; j += blockDim.x) s += (double)expf(p[j * inner] - m);
  s = block_sum_d(s, shd);
  if (logsm) {
    float lse = m + (float)log(s);
    for (int64_t j = threadIdx.x; j < dim; j += blockDim.x) q[j * inner] = p[j * inner] - lse;
  } else {
    float inv = (float)(1.0 / s);
    for (int64_t j = threadIdx.x; j < dim; j += blockDim.x) q[j * inner] = expf(p[j * inner] - m) * inv;
  }
}

__global__ void k_softmax_bwd(const float *__restrict__ s, const float *__restrict__ g, float *__restrict__ out, int64_t dim) {
  __shared__ double shd[TPB / 64];
  int64_t row = blockIdx.x;
  const float *sp = s + row * dim, *gp = g + row * dim;
  double dot = 0;
  for (int64_t j = threadIdx.x; j < dim; j += blockDim.x) dot += (double)sp[j] * (double)gp[j];
  dot = block_sum_d(dot, shd);
  float d = (float)dot;
  for (int64_t j = threadIdx.x; j < dim; j += blockDim.x) out[row * dim + j] = sp[j] * (gp[j] - d);
}

// First index of the maximum; strict > from -inf so NaN is never selected (cpu_ref.ts:743-751).
__global__ void k_argmax(const float *__restrict__ a, int32_t *__restrict__ out, int64_t dim, int64_t inner) {
  __shared__ float shv[TPB / 64];
  __shared__ int64_t shi[TPB / 64];
  int64_t line = blockIdx.x, o = line / inner, i = line % inner;
  const float *p = a + o * dim * inner + i;
  float bv = -INFINITY; int64_t bi = 0;
  for (int64_t j = threadIdx.x; j < dim; j += blockDim.x) {   // ascending j per thread: first maximum kept
    float v = p[j * inner];
    if (v > bv) { bv = v; bi = j; }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    float ov = __shfl_xor(bv, off, 64);
    int64_t oi = __shfl_xor(bi, off, 64);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  int w = threadIdx.x >> 6, l = threadIdx.x & 63;
  if (l == 0) { shv[w] = bv; shi[w] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < (int)(blockDim.x >> 6); k++)
      if (shv[k] > bv || (shv[k] == bv && shi[k] < bi)) { bv = shv[k]; bi = shi[k]; }
    out[line] = (int32_t)bi;
  }
}

// Partial sums of ah_sum_sq_static: device memory that exists from load time to process exit, so that entry point never
// allocates.  In host code this name is only a stand-in for the symbol; the device address comes from hipGetSymbolAddress
// (static_partials_init) and is what every launch is given.
constexpr int STATIC_PARTIALS = 4096;
static __device__ __align__(256) double g_static_partials[STATIC_PARTIALS];
constexpr int MAX_DEVICES = 16;
double *g_static_partials_ptr[MAX_DEVICES] = {};

int partial_blocks(uint64_t n) {
  int64_t b = cdiv((int64_t)cdiv((int64_t)n, 4), TPB);
  int64_t cap = (int64_t)num_cus() * 8;
  return (int)(b < 1 ? 1 : (b > cap ? cap : b));
}

}  // namespace

namespace ah {
// Called by ah_init with the device current: each device holds its own copy of the array at its own address.
int32_t static_partials_init(int device) {
  if (device < 0 || device >= MAX_DEVICES) return fail(AH_ERR_ARG, "ah_init: device %d beyond the %d this library keeps static scratch for", device, MAX_DEVICES);
  void *ptr = nullptr;
  hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_partials));
  if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(g_static_partials)");
  g_static_partials_ptr[device] = static_cast<double *>(ptr);
  return AH_OK;
}
}  // namespace ah

extern "C" {

int32_t ah_sum_axis(ah_ptr a, ah_ptr out, int64_t outer, int64_t dim, int64_t inner, int32_t mean) {
  AH_REQUIRE_READY();
  AH_ARG(outer >= 0 && dim >= 0 && inner >= 0, "ah_sum_axis: negative extent");
  int64_t lines = outer * inner;
  if (lines == 0) return AH_OK;
  AH_ARG(a && out, "ah_sum_axis: null operand");
  if (dim == 0) return ah_fill_f32(out, mean ? NAN : 0.f, (uint64_t)lines);      // a sum of no terms; its mean is 0 / 0 (cpu_ref.ts:325-330)
  if (inner > 1 && lines >= 4096) {
    ah::launch_kernel(k_sum_strided, dim3((unsigned)cdiv(lines, TPB)), dim3(TPB), 0, dp<const float>(a),
                       dp<float>(out), outer, dim, inner, mean);
  } else {
    AH_ARG(lines < (int64_t(1) << 31), "ah_sum_axis: too many lines");
    ah::launch_kernel(k_sum_lines, dim3((unsigned)lines), dim3(TPB), 0, dp<const float>(a), dp<float>(out), dim, inner, mean);
  }
  AH_LAUNCH_CHECK();
  return AH_OK;
}

static int32_t full_reduce(ah_ptr a, uint64_t n, ah_ptr out, double div, int sq, const char *who) {
  AH_REQUIRE_READY();
  AH_ARG(out != 0, "%s: null out", who);
  if (n == 0) return ah_fill_f32(out, div == 0.0 ? NAN : 0.f, 1);      // the mean of nothing is 0 / 0 (cpu_ref.ts:317-320)
  AH_ARG(a != 0, "%s: null input", who);
  int nb = partial_blocks(n);
  double *partial = (double *)scratch(sizeof(double) * (size_t)nb);
  if (!partial) return fail(AH_ERR_OOM, "%s: no scratch", who);
  if (sq) ah::launch_kernel(k_partial_sum<1>, dim3(nb), dim3(TPB), 0, dp<const float>(a), n, partial);
  else ah::launch_kernel(k_partial_sum<0>, dim3(nb), dim3(TPB), 0, dp<const float>(a), n, partial);
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_final_sum, dim3(1), dim3(TPB), 0, partial, nb, dp<float>(out), div);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_sum_all(ah_ptr a, ah_ptr out, uint64_t n, int32_t mean) {
  return full_reduce(a, n, out, mean ? (double)n : 1.0, 0, "ah_sum_all");
}
int32_t ah_sum_sq(ah_ptr x, uint64_t n, ah_ptr out) { return full_reduce(x, n, out, 1.0, 1, "ah_sum_sq"); }

int32_t ah_sum_sq_list(const ah_ptr *xs, const uint64_t *ns, int32_t count, ah_ptr out) {
  AH_REQUIRE_READY();
  AH_ARG(out != 0, "ah_sum_sq_list: null out");
  AH_ARG(count >= 0 && (count == 0 || (xs && ns)), "ah_sum_sq_list: bad list");
  uint64_t blocks = 0;
  for (int i = 0; i < count; i++) {
    AH_ARG(ns[i] == 0 || xs[i] != 0, "ah_sum_sq_list: null tensor %d", i);
    blocks += (ns[i] + SL_CHUNK - 1) / SL_CHUNK;
  }
  if (blocks == 0) return ah_fill_f32(out, 0.f, 1);
  AH_ARG(blocks < (uint64_t(1) << 24), "ah_sum_sq_list: too many elements");
  double *partial = (double *)scratch(sizeof(double) * (size_t)blocks);
  if (!partial) return fail(AH_ERR_OOM, "ah_sum_sq_list: no scratch");
  uint32_t done = 0;
  int i = 0;
  while (i < count) {                                // launches of up to SL_MAX non-empty tensors, partial sums side by side
    SumList L;
    L.count = 0;
    uint32_t nb = 0;
    for (; i < count && L.count < SL_MAX; i++) {
      if (ns[i] == 0) continue;
      L.x[L.count] = dp<const float>(xs[i]);
      L.n[L.count] = ns[i];
      L.first[L.count] = nb;
      nb += (uint32_t)((ns[i] + SL_CHUNK - 1) / SL_CHUNK);
      L.count++;
    }
    if (L.count == 0) break;
    L.first[L.count] = nb;
    for (int k = L.count; k < SL_MAX; k++) { L.x[k] = nullptr; L.n[k] = 0; L.first[k + 1] = nb; }
    ah::launch_kernel(k_sum_sq_list, dim3(nb), dim3(TPB), 0, L, partial + done);
    AH_LAUNCH_CHECK();
    done += nb;
  }
  ah::launch_kernel(k_final_sum, dim3(1), dim3(TPB), 0, (const double *)partial, (int)done, dp<float>(out), 1.0);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_sum_sq_static(ah_ptr x, uint64_t n, ah_ptr out) {
  AH_REQUIRE_READY();
  AH_ARG(out != 0, "ah_sum_sq_static: null out");
  AH_ARG(n >= 1, "ah_sum_sq_static: n must be at least 1");
  AH_ARG(n <= (uint64_t(1) << 32), "ah_sum_sq_static: n = %llu exceeds the maximum of 2^32 elements", (unsigned long long)n);
  AH_ARG(x != 0, "ah_sum_sq_static: null input");
  int nb = partial_blocks(n);                       // the same partition as ah_sum_sq: results are bit-identical
  if (nb > STATIC_PARTIALS) return fail(AH_ERR_UNSUPPORTED, "ah_sum_sq_static: %d partial sums exceed the static %d", nb, STATIC_PARTIALS);
  double *partial = g_static_partials_ptr[current_device()];
  if (!partial) return fail(AH_ERR_STATE, "ah_sum_sq_static: static scratch of device %d was not set up", current_device());
  // partial[0, nb) is written in full by the first kernel before the second reads exactly that range: nothing to clear.
  ah::launch_kernel(k_partial_sum<1>, dim3(nb), dim3(TPB), 0, dp<const float>(x), n, partial);
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_final_sum, dim3(1), dim3(TPB), 0, partial, nb, dp<float>(out), 1.0);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_softmax(ah_ptr a, ah_ptr out, int64_t outer, int64_t dim, int64_t inner, int32_t log_softmax) {
  AH_REQUIRE_READY();
  int64_t lines = outer * inner;
  if (lines == 0 || dim == 0) return AH_OK;
  AH_ARG(a && out, "ah_softmax: null operand");
  AH_ARG(lines < (int64_t(1) << 31), "ah_softmax: too many lines");
  ah::launch_kernel(k_softmax, dim3((unsigned)lines), dim3(TPB), 0, dp<const float>(a), dp<float>(out), dim, inner, log_softmax);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_softmax_bwd(ah_ptr s, ah_ptr g, ah_ptr out, int64_t rows, int64_t dim) {
  AH_REQUIRE_READY();
  if (rows == 0 || dim == 0) return AH_OK;
  AH_ARG(s && g && out, "ah_softmax_bwd: null operand");
  AH_ARG(rows < (int64_t(1) << 31), "ah_softmax_bwd: too many rows");
  ah::launch_kernel(k_softmax_bwd, dim3((unsigned)rows), dim3(TPB), 0, dp<const float>(s), dp<const float>(g), dp<float>(out), dim);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_argmax(ah_ptr a, ah_ptr out, int64_t outer, int64_t dim, int64_t inner) {
  AH_REQUIRE_READY();
  int64_t lines = outer * inner;
  if (lines == 0) return AH_OK;
  AH_ARG(a && out, "ah_argmax: null operand");
  AH_ARG(dim < (int64_t(1) << 31), "ah_argmax: axis longer than an i32 index");
  AH_ARG(lines < (int64_t(1) << 31), "ah_argmax: too many lines");
  ah::launch_kernel(k_argmax, dim3((unsigned)lines), dim3(TPB), 0, dp<const float>(a), dp<int32_t>(out), dim, inner);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

}  // extern "C"
