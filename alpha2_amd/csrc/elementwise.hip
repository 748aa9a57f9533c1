// Element-wise and data-movement kernels (HBM-bound; coalesced, float4 where alignment allows).
#include "common.h"
#include <cstring>

using namespace ah;

namespace {

constexpr int TPB = 256;

inline int grid_for(uint64_t work_items) {
  int64_t blocks = cdiv((int64_t)work_items, TPB);
#ifndef GRID_CAP_PER_CU
#define GRID_CAP_PER_CU 1024      // (measured: gelu forward / backward on 50 M elements 66 / 102 us, against 72 / 119 us with 16 blocks per CU striding over the array)
#endif
  int64_t cap = (int64_t)num_cus() * GRID_CAP_PER_CU;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

// ---- functors -----------------------------------------------------------------------------------
struct BinOp {
  int op;
  __device__ __forceinline__ float operator()(float x, float y) const {
    switch (op) { case AH_ADD: return x + y; case AH_SUB: return x - y; case AH_MUL: return x * y; default: return x / y; }
  }
};
struct UnOp {
  int op; float p0, p1;
  __device__ __forceinline__ float operator()(float x) const {
    switch (op) {
      case AH_NEG: return -x;
      case AH_EXP: return expf(x);
      case AH_LOG: return logf(x);
      case AH_SQRT: return sqrtf(x);
      case AH_POW: return powf(x, p0);
      case AH_SCALE: return x * p0;
      case AH_CLAMP: { const float m = p1 < x ? p1 : x; return p0 > m ? p0 : m; }      // max(lo, min(hi, x)) with JS's NaN: NaN stays NaN (cpu_ref.ts:358-360)
      case AH_GELU: return gelu_f(x);
      case AH_RELU: return x > 0.f ? x : 0.f;
      case AH_SILU: return x / (1.0f + expf(-x));
      default: return tanhf(x / p0) * p0;     // AH_SOFTCAP
    }
  }
};
struct UnBwd {
  int op; float p0, p1;
  __device__ __forceinline__ float operator()(float x, float g) const {
    switch (op) {
      // gelu' is 1 / 0 beyond +-40 to the last bit; evaluated there, x^3 does not overflow f32 as it would from 7e12 on (the
      // reference computes in f64, ops.ts:401-419).  NaN and the infinities go through as they are (the reference's formula
      // gives NaN for both: 0 x inf).
      case AH_GELU_BWD: { const float ax = fabsf(x); return g * gelu_grad_f(ax > 40.f && ax <= 3.402823466e38f ? copysignf(40.f, x) : x); }
      case AH_RELU_BWD: return g * (x > 0.f ? 1.f : 0.f);       // a product with the mask, as the reference forms it (ops.ts:280-290): an infinite g at x <= 0 is NaN
      case AH_SILU_BWD: { float s = 1.0f / (1.0f + expf(-x)); return g * (s * (1.0f + x * (1.0f - s))); }
      case AH_CLAMP_BWD: return (x > p0 && x < p1) ? g : 0.f;
      default: { float t = tanhf(x / p0); return g * (1.0f - t * t); }   // AH_SOFTCAP_BWD
    }
  }
};

// ---------------------------------------------------------------- per-channel mixtures of activation bases
// out[r][c] = sum over the selected bases k of coef_k[c] * basis_k(x[r][c]); bases: 0 silu, 1 relu, 2 gelu (tanh form),
// 3 identity, 4 square.  The "universal" MLP activation is bases {0, 3}, "kan_spline" all five.
struct ChannelAct {
  const float *coef[5];
  float *dcoef[5];          // backward only
  int mask;
};
// value and derivative of basis k at x (silu and gelu share nothing with the others, so each costs what it costs alone)
__device__ __forceinline__ void basis_eval(int k, float x, float &v, float &d) {
  switch (k) {
    case 0: { float s = 1.0f / (1.0f + expf(-x)); v = x * s; d = s * (1.0f + x * (1.0f - s)); break; }
    case 1: v = x > 0.f ? x : 0.f; d = x > 0.f ? 1.0f : 0.f; break;
    case 2: gelu_both_f(x, v, d); break;
    case 3: v = x; d = 1.0f; break;
    default: v = x * x; d = 2.0f * x; break;
  }
}
// four consecutive elements of an f32 or bf16 row (i counts quads)
template <class T> __device__ __forceinline__ void ld4(const T *p, int64_t i, float v[4]);
template <> __device__ __forceinline__ void ld4<float>(const float *p, int64_t i, float v[4]) {
  float4 u = reinterpret_cast<const float4 *>(p)[i];
  v[0] = u.x; v[1] = u.y; v[2] = u.z; v[3] = u.w;
}
template <> __device__ __forceinline__ void ld4<uint16_t>(const uint16_t *p, int64_t i, float v[4]) {
  uint2 u = reinterpret_cast<const uint2 *>(p)[i];
  v[0] = bf16_bits_to_f32(u.x & 0xffffu); v[1] = bf16_bits_to_f32(u.x >> 16);
  v[2] = bf16_bits_to_f32(u.y & 0xffffu); v[3] = bf16_bits_to_f32(u.y >> 16);
}
template <class T> __device__ __forceinline__ void st4(T *p, int64_t i, const float v[4]);
template <> __device__ __forceinline__ void st4<float>(float *p, int64_t i, const float v[4]) {
  reinterpret_cast<float4 *>(p)[i] = make_float4(v[0], v[1], v[2], v[3]);
}
template <> __device__ __forceinline__ void st4<uint16_t>(uint16_t *p, int64_t i, const float v[4]) {
  reinterpret_cast<uint2 *>(p)[i] = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
}
// coefficient quad of basis k at column quad c4; a null vector is the constant 1 (a plain activation)
__device__ __forceinline__ void coef4(const ChannelAct &p, int k, int c4, float cs[4]) {
  if (p.coef[k]) ld4<float>(p.coef[k], c4, cs);
  else cs[0] = cs[1] = cs[2] = cs[3] = 1.0f;
}
template <class T>
__global__ void k_channel_act(const T *__restrict__ x, ChannelAct p, T *__restrict__ out, int64_t rows, int cols4) {
  int64_t n4 = rows * (int64_t)cols4;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
    int c4 = (int)(i % cols4);
    float xs[4], acc[4] = {0.f, 0.f, 0.f, 0.f};
    ld4<T>(x, i, xs);
#pragma unroll
    for (int k = 0; k < 5; k++)
      if (p.mask >> k & 1) {
        float cs[4];
        coef4(p, k, c4, cs);
#pragma unroll
        for (int e = 0; e < 4; e++) { float v, d; basis_eval(k, xs[e], v, d); acc[e] += cs[e] * v; }
      }
    st4<T>(out, i, acc);
  }
}
// Backward: dx = g * sum_k coef_k basis_k'(x); partial[rb][k][c] = sum over the rows of row block rb of g * basis_k(x).
// A block is 64 column quads x 4 row lanes; a wave reads 1 KB (f32) of one row.
constexpr int CA_ROWLANES = 4;
template <class T>
__global__ __launch_bounds__(256) void k_channel_act_bwd(const T *__restrict__ x, const T *__restrict__ g, ChannelAct p, T *__restrict__ dx,
                                                         float *__restrict__ partial, int64_t rows, int cols4, int rows_per_block) {
  __shared__ float4 red[5][CA_ROWLANES][64];
  const int cq = threadIdx.x & 63, rl = threadIdx.x >> 6, c4 = blockIdx.x * 64 + cq;
  const int64_t r0 = blockIdx.y * (int64_t)rows_per_block, r1 = min(rows, r0 + rows_per_block);
  float sums[5][4] = {};
  if (c4 < cols4) {
    float cs[5][4] = {};
#pragma unroll
    for (int k = 0; k < 5; k++)
      if (p.mask >> k & 1) coef4(p, k, c4, cs[k]);
    for (int64_t r = r0 + rl; r < r1; r += CA_ROWLANES) {
      int64_t i = r * cols4 + c4;
      float xs[4], gs[4], acc[4] = {0.f, 0.f, 0.f, 0.f};
      ld4<T>(x, i, xs);
      ld4<T>(g, i, gs);
#pragma unroll
      for (int k = 0; k < 5; k++)
        if (p.mask >> k & 1) {
#pragma unroll
          for (int e = 0; e < 4; e++) { float v, d; basis_eval(k, xs[e], v, d); acc[e] += cs[k][e] * d; sums[k][e] += gs[e] * v; }
        }
      const float o[4] = {gs[0] * acc[0], gs[1] * acc[1], gs[2] * acc[2], gs[3] * acc[3]};
      st4<T>(dx, i, o);
    }
  }
  if (!partial) return;                               // no coefficient has a gradient (block-uniform)
#pragma unroll
  for (int k = 0; k < 5; k++) red[k][rl][cq] = make_float4(sums[k][0], sums[k][1], sums[k][2], sums[k][3]);
  __syncthreads();
  if (rl == 0 && c4 < cols4) {
#pragma unroll
    for (int k = 0; k < 5; k++)
      if (p.dcoef[k]) {
        float4 a = red[k][0][cq];
        for (int j = 1; j < CA_ROWLANES; j++) { float4 b = red[k][j][cq]; a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w; }
        reinterpret_cast<float4 *>(partial + ((int64_t)blockIdx.y * 5 + k) * cols4 * 4)[c4] = a;
      }
  }
}
// dcoef_k[c] = (accumulate ? dcoef_k[c] : 0) + sum over row blocks of partial[rb][k][c], in double, fixed order
__global__ void k_channel_act_colsum(const float *__restrict__ partial, ChannelAct p, int nrb, int cols, int accumulate) {
  int c = blockIdx.x * blockDim.x + threadIdx.x, k = blockIdx.y;
  if (c >= cols || !p.dcoef[k]) return;
  double s = 0;
  for (int rb = 0; rb < nrb; rb++) s += (double)partial[((int64_t)rb * 5 + k) * cols + c];
  p.dcoef[k][c] = accumulate ? (float)((double)p.dcoef[k][c] + s) : (float)s;
}

// SwiGLU on the packed pre-activation gu = [gate | up], rows of 2 * cols (packages/model/src/gpt.ts:295-299; the element
// arithmetic of Backend.siluMul / siluMulBackward, ops.ts:284-417):  out = silu(gate) * up;
// dgate = g * up * s (1 + gate (1 - s)),  dup = g * gate * s,  s = sigmoid(gate).
template <class T>
__global__ void k_swiglu(const T *__restrict__ gu, T *__restrict__ out, int64_t rows, int cols4) {
  int64_t n4 = rows * (int64_t)cols4;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
    int64_t r = i / cols4, c4 = i - r * cols4;
    float a[4], b[4], o[4];
    ld4<T>(gu, r * 2 * cols4 + c4, a);
    ld4<T>(gu, r * 2 * cols4 + cols4 + c4, b);
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = a[e] / (1.0f + expf(-a[e])) * b[e];
    st4<T>(out, i, o);
  }
}
template <class T>
__global__ void k_swiglu_bwd(const T *__restrict__ gu, const T *__restrict__ g, T *__restrict__ dgu, int64_t rows, int cols4) {
  int64_t n4 = rows * (int64_t)cols4;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
    int64_t r = i / cols4, c4 = i - r * cols4;
    float a[4], b[4], gs[4], da[4], db[4];
    ld4<T>(gu, r * 2 * cols4 + c4, a);
    ld4<T>(gu, r * 2 * cols4 + cols4 + c4, b);
    ld4<T>(g, i, gs);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      float s = 1.0f / (1.0f + expf(-a[e]));
      da[e] = gs[e] * b[e] * s * (1.0f + a[e] * (1.0f - s));
      db[e] = gs[e] * a[e] * s;
    }
    st4<T>(dgu, r * 2 * cols4 + c4, da);
    st4<T>(dgu, r * 2 * cols4 + cols4 + c4, db);
  }
}

template <class F>
__global__ void k_unary(const float *__restrict__ x, float *__restrict__ out, uint64_t n, F f, int vec) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  if (vec) {
    uint64_t n4 = n >> 2;
    for (uint64_t i = tid; i < n4; i += stride) {
      float4 v = reinterpret_cast<const float4 *>(x)[i];
      v.x = f(v.x); v.y = f(v.y); v.z = f(v.z); v.w = f(v.w);
      reinterpret_cast<float4 *>(out)[i] = v;
    }
    for (uint64_t i = (n4 << 2) + tid; i < n; i += stride) out[i] = f(x[i]);
  } else {
    for (uint64_t i = tid; i < n; i += stride) out[i] = f(x[i]);
  }
}
template <class F>
__global__ void k_binary(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ out,
                         uint64_t n, F f, int vec) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  if (vec) {
    uint64_t n4 = n >> 2;
    for (uint64_t i = tid; i < n4; i += stride) {
      float4 u = reinterpret_cast<const float4 *>(a)[i], v = reinterpret_cast<const float4 *>(b)[i], r;
      r.x = f(u.x, v.x); r.y = f(u.y, v.y); r.z = f(u.z, v.z); r.w = f(u.w, v.w);
      reinterpret_cast<float4 *>(out)[i] = r;
    }
    for (uint64_t i = (n4 << 2) + tid; i < n; i += stride) out[i] = f(a[i], b[i]);
  } else {
    for (uint64_t i = tid; i < n; i += stride) out[i] = f(a[i], b[i]);
  }
}

struct Dims6 { int64_t shape[6]; int64_t sa[6]; int64_t sb[6]; int nd; };

__global__ void k_binary_bcast(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ out,
                               uint64_t n, Dims6 d, BinOp f) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = tid; i < n; i += stride) {
    uint64_t rem = i; int64_t ia = 0, ib = 0;
    for (int k = d.nd - 1; k >= 0; k--) {
      uint64_t c = rem % (uint64_t)d.shape[k]; rem /= (uint64_t)d.shape[k];
      ia += (int64_t)c * d.sa[k]; ib += (int64_t)c * d.sb[k];
    }
    out[i] = f(a[ia], b[ib]);
  }
}

// generic strided gather: out[i] = src[offset + sum(coord_k * stride_k)] over `shape`; strided scatter: dst[that] = src[i].
// W is the unit moved (one 4-byte word, or four when the innermost dimension is contiguous on both sides and everything is a
// multiple of four words: shape, strides and offset are then in units of W), I the integer type of the index arithmetic (32-bit
// whenever every index fits: a 64-bit division is the most expensive thing in these kernels).
struct Gather6 { int64_t shape[6]; int64_t stride[6]; int64_t offset; int nd; };
template <class W, class I, bool SCATTER>
__global__ void k_move(const W *__restrict__ src, W *__restrict__ dst, uint64_t n, Gather6 d) {
  const I total = (I)n, step = (I)((uint64_t)gridDim.x * blockDim.x);
  I shp[6], str[6];
#pragma unroll
  for (int k = 0; k < 6; k++) { shp[k] = (I)d.shape[k]; str[k] = (I)d.stride[k]; }
  for (I i = (I)(blockIdx.x * (uint64_t)blockDim.x + threadIdx.x); i < total; i += step) {
    I rem = i, s = (I)d.offset;
#pragma unroll
    for (int k = 5; k >= 0; k--)
      if (k < d.nd) {
        const I q = rem / shp[k], c = rem - q * shp[k];
        rem = q;
        s += c * str[k];
      }
    if (SCATTER) dst[s] = src[i]; else dst[i] = src[s];
    if (i + step < i) break;                                       // (the index type wrapped: i was the last one)
  }
}
// `g` describes the strided side; the other side is contiguous over g.shape.
template <bool SCATTER>
static void launch_move(const void *src, void *dst, uint64_t n, Gather6 g) {
  const int nd = g.nd;
  const uintptr_t both = (uintptr_t)src | (uintptr_t)dst;
  bool vec = nd >= 1 && g.stride[nd - 1] == 1 && g.shape[nd - 1] % 4 == 0 && g.offset % 4 == 0 && (both & 15u) == 0;
  for (int k = 0; vec && k < nd - 1; k++) vec = g.stride[k] % 4 == 0;
  if (vec) {
    g.shape[nd - 1] /= 4; g.offset /= 4; n /= 4;
    for (int k = 0; k < nd - 1; k++) g.stride[k] /= 4;
  }
  uint64_t reach = (uint64_t)g.offset;                             // largest index on the strided side
  bool nonneg = g.offset >= 0;
  for (int k = 0; k < nd; k++) { nonneg = nonneg && g.stride[k] >= 0; if (g.shape[k] > 0 && g.stride[k] > 0) reach += (uint64_t)(g.shape[k] - 1) * (uint64_t)g.stride[k]; }
  const bool small = nonneg && n < (uint64_t(1) << 31) && reach < (uint64_t(1) << 31);
  const dim3 grid(grid_for(n)), blk(TPB);
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  if (vec && small) ah::launch_kernel((k_move<u32x4, uint32_t, SCATTER>), grid, blk, 0, (const u32x4 *)src, (u32x4 *)dst, n, g);
  else if (vec) ah::launch_kernel((k_move<u32x4, uint64_t, SCATTER>), grid, blk, 0, (const u32x4 *)src, (u32x4 *)dst, n, g);
  else if (small) ah::launch_kernel((k_move<uint32_t, uint32_t, SCATTER>), grid, blk, 0, (const uint32_t *)src, (uint32_t *)dst, n, g);
  else ah::launch_kernel((k_move<uint32_t, uint64_t, SCATTER>), grid, blk, 0, (const uint32_t *)src, (uint32_t *)dst, n, g);
}

// 32x32 LDS-tiled transpose of the last two dims of [batch, R, C] (coalesced both ways)
__global__ void k_transpose_last2(const uint32_t *__restrict__ in, uint32_t *__restrict__ out, int64_t R, int64_t C) {
  __shared__ uint32_t tile[32][33];
  int64_t b = blockIdx.z;
  const uint32_t *src = in + b * R * C;
  uint32_t *dst = out + b * R * C;
  int64_t c0 = (int64_t)blockIdx.x * 32, r0 = (int64_t)blockIdx.y * 32;
  for (int j = threadIdx.y; j < 32; j += blockDim.y) {
    int64_t r = r0 + j, c = c0 + threadIdx.x;
    if (r < R && c < C) tile[j][threadIdx.x] = src[r * C + c];
  }
  __syncthreads();
  for (int j = threadIdx.y; j < 32; j += blockDim.y) {
    int64_t c = c0 + j, r = r0 + threadIdx.x;
    if (r < R && c < C) dst[c * R + r] = tile[threadIdx.x][j];
  }
}

// 4-byte elements; 16-byte stores over the aligned middle of the range, single elements at its ragged ends
template <class T>
__global__ void k_fill(T *__restrict__ p, T v, uint64_t n) {
  static_assert(sizeof(T) == 4, "k_fill writes 4-byte elements");
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  uint64_t head = (4 - (((uintptr_t)p >> 2) & 3)) & 3;            // elements before the first 16-byte boundary
  if (head > n) head = n;
  uint64_t n4 = (n - head) >> 2;
  uint32_t bits = __builtin_bit_cast(uint32_t, v);
  uint4 *q = reinterpret_cast<uint4 *>(p + head);
  for (uint64_t i = tid; i < n4; i += stride) q[i] = make_uint4(bits, bits, bits, bits);
  for (uint64_t i = tid; i < head; i += stride) p[i] = v;
  for (uint64_t i = head + (n4 << 2) + tid; i < n; i += stride) p[i] = v;
}

__global__ void k_axpy(float *__restrict__ a, const float *__restrict__ b, float s, uint64_t n) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = tid; i < n; i += stride) a[i] += b[i] * s;
}

// out = a + b on bf16 storage, 8 elements per thread (out may be a or b)
__global__ void k_add_bf16(const uint16_t *a, const uint16_t *b, uint16_t *out, uint64_t n) {
  const uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x, n8 = n >> 3;
  for (uint64_t i = tid; i < n8; i += stride) {
    const uint4 x = reinterpret_cast<const uint4 *>(a)[i], y = reinterpret_cast<const uint4 *>(b)[i];
    const uint32_t xs[4] = {x.x, x.y, x.z, x.w}, ys[4] = {y.x, y.y, y.z, y.w};
    uint32_t o[4];
#pragma unroll
    for (int q = 0; q < 4; q++)
      o[q] = pack_bf16x2(bf16_bits_to_f32(xs[q] & 0xffffu) + bf16_bits_to_f32(ys[q] & 0xffffu), bf16_bits_to_f32(xs[q] >> 16) + bf16_bits_to_f32(ys[q] >> 16));
    reinterpret_cast<uint4 *>(out)[i] = make_uint4(o[0], o[1], o[2], o[3]);
  }
  for (uint64_t i = (n8 << 3) + tid; i < n; i += stride) out[i] = f32_to_bf16_bits(bf16_bits_to_f32(a[i]) + bf16_bits_to_f32(b[i]));
}

__global__ void k_silu_mul(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ out, uint64_t n) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = tid; i < n; i += stride) { float x = a[i]; out[i] = x / (1.0f + expf(-x)) * b[i]; }
}
__global__ void k_silu_mul_bwd(const float *__restrict__ a, const float *__restrict__ b, const float *__restrict__ g,
                               float *__restrict__ da, float *__restrict__ db, uint64_t n) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = tid; i < n; i += stride) {
    float x = a[i], s = 1.0f / (1.0f + expf(-x)), gi = g[i];
    da[i] = gi * b[i] * (s * (1.0f + x * (1.0f - s)));
    db[i] = gi * (x * s);
  }
}
__global__ void k_residual_dropout_add(const float *__restrict__ r, const float *__restrict__ p, const float *__restrict__ m,
                                       float *__restrict__ out, uint64_t n) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = tid; i < n; i += stride) out[i] = r[i] + (m ? p[i] * m[i] : p[i]);
}
// DropoutRng.hash of the reference's CPU path (packages/autograd/src/ops.ts:74-81), bit for bit: the first line is evaluated in
// doubles, one rounding per operation (no fused multiply-add), and only then cut to 32 bits, so products past 2^53 have already
// lost low bits exactly as a JS number does.  (The reference's own GPU kernel wraps in u32 instead,
// packages/helios/src/kernels/nn.ts:5600-5748, and so differs from its CPU path for element indices above ~4.0 M.)
// The sum is an integer-valued double below 2^63: the int64 conversion is exact and its low 32 bits are ToInt32.
__global__ void k_dropout_mask(float *__restrict__ out, uint64_t n, int32_t seed, int32_t counter, double p, float keep) {
#pragma clang fp contract(off)
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  const double base = (double)seed + (double)counter * 2654435761.0;
  for (uint64_t i = tid; i < n; i += stride) {
    double sum = base + (double)i * 2246822519.0;
    uint32_t h = (uint32_t)(int64_t)sum;
    h = (h ^ (h >> 16)) * 0x85ebca6bu;
    h = (h ^ (h >> 13)) * 0xc2b2ae35u;
    h = h ^ (h >> 16);
    out[i] = ((double)h * (1.0 / 4294967296.0) > p) ? keep : 0.f;
  }
}
// out = (residual or 0) + x * mask, the mask of k_dropout_mask made on the fly from a seed that lives in device memory: four
// consecutive elements per thread (8- or 16-byte accesses), the tail one at a time.
__device__ __forceinline__ float drop_keep(double base, uint64_t i, double p, float keep) {
#pragma clang fp contract(off)
  double sum = base + (double)i * 2246822519.0;
  uint32_t h = (uint32_t)(int64_t)sum;
  h = (h ^ (h >> 16)) * 0x85ebca6bu;
  h = (h ^ (h >> 13)) * 0xc2b2ae35u;
  h = h ^ (h >> 16);
  return ((double)h * (1.0 / 4294967296.0) > p) ? keep : 0.f;
}
__device__ __forceinline__ void ld4(const float *p, uint64_t i, float (&v)[4]) { float4 t = *reinterpret_cast<const float4 *>(p + i); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
__device__ __forceinline__ void ld4(const uint16_t *p, uint64_t i, float (&v)[4]) {
  uint2 t = *reinterpret_cast<const uint2 *>(p + i);
  v[0] = bf16_bits_to_f32(t.x & 0xffffu); v[1] = bf16_bits_to_f32(t.x >> 16); v[2] = bf16_bits_to_f32(t.y & 0xffffu); v[3] = bf16_bits_to_f32(t.y >> 16);
}
__device__ __forceinline__ void st4(float *p, uint64_t i, const float (&v)[4]) { *reinterpret_cast<float4 *>(p + i) = make_float4(v[0], v[1], v[2], v[3]); }
__device__ __forceinline__ void st4(uint16_t *p, uint64_t i, const float (&v)[4]) { *reinterpret_cast<uint2 *>(p + i) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])); }
__device__ __forceinline__ float ld1(const float *p, uint64_t i) { return p[i]; }
__device__ __forceinline__ float ld1(const uint16_t *p, uint64_t i) { return bf16_bits_to_f32(p[i]); }
__device__ __forceinline__ void st1(float *p, uint64_t i, float v) { p[i] = v; }
__device__ __forceinline__ void st1(uint16_t *p, uint64_t i, float v) { p[i] = f32_to_bf16_bits(v); }
template <class X, class O>
__global__ void k_dropout_apply(const X *__restrict__ x, const O *__restrict__ residual, O *__restrict__ out, uint64_t n, const int32_t *__restrict__ seed,
                                int32_t counter, double p, float keep, int vec) {
#pragma clang fp contract(off)
  const uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  const double base = (double)seed[0] + (double)counter * 2654435761.0;
  const uint64_t n4 = vec ? n >> 2 : 0;
  for (uint64_t q = tid; q < n4; q += stride) {
    const uint64_t i = q << 2;
    float v[4], r[4] = {0.f, 0.f, 0.f, 0.f};
    ld4(x, i, v);
    if (residual) ld4(residual, i, r);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float m = v[e] * drop_keep(base, i + e, p, keep);
      r[e] = residual ? r[e] + m : m;               // (no residual: the product itself, the sign of a zero included)
    }
    st4(out, i, r);
  }
  for (uint64_t i = (n4 << 2) + tid; i < n; i += stride) {
    const float m = ld1(x, i) * drop_keep(base, i, p, keep);
    st1(out, i, residual ? ld1(residual, i) + m : m);
  }
}
__global__ void k_masked_fill(const float *__restrict__ a, const float *__restrict__ mask, float *__restrict__ out,
                              uint64_t n, uint64_t mask_n, float value) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = tid; i < n; i += stride) out[i] = (mask[i % mask_n] != 0.f) ? value : a[i];
}
__global__ void k_causal_mask(float *__restrict__ out, int64_t size) {
  uint64_t n = (uint64_t)size * size;
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = tid; i < n; i += stride) out[i] = ((int64_t)(i % size) > (int64_t)(i / size)) ? -INFINITY : 0.f;
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { _Float16 h = (_Float16)f; uint16_t u; __builtin_memcpy(&u, &h, 2); return u; }
__device__ __forceinline__ float f16_bits_to_f32(uint16_t u) { _Float16 h; __builtin_memcpy(&h, &u, 2); return (float)h; }

__global__ void k_cast(const void *__restrict__ src, int sd, void *__restrict__ dst, int dd, uint64_t n) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = tid; i < n; i += stride) {
    float v;
    if (sd == AH_F32) v = ((const float *)src)[i];
    else if (sd == AH_BF16) v = bf16_bits_to_f32(((const uint16_t *)src)[i]);
    else if (sd == AH_F16) v = f16_bits_to_f32(((const uint16_t *)src)[i]);
    else v = (float)((const int32_t *)src)[i];
    if (dd == AH_F32) ((float *)dst)[i] = v;
    else if (dd == AH_BF16) ((uint16_t *)dst)[i] = f32_to_bf16_bits(v);
    else if (dd == AH_F16) ((uint16_t *)dst)[i] = f32_to_f16_bits(v);
    else ((int32_t *)dst)[i] = (int32_t)v;
  }
}

__global__ void k_check_finite(const float *__restrict__ x, uint64_t n, float *__restrict__ flag) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  bool bad = false;
  for (uint64_t i = tid; i < n; i += stride) {
    uint32_t u = __float_as_uint(x[i]);
    bad |= ((u & 0x7f800000u) == 0x7f800000u);
  }
  if (__any(bad) && (threadIdx.x & 63) == 0) *flag = 1.0f;   // every writer stores the same value
}

inline bool vec_ok(uint64_t n, ah_ptr a, ah_ptr b, ah_ptr c) {
  (void)n;
  return aligned16(a) && aligned16(b) && aligned16(c);
}

void row_major_strides(int nd, const int64_t *shape, int64_t *st) {
  int64_t s = 1;
  for (int i = nd - 1; i >= 0; i--) { st[i] = s; s *= shape[i]; }
}
int64_t prod(int nd, const int64_t *shape) { int64_t s = 1; for (int i = 0; i < nd; i++) s *= shape[i]; return s; }

}  // namespace

extern "C" {

int32_t ah_fill_f32(ah_ptr dst, float value, uint64_t n) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(dst != 0, "ah_fill_f32: null dst");
  ah::launch_kernel(k_fill<float>, dim3(grid_for(n / 4 + 1)), dim3(TPB), 0, dp<float>(dst), value, n);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_fill_i32(ah_ptr dst, int32_t value, uint64_t n) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(dst != 0, "ah_fill_i32: null dst");
  ah::launch_kernel(k_fill<int32_t>, dim3(grid_for(n / 4 + 1)), dim3(TPB), 0, dp<int32_t>(dst), value, n);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_binary(int32_t op, ah_ptr a, ah_ptr b, ah_ptr out, uint64_t n) {
  AH_REQUIRE_READY();
  AH_ARG(op >= AH_ADD && op <= AH_DIV, "ah_binary: bad op %d", op);
  if (n == 0) return AH_OK;
  AH_ARG(a && b && out, "ah_binary: null operand");
  int vec = vec_ok(n, a, b, out);
  ah::launch_kernel(k_binary<BinOp>, dim3(grid_for(vec ? n / 4 + 1 : n)), dim3(TPB), 0, 
                     dp<const float>(a), dp<const float>(b), dp<float>(out), n, BinOp{op}, vec);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_binary_broadcast(int32_t op, ah_ptr a, ah_ptr b, ah_ptr out, int32_t nd, const int64_t *shape,
                            const int64_t *stride_a, const int64_t *stride_b) {
  AH_REQUIRE_READY();
  AH_ARG(op >= AH_ADD && op <= AH_DIV, "ah_binary_broadcast: bad op %d", op);
  AH_ARG(nd >= 0 && nd <= 6, "ah_binary_broadcast: nd %d > 6", nd);
  Dims6 d; memset(&d, 0, sizeof d); d.nd = nd;      // (zeroed: see the Gather6 arguments below)
  for (int i = 0; i < nd; i++) { d.shape[i] = shape[i]; d.sa[i] = stride_a[i]; d.sb[i] = stride_b[i]; }
  uint64_t n = (uint64_t)prod(nd, shape);
  if (n == 0) return AH_OK;
  AH_ARG(a && b && out, "ah_binary_broadcast: null operand");
  ah::launch_kernel(k_binary_bcast, dim3(grid_for(n)), dim3(TPB), 0, dp<const float>(a), dp<const float>(b),
                     dp<float>(out), n, d, BinOp{op});
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_unary(int32_t op, ah_ptr x, ah_ptr out, uint64_t n, float p0, float p1) {
  AH_REQUIRE_READY();
  AH_ARG(op >= AH_NEG && op <= AH_SOFTCAP, "ah_unary: bad op %d", op);
  if (n == 0) return AH_OK;
  AH_ARG(x && out, "ah_unary: null operand");
  int vec = vec_ok(n, x, x, out);
  ah::launch_kernel(k_unary<UnOp>, dim3(grid_for(vec ? n / 4 + 1 : n)), dim3(TPB), 0, dp<const float>(x),
                     dp<float>(out), n, UnOp{op, p0, p1}, vec);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_add_inplace(ah_ptr a, ah_ptr b, uint64_t n) { return ah_binary(AH_ADD, a, b, a, n); }
int32_t ah_scale_inplace(ah_ptr a, float s, uint64_t n) { return ah_unary(AH_SCALE, a, a, n, s, 0.f); }
int32_t ah_axpy_inplace(ah_ptr a, ah_ptr b, float s, uint64_t n) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(a && b, "ah_axpy_inplace: null operand");
  ah::launch_kernel(k_axpy, dim3(grid_for(n)), dim3(TPB), 0, dp<float>(a), dp<const float>(b), s, n);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_add_bf16(ah_ptr a, ah_ptr b, ah_ptr out, uint64_t n) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(a && b && out, "ah_add_bf16: null operand");
  AH_ARG(aligned16(a) && aligned16(b) && aligned16(out), "ah_add_bf16: operands must be 16-byte aligned");
  ah::launch_kernel(k_add_bf16, dim3(grid_for(n / 8 + 1)), dim3(TPB), 0, dp<const uint16_t>(a), dp<const uint16_t>(b), dp<uint16_t>(out), n);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_unary_bwd(int32_t op, ah_ptr x, ah_ptr grad_out, ah_ptr out, uint64_t n, float p0, float p1) {
  AH_REQUIRE_READY();
  AH_ARG(op >= AH_GELU_BWD && op <= AH_SOFTCAP_BWD, "ah_unary_bwd: bad op %d", op);
  if (n == 0) return AH_OK;
  AH_ARG(x && grad_out && out, "ah_unary_bwd: null operand");
  int vec = vec_ok(n, x, grad_out, out);
  ah::launch_kernel(k_binary<UnBwd>, dim3(grid_for(vec ? n / 4 + 1 : n)), dim3(TPB), 0, dp<const float>(x),
                     dp<const float>(grad_out), dp<float>(out), n, UnBwd{op, p0, p1}, vec);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_silu_mul(ah_ptr a, ah_ptr b, ah_ptr out, uint64_t n) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(a && b && out, "ah_silu_mul: null operand");
  ah::launch_kernel(k_silu_mul, dim3(grid_for(n)), dim3(TPB), 0, dp<const float>(a), dp<const float>(b), dp<float>(out), n);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_silu_mul_bwd(ah_ptr a, ah_ptr b, ah_ptr g, ah_ptr da, ah_ptr db, uint64_t n) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(a && b && g && da && db, "ah_silu_mul_bwd: null operand");
  ah::launch_kernel(k_silu_mul_bwd, dim3(grid_for(n)), dim3(TPB), 0, dp<const float>(a), dp<const float>(b),
                     dp<const float>(g), dp<float>(da), dp<float>(db), n);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
// mask: bit k selects basis k (0 silu, 1 relu, 2 gelu, 3 identity, 4 square); coefs[k] = f32[cols] for the selected ones,
// 0 for the constant 1 (then no gradient is produced for it)
static int32_t channel_act_args(const char *who, int32_t dtype, const ah_ptr *coefs, int32_t mask, int64_t rows, int64_t cols, ChannelAct &p, const ah_ptr *dcoefs) {
  AH_ARG(dtype == AH_F32 || dtype == AH_BF16, "%s: dtype must be AH_F32 or AH_BF16", who);
  AH_ARG(mask > 0 && mask < 32, "%s: basis mask %d selects nothing or an unknown basis", who, mask);
  AH_ARG(rows >= 0 && cols > 0 && cols % 4 == 0 && cols < (1ll << 31), "%s: cols %lld must be a positive multiple of 4", who, (long long)cols);
  p.mask = mask;
  for (int k = 0; k < 5; k++) {
    bool on = (mask >> k & 1) && coefs && coefs[k] != 0;
    AH_ARG(!on || coefs[k] % 16 == 0, "%s: coefficient vector %d is not 16-byte aligned", who, k);
    AH_ARG(!on || !dcoefs || dcoefs[k] != 0, "%s: gradient vector %d missing", who, k);
    p.coef[k] = on ? dp<const float>(coefs[k]) : nullptr;
    p.dcoef[k] = on && dcoefs ? dp<float>(dcoefs[k]) : nullptr;
  }
  return AH_OK;
}
int32_t ah_channel_act(int32_t dtype, ah_ptr x, const ah_ptr *coefs, int32_t mask, ah_ptr out, int64_t rows, int64_t cols) {
  AH_REQUIRE_READY();
  ChannelAct p;
  int32_t rc = channel_act_args("ah_channel_act", dtype, coefs, mask, rows, cols, p, nullptr);
  if (rc) return rc;
  if (rows == 0) return AH_OK;
  AH_ARG(x && out && aligned16(x) && aligned16(out), "ah_channel_act: operands must be non-null and 16-byte aligned");
  const dim3 grid(grid_for((uint64_t)(rows * cols / 4)));
  if (dtype == AH_F32) ah::launch_kernel(k_channel_act<float>, grid, dim3(TPB), 0, dp<const float>(x), p, dp<float>(out), rows, (int)(cols / 4));
  else ah::launch_kernel(k_channel_act<uint16_t>, grid, dim3(TPB), 0, dp<const uint16_t>(x), p, dp<uint16_t>(out), rows, (int)(cols / 4));
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_channel_act_bwd(int32_t dtype, ah_ptr x, const ah_ptr *coefs, int32_t mask, ah_ptr grad_out, ah_ptr dx, const ah_ptr *dcoefs,
                           int32_t accumulate, int64_t rows, int64_t cols) {
  AH_REQUIRE_READY();
  ChannelAct p;
  int32_t rc = channel_act_args("ah_channel_act_bwd", dtype, coefs, mask, rows, cols, p, dcoefs);
  if (rc) return rc;
  bool any = false;
  for (int k = 0; k < 5; k++) any = any || p.dcoef[k];
  if (rows == 0) {
    for (int k = 0; k < 5; k++)
      if (p.dcoef[k] && !accumulate) { rc = ah_fill_f32(dcoefs[k], 0.f, (uint64_t)cols); if (rc) return rc; }
    return AH_OK;
  }
  AH_ARG(x && grad_out && dx && aligned16(x) && aligned16(grad_out) && aligned16(dx), "ah_channel_act_bwd: operands must be non-null and 16-byte aligned");
  const int cols4 = (int)(cols / 4), gx = (int)cdiv(cols4, 64);
  int nrb = (int)cdiv(rows, 64);                                  // >= 64 rows per block amortise the partial write
  int cap = (4 * num_cus() + gx - 1) / gx;
  if (nrb > cap) nrb = cap;
  const int rpb = (int)cdiv(rows, nrb);
  nrb = (int)cdiv(rows, rpb);
  float *partial = nullptr;
  if (any) {
    partial = (float *)scratch(sizeof(float) * 5 * (size_t)nrb * (size_t)cols);
    if (!partial) return fail(AH_ERR_OOM, "ah_channel_act_bwd: no scratch");
  }
  if (dtype == AH_F32)
    ah::launch_kernel(k_channel_act_bwd<float>, dim3(gx, nrb), dim3(256), 0, dp<const float>(x), dp<const float>(grad_out), p, dp<float>(dx), partial,
                       rows, cols4, rpb);
  else
    ah::launch_kernel(k_channel_act_bwd<uint16_t>, dim3(gx, nrb), dim3(256), 0, dp<const uint16_t>(x), dp<const uint16_t>(grad_out), p, dp<uint16_t>(dx),
                       partial, rows, cols4, rpb);
  AH_LAUNCH_CHECK();
  if (any) {
    ah::launch_kernel(k_channel_act_colsum, dim3((unsigned)cdiv(cols, 256), 5), dim3(256), 0, partial, p, nrb, (int)cols, accumulate);
    AH_LAUNCH_CHECK();
  }
  return AH_OK;
}
static int32_t swiglu_args(const char *who, int32_t dtype, int64_t rows, int64_t cols) {
  AH_ARG(dtype == AH_F32 || dtype == AH_BF16, "%s: dtype must be AH_F32 or AH_BF16", who);
  AH_ARG(rows >= 0 && cols > 0 && cols % 4 == 0 && cols < (1ll << 30), "%s: cols %lld must be a positive multiple of 4", who, (long long)cols);
  return AH_OK;
}
int32_t ah_swiglu(int32_t dtype, ah_ptr gate_up, ah_ptr out, int64_t rows, int64_t cols) {
  AH_REQUIRE_READY();
  int32_t rc = swiglu_args("ah_swiglu", dtype, rows, cols);
  if (rc) return rc;
  if (rows == 0) return AH_OK;
  AH_ARG(gate_up && out && aligned16(gate_up) && aligned16(out), "ah_swiglu: operands must be non-null and 16-byte aligned");
  const dim3 grid(grid_for((uint64_t)(rows * cols / 4)));
  if (dtype == AH_F32) ah::launch_kernel(k_swiglu<float>, grid, dim3(TPB), 0, dp<const float>(gate_up), dp<float>(out), rows, (int)(cols / 4));
  else ah::launch_kernel(k_swiglu<uint16_t>, grid, dim3(TPB), 0, dp<const uint16_t>(gate_up), dp<uint16_t>(out), rows, (int)(cols / 4));
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_swiglu_bwd(int32_t dtype, ah_ptr gate_up, ah_ptr grad_out, ah_ptr d_gate_up, int64_t rows, int64_t cols) {
  AH_REQUIRE_READY();
  int32_t rc = swiglu_args("ah_swiglu_bwd", dtype, rows, cols);
  if (rc) return rc;
  if (rows == 0) return AH_OK;
  AH_ARG(gate_up && grad_out && d_gate_up && aligned16(gate_up) && aligned16(grad_out) && aligned16(d_gate_up),
         "ah_swiglu_bwd: operands must be non-null and 16-byte aligned");
  const dim3 grid(grid_for((uint64_t)(rows * cols / 4)));
  if (dtype == AH_F32)
    ah::launch_kernel(k_swiglu_bwd<float>, grid, dim3(TPB), 0, dp<const float>(gate_up), dp<const float>(grad_out), dp<float>(d_gate_up), rows, (int)(cols / 4));
  else
    ah::launch_kernel(k_swiglu_bwd<uint16_t>, grid, dim3(TPB), 0, dp<const uint16_t>(gate_up), dp<const uint16_t>(grad_out), dp<uint16_t>(d_gate_up), rows,
                       (int)(cols / 4));
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_residual_dropout_add(ah_ptr residual, ah_ptr projected, ah_ptr mask, ah_ptr out, uint64_t n) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(residual && projected && out, "ah_residual_dropout_add: null operand");
  ah::launch_kernel(k_residual_dropout_add, dim3(grid_for(n)), dim3(TPB), 0, dp<const float>(residual),
                     dp<const float>(projected), dp<const float>(mask), dp<float>(out), n);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_dropout_mask(ah_ptr out, uint64_t n, int32_t seed, int32_t counter, double p) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(out != 0, "ah_dropout_mask: null out");
  AH_ARG(p >= 0.0 && p < 1.0, "ah_dropout_mask: p must be in [0,1)");
  AH_ARG(n <= (1ull << 32), "ah_dropout_mask: at most 2^32 elements (the hash sum must stay below 2^63)");
  ah::launch_kernel(k_dropout_mask, dim3(grid_for(n)), dim3(TPB), 0, dp<float>(out), n, seed, counter, p,
                     (float)(1.0 / (1.0 - p)));
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_dropout_apply(ah_ptr x, int32_t x_dtype, ah_ptr residual, ah_ptr out, int32_t out_dtype, uint64_t n, ah_ptr seed_i32,
                         int32_t counter, double p) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(x != 0 && out != 0 && seed_i32 != 0, "ah_dropout_apply: null operand");
  AH_ARG((x_dtype == AH_F32 || x_dtype == AH_BF16) && (out_dtype == AH_F32 || out_dtype == AH_BF16), "ah_dropout_apply: f32 or bf16 operands");
  AH_ARG(p >= 0.0 && p < 1.0, "ah_dropout_apply: p must be in [0,1)");
  AH_ARG(n <= (1ull << 32), "ah_dropout_apply: at most 2^32 elements (the hash sum must stay below 2^63)");
  const int xs = x_dtype == AH_F32 ? 4 : 2, os = out_dtype == AH_F32 ? 4 : 2;
  AH_ARG(x % xs == 0 && out % os == 0 && residual % os == 0 && seed_i32 % 4 == 0, "ah_dropout_apply: misaligned operand");
  const int vec = x % (4 * xs) == 0 && out % (4 * os) == 0 && residual % (4 * os) == 0;
  const float keep = (float)(1.0 / (1.0 - p));
  const dim3 grid(grid_for(vec ? n / 4 + 1 : n)), blk(TPB);
  const int32_t *seed = dp<const int32_t>(seed_i32);
  if (x_dtype == AH_F32 && out_dtype == AH_F32)
    ah::launch_kernel(k_dropout_apply<float, float>, grid, blk, 0, dp<const float>(x), dp<const float>(residual), dp<float>(out), n, seed, counter, p, keep, vec);
  else if (x_dtype == AH_F32)
    ah::launch_kernel(k_dropout_apply<float, uint16_t>, grid, blk, 0, dp<const float>(x), dp<const uint16_t>(residual), dp<uint16_t>(out), n, seed, counter, p, keep, vec);
  else if (out_dtype == AH_F32)
    ah::launch_kernel(k_dropout_apply<uint16_t, float>, grid, blk, 0, dp<const uint16_t>(x), dp<const float>(residual), dp<float>(out), n, seed, counter, p, keep, vec);
  else
    ah::launch_kernel(k_dropout_apply<uint16_t, uint16_t>, grid, blk, 0, dp<const uint16_t>(x), dp<const uint16_t>(residual), dp<uint16_t>(out), n, seed, counter, p, keep, vec);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_masked_fill(ah_ptr a, ah_ptr mask, ah_ptr out, uint64_t n, uint64_t mask_n, float value) {
  AH_REQUIRE_READY();
  if (n == 0) return AH_OK;
  AH_ARG(a && mask && out && mask_n > 0, "ah_masked_fill: null operand or empty mask");
  ah::launch_kernel(k_masked_fill, dim3(grid_for(n)), dim3(TPB), 0, dp<const float>(a), dp<const float>(mask),
                     dp<float>(out), n, mask_n, value);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_causal_mask(ah_ptr out, int64_t size) {
  AH_REQUIRE_READY();
  if (size <= 0) return AH_OK;
  AH_ARG(out != 0, "ah_causal_mask: null out");
  ah::launch_kernel(k_causal_mask, dim3(grid_for((uint64_t)size * size)), dim3(TPB), 0, dp<float>(out), size);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_cast(ah_ptr src, int32_t sd, ah_ptr dst, int32_t dd, uint64_t n) {
  AH_REQUIRE_READY();
  AH_ARG(sd >= AH_F32 && sd <= AH_F16 && dd >= AH_F32 && dd <= AH_F16, "ah_cast: bad dtype");
  if (n == 0) return AH_OK;
  AH_ARG(src && dst, "ah_cast: null operand");
  ah::launch_kernel(k_cast, dim3(grid_for(n)), dim3(TPB), 0, dp<const void>(src), sd, dp<void>(dst), dd, n);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t ah_check_finite(ah_ptr x, uint64_t n, ah_ptr out_flag) {
  AH_REQUIRE_READY();
  AH_ARG(out_flag != 0, "ah_check_finite: null out");
  int32_t rc = ah_fill_f32(out_flag, 0.f, 1);
  if (rc) return rc;
  if (n == 0) return AH_OK;
  AH_ARG(x != 0, "ah_check_finite: null x");
  ah::launch_kernel(k_check_finite, dim3(grid_for(n)), dim3(TPB), 0, dp<const float>(x), n, dp<float>(out_flag));
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_transpose(ah_ptr a, ah_ptr out, int32_t nd, const int64_t *shape, int32_t d0, int32_t d1) {
  AH_REQUIRE_READY();
  AH_ARG(nd >= 1 && nd <= 6, "ah_transpose: nd %d out of range", nd);
  if (d0 < 0) d0 += nd;
  if (d1 < 0) d1 += nd;
  AH_ARG(d0 >= 0 && d0 < nd && d1 >= 0 && d1 < nd, "ah_transpose: axis out of range for ndim %d", nd);
  uint64_t n = (uint64_t)prod(nd, shape);
  if (n == 0) return AH_OK;
  AH_ARG(a && out, "ah_transpose: null operand");
  if (d0 == d1) return ah_copy(out, a, n * 4);
  if (d0 > d1) { int t = d0; d0 = d1; d1 = t; }
  if (d0 == nd - 2 && d1 == nd - 1) {
    int64_t R = shape[nd - 2], C = shape[nd - 1], batch = (int64_t)(n / (uint64_t)(R * C));
    if (batch <= 65535) {
      dim3 grid((unsigned)cdiv(C, 32), (unsigned)cdiv(R, 32), (unsigned)batch);
      ah::launch_kernel(k_transpose_last2, grid, dim3(32, 8), 0, dp<const uint32_t>(a), dp<uint32_t>(out), R, C);
      AH_LAUNCH_CHECK();
      return AH_OK;
    }
  }
  // out[i] over the transposed shape gathers from a with swapped strides
  int64_t st[6]; row_major_strides(nd, shape, st);
  Gather6 g; memset(&g, 0, sizeof g); g.nd = nd; g.offset = 0;      // (zeroed: the unused dimensions and the padding are part of the argument a step plan compares)
  for (int i = 0; i < nd; i++) { g.shape[i] = shape[i]; g.stride[i] = st[i]; }
  { int64_t t = g.shape[d0]; g.shape[d0] = g.shape[d1]; g.shape[d1] = t; t = g.stride[d0]; g.stride[d0] = g.stride[d1]; g.stride[d1] = t; }
  launch_move<false>(dp<const void>(a), dp<void>(out), n, g);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_slice(ah_ptr a, ah_ptr out, int32_t nd, const int64_t *shape, const int64_t *starts, const int64_t *ends) {
  AH_REQUIRE_READY();
  AH_ARG(nd >= 1 && nd <= 6, "ah_slice: nd %d out of range", nd);
  int64_t st[6]; row_major_strides(nd, shape, st);
  Gather6 g; memset(&g, 0, sizeof g); g.nd = nd; g.offset = 0;      // (zeroed: the unused dimensions and the padding are part of the argument a step plan compares)
  for (int i = 0; i < nd; i++) {
    AH_ARG(starts[i] >= 0 && ends[i] <= shape[i] && starts[i] <= ends[i], "ah_slice: range [%lld,%lld) outside dim %d of size %lld",
           (long long)starts[i], (long long)ends[i], i, (long long)shape[i]);
    g.shape[i] = ends[i] - starts[i]; g.stride[i] = st[i]; g.offset += starts[i] * st[i];
  }
  uint64_t n = (uint64_t)prod(nd, g.shape);
  if (n == 0) return AH_OK;
  AH_ARG(a && out, "ah_slice: null operand");
  launch_move<false>(dp<const void>(a), dp<void>(out), n, g);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_scatter_slice(ah_ptr grad, ah_ptr out, int32_t nd, const int64_t *gshape, const int64_t *orig, const int64_t *starts) {
  AH_REQUIRE_READY();
  AH_ARG(nd >= 1 && nd <= 6, "ah_scatter_slice: nd %d out of range", nd);
  int64_t st[6]; row_major_strides(nd, orig, st);
  Gather6 g; memset(&g, 0, sizeof g); g.nd = nd; g.offset = 0;      // (zeroed: the unused dimensions and the padding are part of the argument a step plan compares)
  for (int i = 0; i < nd; i++) {
    AH_ARG(starts[i] >= 0 && starts[i] + gshape[i] <= orig[i], "ah_scatter_slice: slice does not fit dim %d", i);
    g.shape[i] = gshape[i]; g.stride[i] = st[i]; g.offset += starts[i] * st[i];
  }
  uint64_t total = (uint64_t)prod(nd, orig), n = (uint64_t)prod(nd, gshape);
  if (total == 0) return AH_OK;
  AH_ARG(out != 0, "ah_scatter_slice: null out");
  int32_t rc = ah_fill_f32(out, 0.f, total);
  if (rc) return rc;
  if (n == 0) return AH_OK;
  AH_ARG(grad != 0, "ah_scatter_slice: null grad");
  launch_move<true>(dp<const void>(grad), dp<void>(out), n, g);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_cat_part(ah_ptr src, ah_ptr dst, int32_t nd, const int64_t *src_shape, const int64_t *dst_shape, int32_t axis,
                    int64_t axis_offset) {
  AH_REQUIRE_READY();
  AH_ARG(nd >= 1 && nd <= 6, "ah_cat_part: nd %d out of range", nd);
  if (axis < 0) axis += nd;
  AH_ARG(axis >= 0 && axis < nd, "ah_cat_part: axis out of range");
  int64_t st[6]; row_major_strides(nd, dst_shape, st);
  Gather6 g; memset(&g, 0, sizeof g); g.nd = nd; g.offset = axis_offset * st[axis];
  for (int i = 0; i < nd; i++) {
    if (i != axis) AH_ARG(src_shape[i] == dst_shape[i], "cat: shape mismatch at dim %d", i);
    g.shape[i] = src_shape[i]; g.stride[i] = st[i];
  }
  AH_ARG(axis_offset >= 0 && axis_offset + src_shape[axis] <= dst_shape[axis], "ah_cat_part: operand does not fit");
  uint64_t n = (uint64_t)prod(nd, src_shape);
  if (n == 0) return AH_OK;
  AH_ARG(src && dst, "ah_cat_part: null operand");
  launch_move<true>(dp<const void>(src), dp<void>(dst), n, g);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_slice_qkv(ah_ptr qkv, ah_ptr q, ah_ptr k, ah_ptr v, int64_t rows, int64_t d) {
  int64_t shape[2] = {rows, 3 * d};
  ah_ptr outs[3] = {q, k, v};
  for (int i = 0; i < 3; i++) {
    int64_t s[2] = {0, i * d}, e[2] = {rows, (i + 1) * d};
    int32_t rc = ah_slice(qkv, outs[i], 2, shape, s, e);
    if (rc) return rc;
  }
  return AH_OK;
}

int32_t ah_broadcast(ah_ptr a, ah_ptr out, int32_t nd, const int64_t *out_shape, const int64_t *stride_a) {
  AH_REQUIRE_READY();
  AH_ARG(nd >= 0 && nd <= 6, "ah_broadcast: nd %d out of range", nd);
  Gather6 g; memset(&g, 0, sizeof g); g.nd = nd; g.offset = 0;      // (zeroed: the unused dimensions and the padding are part of the argument a step plan compares)
  for (int i = 0; i < nd; i++) { g.shape[i] = out_shape[i]; g.stride[i] = stride_a[i]; }
  uint64_t n = (uint64_t)prod(nd, out_shape);
  if (n == 0) return AH_OK;
  AH_ARG(a && out, "ah_broadcast: null operand");
  launch_move<false>(dp<const void>(a), dp<void>(out), n, g);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

}  // extern "C"
