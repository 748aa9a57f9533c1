// Bandwidth-bound neural-network kernels: embedding gather / scatter-add, LayerNorm forward and
// backward, softmax-cross-entropy forward and backward.  One wave64 owns one row; rows live in
// registers between the statistics pass and the write, so each tensor is read once.
#include "common.h"

using namespace ah;

namespace {

constexpr int TPB = 256;
constexpr int WPB = TPB / 64;

// ---------------------------------------------------------------- embedding
template <class OUT>
__global__ void k_embedding(const float *__restrict__ w, const int32_t *__restrict__ idx, OUT *__restrict__ out,
                            int64_t n_idx, int64_t dim, int64_t vocab) {
  int64_t row = blockIdx.x * (int64_t)WPB + (threadIdx.x >> 6);
  if (row >= n_idx) return;
  int lane = threadIdx.x & 63;
  int64_t r = idx[row];
  bool ok = r >= 0 && r < vocab;                 // an out-of-range id yields a row of NaN, as reading past the weight array
  const float *src = w + (ok ? r : 0) * dim;     // does in the reference's loop (cpu_ref.ts:364-385), and no fault
  OUT *dst = out + row * dim;
  for (int64_t j = lane; j < dim; j += 64) Io<OUT>::st(dst, j, ok ? src[j] : NAN);
}
template <class OUT>
__global__ void k_embedding_tok_pos(const float *__restrict__ wte, const float *__restrict__ wpe, const int32_t *__restrict__ tok,
                                    OUT *__restrict__ out, int64_t n_idx, int64_t T, int64_t dim, int64_t vocab) {
  int64_t row = blockIdx.x * (int64_t)WPB + (threadIdx.x >> 6);
  if (row >= n_idx) return;
  int lane = threadIdx.x & 63;
  int64_t r = tok[row];
  bool ok = r >= 0 && r < vocab;
  const float *a = wte + (ok ? r : 0) * dim, *b = wpe + (row % T) * dim;
  OUT *dst = out + row * dim;
  if ((dim & 3) == 0) {
    for (int64_t j = lane; j < (dim >> 2); j += 64) {
      float4 u = reinterpret_cast<const float4 *>(a)[j], v = reinterpret_cast<const float4 *>(b)[j];
      if (!ok) u = make_float4(NAN, NAN, NAN, NAN);      // (as k_embedding: what the reference's loop reads past the array)
      if constexpr (sizeof(OUT) == 4) reinterpret_cast<float4 *>(dst)[j] = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
      else reinterpret_cast<uint2 *>(dst)[j] = make_uint2(pack_bf16x2(u.x + v.x, u.y + v.y), pack_bf16x2(u.z + v.z, u.w + v.w));
    }
  } else {
    for (int64_t j = lane; j < dim; j += 64) Io<OUT>::st(dst, j, (ok ? a[j] : NAN) + b[j]);
  }
}
// scatter-add with hardware f32 atomics (the reference's GPU kernel uses CAS-loop atomics:
// packages/helios/src/kernels/nn.ts:5300-5345); summation order is not fixed.
__global__ void k_embedding_bwd(const int32_t *__restrict__ idx, const float *__restrict__ g, float *__restrict__ gw,
                                int64_t n_idx, int64_t dim, int64_t vocab) {
  int64_t row = blockIdx.x * (int64_t)WPB + (threadIdx.x >> 6);
  if (row >= n_idx) return;
  int lane = threadIdx.x & 63;
  int64_t r = idx[row];
  if (r < 0 || r >= vocab) return;
  const float *src = g + row * dim;
  float *dst = gw + r * dim;
  for (int64_t j = lane; j < dim; j += 64) unsafeAtomicAdd(dst + j, src[j]);
}
// The same with the repeats inside a block of 64 consecutive positions summed first: a block's first occurrence of an id
// adds up the rows of all its occurrences in the block (in position order) and issues ONE atomic per element.  Token ids
// follow a power law; the most frequent one takes a twelfth of all positions, and atomics to one address are served one
// after the other, which made that row the whole cost of the plain kernel.  One wave per position, 16 at a time; lane l
// holds columns l, l + 64, ... of the 1024 that group y covers.
constexpr int EB_POS = 64;
__global__ __launch_bounds__(1024) void k_embedding_bwd_blocks(const int32_t *__restrict__ idx, const float *__restrict__ g, float *__restrict__ gw,
                                                               int64_t n_idx, int64_t dim, int64_t vocab) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t p0 = blockIdx.x * (int64_t)EB_POS;
  int32_t mine = p0 + lane < n_idx ? idx[p0 + lane] : -1;
  if (mine < 0 || mine >= vocab) mine = -1;                 // ids out of range are skipped
  const int64_t c0 = blockIdx.y * (int64_t)1024 + lane;
  for (int p = wave; p < EB_POS; p += 16) {
    const int32_t t = __shfl(mine, p, 64);
    if (t < 0) continue;
    uint64_t m = __ballot(mine == t);
    if (m & ((1ull << p) - 1)) continue;                    // a repeat: its row is added by the first occurrence
    float acc[16];
#pragma unroll
    for (int k = 0; k < 16; k++) acc[k] = 0.f;
    while (m) {
      const int q = __builtin_ctzll(m);
      m &= m - 1;
      const float *src = g + (p0 + q) * dim;
#pragma unroll
      for (int k = 0; k < 16; k++)
        if (c0 + 64 * k < dim) acc[k] += src[c0 + 64 * k];
    }
    float *dst = gw + (int64_t)t * dim;
#pragma unroll
    for (int k = 0; k < 16; k++)
      if (c0 + 64 * k < dim) unsafeAtomicAdd(dst + c0 + 64 * k, acc[k]);
  }
}
// ---- the same sum with a fixed order of additions (what ah_embedding_bwd runs when the sizes allow) ---------------------
// The reference adds the rows of an id in position order (packages/autograd/src/ops.ts:491-507); atomics add them in whatever
// order the launch happens to take, so the last bit of the gradient changed from run to run.  Here:
//   1. one workgroup sorts the keys (id << 16 | position) of all positions in LDS (bitonic network; ids out of range sort last);
//   2. a wave takes 32 consecutive sorted keys and a slice of 256 columns and adds the rows of each id in its chunk in
//      position order.  An id whose run lies inside the chunk is finished: its row is stored (nobody else writes it).  A run
//      that crosses a chunk border leaves its part in one of the chunk's two side slots;
//   3. for every run that crosses borders, the wave of the chunk where it starts adds the parts chunk by chunk.
// Every row of the result is written by exactly one lane, the order of every addition is a function of the token ids alone.
constexpr int ES_MAX = 32768;           // positions per call (keys must fit the 64 KB ... 128 KB of LDS the sort uses)
constexpr int ES_CHUNK = 32;
__global__ __launch_bounds__(1024) void k_emb_sort(const int32_t *__restrict__ idx, uint32_t *__restrict__ sorted, int n, int npad, int vocab) {
  __shared__ uint32_t keys[ES_MAX];
  for (int i = threadIdx.x; i < npad; i += 1024) {
    uint32_t key = 0xFFFFFFFFu;
    if (i < n) { int32_t t = idx[i]; if (t >= 0 && t < vocab) key = ((uint32_t)t << 16) | (uint32_t)i; }
    keys[i] = key;
  }
  for (int k = 2; k <= npad; k <<= 1)
    for (int j = k >> 1; j > 0; j >>= 1) {
      __syncthreads();
      for (int t = threadIdx.x; t < (npad >> 1); t += 1024) {
        int i = ((t & ~(j - 1)) << 1) | (t & (j - 1)), p = i | j;
        uint32_t a = keys[i], b = keys[p];
        bool up = (i & k) == 0;
        if ((a > b) == up) { keys[i] = b; keys[p] = a; }
      }
    }
  __syncthreads();
  for (int i = threadIdx.x; i < npad; i += 1024) sorted[i] = keys[i];
}
// The same order for up to 16384 positions by a stable radix sort on the id (4 passes of 4 bits; positions enter in order and
// a stable sort keeps them so inside an id): a thread owns npad / 1024 consecutive keys, counts its digits into its own
// column of hist[digit][thread], one scan over hist in (digit, thread) order turns the counts into output offsets, and the
// thread scatters its keys in order.  ~15 us against ~120 us for the bitonic network at 16384 keys.
constexpr int ER_MAX = 16384;
__global__ __launch_bounds__(1024) void k_emb_sort_radix(const int32_t *__restrict__ idx, uint32_t *__restrict__ sorted, int n, int npad, int vocab) {
  __shared__ uint32_t ka[ER_MAX], kb[ER_MAX];
  __shared__ uint16_t hist[16 * 1024];                               // with the keys: all 160 KB of the CU
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per = npad >> 10;                                        // keys per thread (npad is a power of two >= 1024 here)
  for (int i = tid; i < npad; i += 1024) {
    uint32_t key = 0xFFFFFFFFu;
    if (i < n) { int32_t t = idx[i]; if (t >= 0 && t < vocab) key = ((uint32_t)t << 16) | (uint32_t)i; }
    ka[i] = key;
  }
  uint32_t *src = ka, *dst = kb;
  for (int shift = 16; shift < 32; shift += 4) {
    for (int d = 0; d < 16; d++) hist[d * 1024 + tid] = 0;
    __syncthreads();                                                 // keys of the previous pass are in place, own column is clear
    for (int e = 0; e < per; e++) {
      const int d = (src[tid * per + e] >> shift) & 15;
      hist[d * 1024 + tid] = (uint16_t)(hist[d * 1024 + tid] + 1);
    }
    __syncthreads();
    // exclusive scan of hist as one array of 16384 counts: thread t takes entries [16 t, 16 t + 16)
    uint32_t c[16], sum = 0;
#pragma unroll
    for (int q = 0; q < 16; q++) { c[q] = hist[tid * 16 + q]; sum += c[q]; }
    uint32_t incl = sum;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) { uint32_t v = __shfl_up(incl, o, 64); if (lane >= o) incl += v; }
    __syncthreads();                                                 // every count is in registers: hist[0 .. 15] can carry the wave totals
    if (lane == 63) hist[wave] = (uint16_t)incl;                     // at most npad = 16384
    __syncthreads();
    uint32_t base = 0;
    for (int w = 0; w < wave; w++) base += hist[w];
    __syncthreads();
    uint32_t run = base + incl - sum;
#pragma unroll
    for (int q = 0; q < 16; q++) { hist[tid * 16 + q] = (uint16_t)run; run += c[q]; }
    __syncthreads();
    for (int e = 0; e < per; e++) {
      const uint32_t key = src[tid * per + e];
      const int d = (key >> shift) & 15;
      const uint16_t off = hist[d * 1024 + tid];
      hist[d * 1024 + tid] = (uint16_t)(off + 1);
      dst[off] = key;
    }
    __syncthreads();
    uint32_t *t_ = src; src = dst; dst = t_;
  }
  for (int i = tid; i < npad; i += 1024) sorted[i] = src[i];
}
struct EmbChunk { int32_t first_id, last_id, flags, pad; };        // flags: 1 one run only, 2 first run continues the previous chunk's, 4 last run goes on
__device__ __forceinline__ int es_id(uint32_t key) { return key == 0xFFFFFFFFu ? -1 : (int)(key >> 16); }
__global__ __launch_bounds__(256) void k_emb_runs(const uint32_t *__restrict__ sorted, const float *__restrict__ g, float *__restrict__ gw,
                                                  float *__restrict__ part, EmbChunk *__restrict__ meta, int npad, int64_t dim, int accumulate) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = blockIdx.x * 4 + wave;
  if (c * ES_CHUNK >= npad) return;
  const int64_t col = blockIdx.y * (int64_t)256 + lane * 4;
  const bool col_live = col < dim;
  const uint32_t mykey = sorted[c * ES_CHUNK + (lane & 31)];
  const int prev_id = c > 0 ? es_id(sorted[c * ES_CHUNK - 1]) : -1;
  const int next_id = (c + 1) * ES_CHUNK < npad ? es_id(sorted[(c + 1) * ES_CHUNK]) : -1;
  const int first_id = es_id(__shfl(mykey, 0, 64));
  if (first_id < 0) {                                               // nothing but padding
    if (blockIdx.y == 0 && lane == 0) meta[c] = EmbChunk{-1, -1, 0, 0};
    return;
  }
  // all rows of the chunk are requested before the first addition: the additions then run in order at register speed
  float4 rows[ES_CHUNK];
#pragma unroll
  for (int e = 0; e < ES_CHUNK; e++) {
    const uint32_t key = __shfl(mykey, e, 64);
    rows[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (key != 0xFFFFFFFFu && col_live) rows[e] = *reinterpret_cast<const float4 *>(g + (int64_t)(key & 0xFFFFu) * dim + col);
  }
  const bool head_cont = first_id == prev_id;
  int cur = first_id, run = 0, last_id = first_id;
  bool tail_cont = false;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  auto emit = [&](int id, bool is_first, bool is_last_and_goes_on) {
    if (!col_live) return;
    if (is_first && head_cont) *reinterpret_cast<float4 *>(part + ((int64_t)c * 2 + 0) * dim + col) = acc;
    else if (is_last_and_goes_on) *reinterpret_cast<float4 *>(part + ((int64_t)c * 2 + 1) * dim + col) = acc;
    else {
      float4 *dst = reinterpret_cast<float4 *>(gw + (int64_t)id * dim + col);
      if (accumulate) { float4 o = *dst; acc.x += o.x; acc.y += o.y; acc.z += o.z; acc.w += o.w; }
      *dst = acc;
    }
  };
#pragma unroll
  for (int e = 0; e < ES_CHUNK; e++) {
    const int id = es_id(__shfl(mykey, e, 64));
    if (id >= 0) {                                                  // wave-uniform
      if (id != cur) {
        emit(cur, run == 0, false);
        cur = id; run++;
        acc = make_float4(0.f, 0.f, 0.f, 0.f);
      }
      acc.x += rows[e].x; acc.y += rows[e].y; acc.z += rows[e].z; acc.w += rows[e].w;
      last_id = id;
      if (e == ES_CHUNK - 1) tail_cont = id == next_id;
    }
  }
  emit(cur, run == 0, tail_cont);
  if (blockIdx.y == 0 && lane == 0) meta[c] = EmbChunk{first_id, last_id, (run == 0 ? 1 : 0) | (head_cont ? 2 : 0) | (tail_cont ? 4 : 0), 0};
}
__global__ __launch_bounds__(256) void k_emb_join(const float *__restrict__ part, const EmbChunk *__restrict__ meta, float *__restrict__ gw,
                                                  int nchunks, int64_t dim, int accumulate) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c = blockIdx.x * 4 + wave;
  if (c >= nchunks) return;
  const int64_t col = blockIdx.y * (int64_t)256 + lane * 4;
  if (col >= dim) return;
  const EmbChunk m = meta[c];
  // the run that crosses this chunk's right border starts here unless the whole chunk is the middle of a longer run
  if (!(m.flags & 4) || ((m.flags & 1) && (m.flags & 2))) return;
  float4 acc = *reinterpret_cast<const float4 *>(part + ((int64_t)c * 2 + 1) * dim + col);
  for (int cc = c + 1; cc < nchunks; cc++) {
    const EmbChunk mm = meta[cc];
    float4 x = *reinterpret_cast<const float4 *>(part + ((int64_t)cc * 2 + 0) * dim + col);
    acc.x += x.x; acc.y += x.y; acc.z += x.z; acc.w += x.w;
    if (!((mm.flags & 1) && (mm.flags & 4))) break;                // the run ends inside chunk cc
  }
  float4 *dst = reinterpret_cast<float4 *>(gw + (int64_t)m.last_id * dim + col);
  if (accumulate) { float4 o = *dst; acc.x += o.x; acc.y += o.y; acc.z += o.z; acc.w += o.w; }
  *dst = acc;
}

__global__ void k_pos_embedding_bwd(const float *__restrict__ g, float *__restrict__ gw, int64_t batch, int64_t td, int accumulate) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (i >= td) return;
  float s = accumulate ? gw[i] : 0.f;
  for (int64_t b = 0; b < batch; b++) s += g[b * td + i];
  gw[i] = s;
}

// four values of a row as loaded (f32: 16 bytes, bf16: 8 bytes) and widened to float4 at the point of use;
// load_nt: past the caches, for data that is read here for the last time
template <class G> struct Raw4;
template <> struct Raw4<float> {
  float4 v;
  __device__ __forceinline__ void load(const float *p, int j) { v = reinterpret_cast<const float4 *>(p)[j]; }
  __device__ __forceinline__ void load_nt(const float *p, int j) {
    typedef float f4v __attribute__((ext_vector_type(4)));
    const f4v t = __builtin_nontemporal_load(reinterpret_cast<const f4v *>(p) + j);
    v = make_float4(t.x, t.y, t.z, t.w);
  }
  __device__ __forceinline__ void zero() { v = make_float4(0, 0, 0, 0); }
  __device__ __forceinline__ float4 get() const { return v; }
};
template <> struct Raw4<uint16_t> {
  uint2 v;
  __device__ __forceinline__ void load(const uint16_t *p, int j) { v = reinterpret_cast<const uint2 *>(p)[j]; }
  __device__ __forceinline__ void load_nt(const uint16_t *p, int j) {
    typedef unsigned u2v __attribute__((ext_vector_type(2)));
    const u2v t = __builtin_nontemporal_load(reinterpret_cast<const u2v *>(p) + j);
    v = make_uint2(t.x, t.y);
  }
  __device__ __forceinline__ void zero() { v = make_uint2(0, 0); }
  __device__ __forceinline__ float4 get() const {
    return make_float4(bf16_bits_to_f32(v.x & 0xffff), bf16_bits_to_f32(v.x >> 16), bf16_bits_to_f32(v.y & 0xffff), bf16_bits_to_f32(v.y >> 16));
  }
};

// ---------------------------------------------------------------- LayerNorm
// NV = float4 per lane held in registers (row length <= 256*NV); NV == 0: generic re-reading path.
template <int NV, class OUT, class IN = float>
__global__ void k_layernorm(const IN *__restrict__ x, const float *__restrict__ w, const float *__restrict__ b,
                            OUT *__restrict__ out, int64_t rows, int dim, float eps) {
  int64_t row = blockIdx.x * (int64_t)WPB + (threadIdx.x >> 6);
  if (row >= rows) return;
  int lane = threadIdx.x & 63;
  const IN *xr = x + row * (int64_t)dim;
  OUT *orow = out + row * (int64_t)dim;
  float inv_dim = 1.0f / (float)dim;
  if constexpr (NV > 0) {
    int nv = dim >> 2;
    float4 v[NV > 0 ? NV : 1], wv[NV > 0 ? NV : 1], bv[NV > 0 ? NV : 1];
    const bool out_vec = (((uintptr_t)out | ((uintptr_t)dim * sizeof(OUT))) & 7u) == 0;      // 8-byte aligned rows of a 2-byte output
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      int j = lane + 64 * i;
      Raw4<IN> raw;
      if (j < nv) raw.load(xr, j); else raw.zero();
      v[i] = raw.get();
    }
#pragma unroll
    for (int i = 0; i < NV; i++) {       // weight and bias travel with the row instead of behind the two reductions
      int j = lane + 64 * i;
      wv[i] = j < nv ? reinterpret_cast<const float4 *>(w)[j] : make_float4(0, 0, 0, 0);
      bv[i] = j < nv ? reinterpret_cast<const float4 *>(b)[j] : make_float4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < NV; i++) s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    float mean = wave_sum(s) * inv_dim;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      int j = lane + 64 * i;
      if (j < nv) {
        float a = v[i].x - mean, c = v[i].y - mean, d = v[i].z - mean, e = v[i].w - mean;
        q += (a * a + c * c) + (d * d + e * e);
      }
    }
    float rstd = 1.0f / sqrtf(wave_sum(q) * inv_dim + eps);
#pragma unroll
    for (int i = 0; i < NV; i++) {
      int j = lane + 64 * i;
      if (j < nv) {
        float4 ww = wv[i], bb = bv[i];
        float o0 = (v[i].x - mean) * rstd * ww.x + bb.x, o1 = (v[i].y - mean) * rstd * ww.y + bb.y;
        float o2 = (v[i].z - mean) * rstd * ww.z + bb.z, o3 = (v[i].w - mean) * rstd * ww.w + bb.w;
        if constexpr (sizeof(OUT) == 4) reinterpret_cast<float4 *>(orow)[j] = make_float4(o0, o1, o2, o3);
        else if (out_vec) reinterpret_cast<uint2 *>(orow)[j] = make_uint2(pack_bf16x2(o0, o1), pack_bf16x2(o2, o3));
        else {
          Io<OUT>::st(orow, 4 * j + 0, o0); Io<OUT>::st(orow, 4 * j + 1, o1);
          Io<OUT>::st(orow, 4 * j + 2, o2); Io<OUT>::st(orow, 4 * j + 3, o3);
        }
      }
    }
  } else {
    float s = 0.f;
    for (int j = lane; j < dim; j += 64) s += Io<IN>::ld(xr, j);
    float mean = wave_sum(s) * inv_dim;
    float q = 0.f;
    for (int j = lane; j < dim; j += 64) { float d = Io<IN>::ld(xr, j) - mean; q += d * d; }
    float rstd = 1.0f / sqrtf(wave_sum(q) * inv_dim + eps);
    for (int j = lane; j < dim; j += 64) Io<OUT>::st(orow, j, (Io<IN>::ld(xr, j) - mean) * rstd * w[j] + b[j]);
  }
}

// Backward.  Each wave walks rows r = wave_global, += total_waves; per row it recomputes mean / rstd,
// writes dx (+ residual gradient), and adds g*xhat and g into per-lane column accumulators.  The four
// waves of a block then combine through LDS into one partial row of dw/db per block; a second kernel
// sums the partials column-wise in fixed order (deterministic, no [rows, dim] temporaries).
template <class G>
__global__ void k_layernorm_bwd(const float *__restrict__ x, const float *__restrict__ w, const G *__restrict__ g,
                                const float *__restrict__ res, float *__restrict__ dx, uint16_t *__restrict__ dx16, float *__restrict__ part_dw,
                                float *__restrict__ part_db, int64_t rows, int dim, float eps) {
  extern __shared__ float sh[];      // [2][WPB][dim]
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float *my_dw = sh + (size_t)wave * dim, *my_db = sh + (size_t)(WPB + wave) * dim;
  for (int j = lane; j < dim; j += 64) { my_dw[j] = 0.f; my_db[j] = 0.f; }
  float inv_dim = 1.0f / (float)dim;
  int64_t stride = (int64_t)gridDim.x * WPB;
  for (int64_t row = blockIdx.x * (int64_t)WPB + wave; row < rows; row += stride) {
    const float *xr = x + row * (int64_t)dim;
    const G *gr = g + row * (int64_t)dim;
    float s = 0.f;
    for (int j = lane; j < dim; j += 64) s += xr[j];
    float mean = wave_sum(s) * inv_dim;
    float q = 0.f;
    for (int j = lane; j < dim; j += 64) { float d = xr[j] - mean; q += d * d; }
    float rstd = 1.0f / sqrtf(wave_sum(q) * inv_dim + eps);
    float s1 = 0.f, s2 = 0.f;
    for (int j = lane; j < dim; j += 64) {
      float gv = Io<G>::ld(gr, j), xh = (xr[j] - mean) * rstd, dy = gv * w[j];
      s1 += dy; s2 += dy * xh;
      my_dw[j] += gv * xh; my_db[j] += gv;
    }
    s1 = wave_sum(s1); s2 = wave_sum(s2);
    for (int j = lane; j < dim; j += 64) {
      float gv = Io<G>::ld(gr, j), xh = (xr[j] - mean) * rstd, dy = gv * w[j];
      float d = rstd * (dy - (s1 + xh * s2) * inv_dim);
      if (res) d += res[row * (int64_t)dim + j];
      dx[row * (int64_t)dim + j] = d;
      if (dx16) dx16[row * (int64_t)dim + j] = f32_to_bf16_bits(d);
    }
  }
  __syncthreads();
  for (int j = threadIdx.x; j < dim; j += blockDim.x) {
    float a = 0.f, c = 0.f;
    for (int k = 0; k < WPB; k++) { a += sh[(size_t)k * dim + j]; c += sh[(size_t)(WPB + k) * dim + j]; }
    part_dw[(size_t)blockIdx.x * dim + j] = a;
    part_db[(size_t)blockIdx.x * dim + j] = c;
  }
}
// column sums of the per-block partials: 32 columns per block, 32 row slices per column (1024 threads, so that the few
// blocks of this launch keep many loads in flight), fixed summation order
__device__ __forceinline__ void colsum_partials(const float *__restrict__ part_dw, const float *__restrict__ part_db, int nparts, int dim,
                                                float *__restrict__ dw, float *__restrict__ db, int accumulate) {
  __shared__ double sa[32][33], sc[32][33];
  int cx = threadIdx.x & 31, sl = threadIdx.x >> 5, j = blockIdx.x * 32 + cx;
  double a = 0, c = 0;
  if (j < dim) {
    int p = sl;
    for (; p + 96 < nparts; p += 128) {        // four independent loads per array in flight
      float a0 = part_dw[(size_t)p * dim + j], a1 = part_dw[(size_t)(p + 32) * dim + j], a2 = part_dw[(size_t)(p + 64) * dim + j],
            a3 = part_dw[(size_t)(p + 96) * dim + j];
      float c0 = part_db[(size_t)p * dim + j], c1 = part_db[(size_t)(p + 32) * dim + j], c2 = part_db[(size_t)(p + 64) * dim + j],
            c3 = part_db[(size_t)(p + 96) * dim + j];
      a += a0; a += a1; a += a2; a += a3;
      c += c0; c += c1; c += c2; c += c3;
    }
    for (; p < nparts; p += 32) { a += part_dw[(size_t)p * dim + j]; c += part_db[(size_t)p * dim + j]; }
  }
  sa[sl][cx] = a; sc[sl][cx] = c;
  __syncthreads();
  if (sl == 0 && j < dim) {
    for (int k = 1; k < 32; k++) { a += sa[k][cx]; c += sc[k][cx]; }
    dw[j] = (accumulate ? dw[j] : 0.f) + (float)a;
    db[j] = (accumulate ? db[j] : 0.f) + (float)c;
  }
}
__global__ __launch_bounds__(1024) void k_colsum_partials(const float *__restrict__ part_dw, const float *__restrict__ part_db, int nparts, int dim,
                                                          float *__restrict__ dw, float *__restrict__ db, int accumulate) {
  colsum_partials(part_dw, part_db, nparts, dim, dw, db, accumulate);
}
// the column sums of several LayerNorms in one launch (job y), the jobs passed by value
struct ColsumJob { const float *part; float *dw, *db; int nparts, dim, accumulate, pad; };
constexpr int COLSUM_JOBS = 64;
struct ColsumJobs { ColsumJob j[COLSUM_JOBS]; };
__global__ __launch_bounds__(1024) void k_colsum_partials_batched(ColsumJobs jobs) {
  const ColsumJob &q = jobs.j[blockIdx.y];
  if ((int)blockIdx.x * 32 >= q.dim) return;
  colsum_partials(q.part, q.part + (size_t)q.nparts * q.dim, q.nparts, q.dim, q.dw, q.db, q.accumulate);
}

// Register-resident LayerNorm backward for rows of up to 256*NV floats (dim % 4 == 0): x, g and the residual gradient
// are each read once; dw / db accumulate in per-lane registers over all rows a wave walks.
// A wave walks its rows with the NEXT row's x, g and residual gradient already in flight while it reduces the current
// one: a row is three dependent wave reductions long, and with the few waves per SIMD that the register-resident
// column sums allow, nothing else would cover the load latency.
// X = type of x and of the residual gradient (the residual stream and its gradient stream: f32, or bf16 when the caller keeps
// them in bf16; dx may then be null, dx16 being the stream)
template <int NV, class G, class X = float>
__global__ __launch_bounds__(256) void k_layernorm_bwd_vec(const X *__restrict__ x, const float *__restrict__ w, const G *__restrict__ g,
                                                           const X *__restrict__ res, float *__restrict__ dx, uint16_t *__restrict__ dx16,
                                                           float *__restrict__ part_dw, float *__restrict__ part_db, int64_t rows, int dim, float eps) {
  extern __shared__ float sh[];      // [2][WPB][dim]
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nv = dim >> 2;
  float inv_dim = 1.0f / (float)dim;
  float4 wv[NV], adw[NV], adb[NV];
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int j = lane + 64 * i;
    wv[i] = j < nv ? reinterpret_cast<const float4 *>(w)[j] : make_float4(0, 0, 0, 0);
    adw[i] = make_float4(0, 0, 0, 0); adb[i] = make_float4(0, 0, 0, 0);
  }
  float4 xv[NV], rv[NV];
  Raw4<X> nx[NV], nr[NV];
  Raw4<G> gr[NV], ng[NV];
  auto load_row = [&](int64_t row, Raw4<X> (&xo)[NV], Raw4<G> (&go)[NV], Raw4<X> (&ro)[NV]) {
    const X *xr = x + row * (int64_t)dim;
    const G *grow = g + row * (int64_t)dim;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      int j = lane + 64 * i;
      if (j < nv) {
        // x and the residual gradient were written long ago and are used here for the last time; dx (f32) is next read two
        // GEMMs and an attention later: all three go past the caches (the bf16 copy of dx, the next GEMM's operand, does not)
        xo[i].load_nt(xr, j);
        go[i].load(grow, j);
        if (res) ro[i].load_nt(res + row * (int64_t)dim, j);
        else ro[i].zero();
      } else {
        xo[i].zero(); go[i].zero(); ro[i].zero();
      }
    }
  };
  int64_t stride = (int64_t)gridDim.x * WPB, row = blockIdx.x * (int64_t)WPB + wave;
  if (row < rows) {
    load_row(row, nx, gr, nr);
#pragma unroll
    for (int i = 0; i < NV; i++) { xv[i] = nx[i].get(); rv[i] = nr[i].get(); }
  }
  for (; row < rows; row += stride) {
    if (row + stride < rows) load_row(row + stride, nx, ng, nr);
    float4 gv[NV];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      gv[i] = gr[i].get();
      s += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
    }
    float mean = wave_sum(s) * inv_dim, q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++)
      if (lane + 64 * i < nv) {
        float a = xv[i].x - mean, b = xv[i].y - mean, c = xv[i].z - mean, d = xv[i].w - mean;
        q += (a * a + b * b) + (c * c + d * d);
      }
    float rstd = 1.0f / sqrtf(wave_sum(q) * inv_dim + eps), s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {       // xv becomes xhat; out-of-range lanes hold g = w = 0 and contribute nothing
      xv[i].x = (xv[i].x - mean) * rstd; xv[i].y = (xv[i].y - mean) * rstd; xv[i].z = (xv[i].z - mean) * rstd; xv[i].w = (xv[i].w - mean) * rstd;
      float d0 = gv[i].x * wv[i].x, d1 = gv[i].y * wv[i].y, d2 = gv[i].z * wv[i].z, d3 = gv[i].w * wv[i].w;
      s1 += (d0 + d1) + (d2 + d3);
      s2 += (d0 * xv[i].x + d1 * xv[i].y) + (d2 * xv[i].z + d3 * xv[i].w);
      adw[i].x += gv[i].x * xv[i].x; adw[i].y += gv[i].y * xv[i].y; adw[i].z += gv[i].z * xv[i].z; adw[i].w += gv[i].w * xv[i].w;
      adb[i].x += gv[i].x; adb[i].y += gv[i].y; adb[i].z += gv[i].z; adb[i].w += gv[i].w;
    }
    s1 = wave_sum(s1) * inv_dim; s2 = wave_sum(s2) * inv_dim;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      int j = lane + 64 * i;
      if (j < nv) {
        float4 d;
        d.x = rstd * (gv[i].x * wv[i].x - (s1 + xv[i].x * s2)); d.y = rstd * (gv[i].y * wv[i].y - (s1 + xv[i].y * s2));
        d.z = rstd * (gv[i].z * wv[i].z - (s1 + xv[i].z * s2)); d.w = rstd * (gv[i].w * wv[i].w - (s1 + xv[i].w * s2));
        if (res) { d.x += rv[i].x; d.y += rv[i].y; d.z += rv[i].z; d.w += rv[i].w; }
        if (dx) { typedef float f4v __attribute__((ext_vector_type(4))); __builtin_nontemporal_store(f4v{d.x, d.y, d.z, d.w}, reinterpret_cast<f4v *>(dx + row * (int64_t)dim) + j); }
        if (dx16) reinterpret_cast<uint2 *>(dx16 + row * (int64_t)dim)[j] = make_uint2(pack_bf16x2(d.x, d.y), pack_bf16x2(d.z, d.w));
      }
    }
#pragma unroll
    for (int i = 0; i < NV; i++) { xv[i] = nx[i].get(); gr[i] = ng[i]; rv[i] = nr[i].get(); }
  }
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int j = lane + 64 * i;
    if (j < nv) {
      reinterpret_cast<float4 *>(sh + (size_t)wave * dim)[j] = adw[i];
      reinterpret_cast<float4 *>(sh + (size_t)(WPB + wave) * dim)[j] = adb[i];
    }
  }
  __syncthreads();
  for (int j = threadIdx.x; j < dim; j += blockDim.x) {
    float a = 0.f, c = 0.f;
    for (int k = 0; k < WPB; k++) { a += sh[(size_t)k * dim + j]; c += sh[(size_t)(WPB + k) * dim + j]; }
    part_dw[(size_t)blockIdx.x * dim + j] = a;
    part_db[(size_t)blockIdx.x * dim + j] = c;
  }
}

// ---------------------------------------------------------------- softmax cross-entropy
// exp(v - m) through the bare base-2 exponential (the vector paths of the three kernels below use the same form, so their
// results agree bit for bit).  The difference is taken first, as the reference takes it (cpu_ref.ts:493-563): folded into
// one multiply-add, v log2(e) - m log2(e), the rounding of the second product is an error of |m| 2^-24 in the exponent -
// nothing at |m| < 100, a wrong loss for logits of 1e6, an infinite one at 1e30.
constexpr float CE_LOG2E = 1.4426950408889634f;
__device__ __forceinline__ float exp_minus(float v, float m) { return __builtin_amdgcn_exp2f((v - m) * CE_LOG2E); }
__device__ __forceinline__ void online_merge(float &m, float &s, float m2, float s2) {
  float nm = fmaxf(m, m2);
  if (nm == -INFINITY) { m = nm; s = 0.f; return; }
  s = s * expf(m - nm) + s2 * expf(m2 - nm);
  m = nm;
}
// one block per row: single read of the row with an online (max, sum-exp) pair per thread
template <class T>
__global__ void k_ce_fwd(const T *__restrict__ logits, const int32_t *__restrict__ targets, float *__restrict__ row_loss,
                         float *__restrict__ lse_out, int64_t c) {
  __shared__ float shm[16], shs[16];                    // one pair per wave of the block (up to 1024 threads)
  int64_t row = blockIdx.x;
  const T *p = logits + row * c;
  float m = -INFINITY, s = 0.f;
  constexpr int VW = 16 / sizeof(T);                    // elements per 16-byte load
  int64_t nvec = ((((uintptr_t)p) & 15u) == 0) ? c / VW : 0;
  for (int64_t j = threadIdx.x; j < nvec; j += blockDim.x) {
    uint4 u = reinterpret_cast<const uint4 *>(p)[j];
    float v[VW];
    if (sizeof(T) == 4) { v[0] = __uint_as_float(u.x); v[1] = __uint_as_float(u.y); v[2] = __uint_as_float(u.z); v[VW - 1] = __uint_as_float(u.w); }
    else {
      v[0] = bf16_bits_to_f32(u.x & 0xffff); v[1] = bf16_bits_to_f32(u.x >> 16); v[2] = bf16_bits_to_f32(u.y & 0xffff); v[3] = bf16_bits_to_f32(u.y >> 16);
      v[VW - 4] = bf16_bits_to_f32(u.z & 0xffff); v[VW - 3] = bf16_bits_to_f32(u.z >> 16); v[VW - 2] = bf16_bits_to_f32(u.w & 0xffff); v[VW - 1] = bf16_bits_to_f32(u.w >> 16);
    }
    float vm = v[0];
#pragma unroll
    for (int i = 1; i < VW; i++) vm = fmaxf(vm, v[i]);
    if (vm > m) { s *= __expf(m - vm); m = vm; }
#pragma unroll
    for (int i = 0; i < VW; i++) s += exp_minus(v[i], m);
  }
  for (int64_t j = nvec * VW + threadIdx.x; j < c; j += blockDim.x) {
    float v = Io<T>::ld(p, j);
    if (v > m) { s = s * expf(m - v) + 1.0f; m = v; } else { s += expf(v - m); }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) online_merge(m, s, __shfl_xor(m, off, 64), __shfl_xor(s, off, 64));
  int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) { shm[wv] = m; shs[wv] = s; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < (int)(blockDim.x >> 6); k++) online_merge(m, s, shm[k], shs[k]);
    float lse = m + logf(s);
    int32_t t = targets[row];
    float picked = (t >= 0 && t < c) ? Io<T>::ld(p, t) : lse;     // an out-of-range target contributes 0 loss
    row_loss[row] = lse - picked;
    if (lse_out) lse_out[row] = lse;
  }
}
__global__ void k_mean_rows(const float *__restrict__ v, int64_t n, float *__restrict__ out) {
  __shared__ double sh[WPB];
  double s = 0;
  int64_t i = threadIdx.x;
  for (; i + 7 * (int64_t)blockDim.x < n; i += 8 * (int64_t)blockDim.x) {        // eight independent loads in flight (one block runs this)
    float x[8];
#pragma unroll
    for (int k = 0; k < 8; k++) x[k] = v[i + k * (int64_t)blockDim.x];
#pragma unroll
    for (int k = 0; k < 8; k++) s += (double)x[k];
  }
  for (; i < n; i += blockDim.x) s += (double)v[i];
  s = wave_sum_d(s);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    double t = 0;
    for (int k = 0; k < WPB; k++) t += sh[k];
    out[0] = (float)(t / (double)n);
  }
}
// (softmax - onehot) * scale for 8 bf16 logits: the subtraction of the one-hot is only spelled out in the one chunk of
// a row that holds the target (`hot` = its position there, else -1); everywhere else (e - 0) * scale == e * scale bit for bit.
__device__ __forceinline__ void ce_grad8(const uint4 &u, float lse, float scale, int hot, uint32_t (&o)[4]) {
  const uint32_t in[4] = {u.x, u.y, u.z, u.w};
  float e[8];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    e[2 * i] = exp_minus(bf16_bits_to_f32(in[i] & 0xffff), lse);
    e[2 * i + 1] = exp_minus(bf16_bits_to_f32(in[i] >> 16), lse);
  }
  if (hot >= 0) {
#pragma unroll
    for (int i = 0; i < 8; i++) e[i] -= (i == hot ? 1.0f : 0.0f);
  }
#pragma unroll
  for (int i = 0; i < 4; i++) o[i] = pack_bf16x2(e[2 * i] * scale, e[2 * i + 1] * scale);
}
template <class T>
__global__ void k_ce_bwd(const T *__restrict__ logits, const int32_t *__restrict__ targets, const float *__restrict__ lse,
                         const float *__restrict__ g, float g_mul, T *__restrict__ out, int64_t n, int64_t c) {
  int64_t row = blockIdx.y;
  float scale = (g ? g[0] : 1.0f) * g_mul / (float)n;
  float l = lse[row];
  int32_t t = targets[row];
  const T *p = logits + row * c;
  T *q = out + row * c;
  if (sizeof(T) == 2 && (c & 7) == 0 && (((uintptr_t)logits | (uintptr_t)out) & 15u) == 0) {      // bf16: 8 classes per 16-byte access
    for (int64_t j8 = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; j8 < (c >> 3); j8 += (int64_t)gridDim.x * blockDim.x) {
      uint4 u = reinterpret_cast<const uint4 *>(p)[j8];
      uint32_t o[4];
      ce_grad8(u, l, scale, j8 == (t >> 3) ? (int)(t & 7) : -1, o);
      reinterpret_cast<uint4 *>(q)[j8] = make_uint4(o[0], o[1], o[2], o[3]);
    }
    return;
  }
  for (int64_t j = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; j < c; j += (int64_t)gridDim.x * blockDim.x) {
    float prob = expf(Io<T>::ld(p, j) - l);
    Io<T>::st(q, j, (prob - (j == t ? 1.0f : 0.0f)) * scale);
  }
}

// Forward and backward of the loss in ONE pass over bf16 logits: the block keeps its whole row in registers (up to
// CE_CHUNKS 16-byte chunks per thread), so the logits are read once instead of twice.  Same per-thread order of the online
// (max, sum) updates and the same expressions as k_ce_fwd / k_ce_bwd: results are bit-identical to that pair.
#ifndef CE_TPB
#define CE_TPB 512        // measured at 16384 x 50304: 636 us with 512 threads per row, 670 with 256, 793 with 1024
#endif
constexpr int CE_CHUNKS = (51200 / 8 + CE_TPB - 1) / CE_TPB;      // CE_CHUNKS x CE_TPB threads x 8 classes >= 51200 classes per row
constexpr int CE_WPB = CE_TPB / 64;
__global__ __launch_bounds__(CE_TPB) void k_ce_fwd_bwd(const uint16_t *__restrict__ logits, const int32_t *__restrict__ targets,
                                                    float *__restrict__ row_loss, float *__restrict__ lse_out, const float *__restrict__ g,
                                                    float g_mul, uint16_t *__restrict__ out, int64_t n, int64_t c) {
  __shared__ float shm[CE_WPB], shs[CE_WPB], sh_lse;
  const int64_t row = blockIdx.x;
  const uint16_t *p = logits + row * c;
  const int nvec = (int)(c >> 3);
  uint4 r[CE_CHUNKS];
  float m = -INFINITY, s = 0.f;
#pragma unroll
  for (int k = 0; k < CE_CHUNKS; k++) {
    const int j = threadIdx.x + k * CE_TPB;
    if (j < nvec) {
      typedef unsigned u4v __attribute__((ext_vector_type(4)));     // 1.65 GB read once and written once: non-temporal (-6 %)
      const u4v un = __builtin_nontemporal_load(reinterpret_cast<const u4v *>(p) + j);
      const uint4 u = make_uint4(un.x, un.y, un.z, un.w);
      r[k] = u;
      float v[8] = {bf16_bits_to_f32(u.x & 0xffff), bf16_bits_to_f32(u.x >> 16), bf16_bits_to_f32(u.y & 0xffff), bf16_bits_to_f32(u.y >> 16),
                    bf16_bits_to_f32(u.z & 0xffff), bf16_bits_to_f32(u.z >> 16), bf16_bits_to_f32(u.w & 0xffff), bf16_bits_to_f32(u.w >> 16)};
      float vm = v[0];
#pragma unroll
      for (int i = 1; i < 8; i++) vm = fmaxf(vm, v[i]);
      if (vm > m) { s *= __expf(m - vm); m = vm; }
#pragma unroll
      for (int i = 0; i < 8; i++) s += exp_minus(v[i], m);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) online_merge(m, s, __shfl_xor(m, off, 64), __shfl_xor(s, off, 64));
  const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) { shm[wv] = m; shs[wv] = s; }
  __syncthreads();
  const int32_t t = targets[row];
  if (threadIdx.x == 0) {
    for (int k = 1; k < CE_WPB; k++) online_merge(m, s, shm[k], shs[k]);
    const float lse = m + logf(s);
    const float picked = (t >= 0 && t < c) ? bf16_bits_to_f32(p[t]) : lse;     // an out-of-range target contributes 0 loss
    row_loss[row] = lse - picked;
    if (lse_out) lse_out[row] = lse;
    sh_lse = lse;
  }
  __syncthreads();
  const float l = sh_lse, scale = (g ? g[0] : 1.0f) * g_mul / (float)n;
  uint16_t *q = out + row * c;
#pragma unroll
  for (int k = 0; k < CE_CHUNKS; k++) {
    const int j8 = threadIdx.x + k * CE_TPB;
    if (j8 < nvec) {
      uint32_t o[4];
      ce_grad8(r[k], l, scale, j8 == (t >> 3) ? (int)(t & 7) : -1, o);
      typedef unsigned u4v __attribute__((ext_vector_type(4)));
      __builtin_nontemporal_store(u4v{o[0], o[1], o[2], o[3]}, reinterpret_cast<u4v *>(q) + j8);
    }
  }
}

// Token windows of a device-resident corpus: one block row per batch item, modulo indexing reproduces the packed
// loader's wrap-around (and is a no-op for random windows, which never reach the end of the corpus).
__global__ void k_token_windows(const int32_t *__restrict__ corpus, int64_t n_tokens, const int64_t *__restrict__ starts, int64_t T,
                                int32_t *__restrict__ inputs, int32_t *__restrict__ targets) {
  int64_t b = blockIdx.y, start = starts[b];
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < T; t += (int64_t)gridDim.x * blockDim.x) {
    int64_t p = (start + t) % n_tokens, q = p + 1 == n_tokens ? 0 : p + 1;
    inputs[b * T + t] = corpus[p];
    targets[b * T + t] = corpus[q];
  }
}

}  // namespace

template <class OUT, class IN>
static int32_t launch_ln(ah_ptr x, ah_ptr w, ah_ptr b, ah_ptr out, int64_t rows, int64_t dim, float eps) {
  dim3 grid((unsigned)cdiv(rows, WPB)), blk(TPB);
  bool vec = (dim % 4 == 0) && dim <= 2048 && x % (4 * sizeof(IN)) == 0 && aligned16(w) && aligned16(b) && (sizeof(OUT) == 2 || aligned16(out));
  int nvl = vec ? (int)cdiv(dim / 4, 64) : 0;
#define LN_CASE(NV) ah::launch_kernel((k_layernorm<NV, OUT, IN>), grid, blk, 0, dp<const IN>(x), dp<const float>(w), dp<const float>(b), dp<OUT>(out), rows, (int)dim, eps)
  switch (nvl) {
    case 1: LN_CASE(1); break;
    case 2: LN_CASE(2); break;
    case 3: LN_CASE(3); break;
    case 4: LN_CASE(4); break;
    case 5: case 6: LN_CASE(6); break;
    case 7: case 8: LN_CASE(8); break;
    default: LN_CASE(0); break;
  }
#undef LN_CASE
  AH_LAUNCH_CHECK();
  return AH_OK;
}

extern "C" {

int32_t ah_embedding(ah_ptr weight, ah_ptr idx, ah_ptr out, int64_t n_idx, int64_t dim, int64_t vocab, int32_t out_dtype) {
  AH_REQUIRE_READY();
  AH_ARG(out_dtype == AH_F32 || out_dtype == AH_BF16, "ah_embedding: out dtype must be f32 or bf16");
  if (n_idx == 0 || dim == 0) return AH_OK;
  AH_ARG(weight && idx && out, "ah_embedding: null operand");
  dim3 grid((unsigned)cdiv(n_idx, WPB));
  if (out_dtype == AH_F32)
    ah::launch_kernel(k_embedding<float>, grid, dim3(TPB), 0, dp<const float>(weight), dp<const int32_t>(idx), dp<float>(out), n_idx, dim, vocab);
  else
    ah::launch_kernel(k_embedding<uint16_t>, grid, dim3(TPB), 0, dp<const float>(weight), dp<const int32_t>(idx), dp<uint16_t>(out), n_idx, dim, vocab);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_embedding_tok_pos(ah_ptr wte, ah_ptr wpe, ah_ptr tok, ah_ptr out, int64_t n_idx, int64_t T, int64_t dim, int64_t vocab,
                             int32_t out_dtype) {
  AH_REQUIRE_READY();
  AH_ARG(out_dtype == AH_F32 || out_dtype == AH_BF16, "ah_embedding_tok_pos: out dtype must be f32 or bf16");
  if (n_idx == 0 || dim == 0) return AH_OK;
  AH_ARG(wte && wpe && tok && out && T > 0, "ah_embedding_tok_pos: null operand");
  AH_ARG(aligned16(wte) && aligned16(wpe) && aligned16(out), "ah_embedding_tok_pos: operands must be 16-byte aligned");
  if (out_dtype == AH_F32)
    ah::launch_kernel(k_embedding_tok_pos<float>, dim3((unsigned)cdiv(n_idx, WPB)), dim3(TPB), 0, dp<const float>(wte),
                       dp<const float>(wpe), dp<const int32_t>(tok), dp<float>(out), n_idx, T, dim, vocab);
  else
    ah::launch_kernel(k_embedding_tok_pos<uint16_t>, dim3((unsigned)cdiv(n_idx, WPB)), dim3(TPB), 0, dp<const float>(wte),
                       dp<const float>(wpe), dp<const int32_t>(tok), dp<uint16_t>(out), n_idx, T, dim, vocab);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_token_windows(ah_ptr corpus, int64_t n_tokens, ah_ptr starts, int64_t batch, int64_t T, ah_ptr inputs, ah_ptr targets) {
  AH_REQUIRE_READY();
  AH_ARG(batch >= 0 && T >= 0 && batch <= 65535, "ah_token_windows: bad batch %lld / block %lld", (long long)batch, (long long)T);
  if (batch == 0 || T == 0) return AH_OK;
  AH_ARG(n_tokens > 0, "ah_token_windows: empty corpus");
  AH_ARG(corpus && starts && inputs && targets, "ah_token_windows: null operand");
  unsigned bx = (unsigned)(cdiv(T, 256) < 64 ? cdiv(T, 256) : 64);
  ah::launch_kernel(k_token_windows, dim3(bx, (unsigned)batch), dim3(256), 0, dp<const int32_t>(corpus), n_tokens,
                     dp<const int64_t>(starts), T, dp<int32_t>(inputs), dp<int32_t>(targets));
  AH_LAUNCH_CHECK();
  return AH_OK;
}

static int es_npad(int64_t n_idx) {
  int npad = 64;
  while (npad < n_idx) npad <<= 1;
  return npad;
}
int64_t ah_embedding_index_bytes(int64_t n_idx, int64_t vocab) {
  return (n_idx >= 1 && n_idx <= ES_MAX && vocab >= 1 && vocab < 65535) ? (int64_t)es_npad(n_idx) * 4 : 0;
}
int32_t ah_embedding_index(ah_ptr idx, int64_t n_idx, int64_t vocab, ah_ptr index_out) {
  AH_REQUIRE_READY();
  AH_ARG(ah_embedding_index_bytes(n_idx, vocab) > 0, "ah_embedding_index: %lld positions over %lld ids is outside the indexed path (at most %d positions, ids below 65535)",
         (long long)n_idx, (long long)vocab, ES_MAX);
  AH_ARG(idx && index_out, "ah_embedding_index: null operand");
  const int npad = es_npad(n_idx);
  if (npad >= 1024 && npad <= ER_MAX)
    ah::launch_kernel(k_emb_sort_radix, dim3(1), dim3(1024), 0, dp<const int32_t>(idx), dp<uint32_t>(index_out), (int)n_idx, npad, (int)vocab);
  else
    ah::launch_kernel(k_emb_sort, dim3(1), dim3(1024), 0, dp<const int32_t>(idx), dp<uint32_t>(index_out), (int)n_idx, npad, (int)vocab);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
// zero fill (unless accumulating) must already have happened
static int32_t embedding_bwd_sorted(ah_ptr index, ah_ptr grad_out, ah_ptr grad_w, int64_t n_idx, int64_t dim, int32_t accumulate) {
  const int npad = es_npad(n_idx), nchunks = npad / ES_CHUNK;
  const size_t b_meta = ((size_t)nchunks * sizeof(EmbChunk) + 255) & ~size_t(255), b_part = (size_t)nchunks * 2 * dim * 4;
  ah_ptr ws = 0;
  int32_t rc = ah_alloc(b_meta + b_part, &ws);
  if (rc) return rc;
  EmbChunk *meta = dp<EmbChunk>(ws);
  float *part = reinterpret_cast<float *>(dp<char>(ws) + b_meta);
  dim3 grid((unsigned)cdiv(nchunks, 4), (unsigned)cdiv(dim, 256));
  ah::launch_kernel(k_emb_runs, grid, dim3(256), 0, dp<const uint32_t>(index), dp<const float>(grad_out), dp<float>(grad_w), part, meta, npad, dim,
                    (int)accumulate);
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_emb_join, grid, dim3(256), 0, (const float *)part, (const EmbChunk *)meta, dp<float>(grad_w), nchunks, dim, (int)accumulate);
  AH_LAUNCH_CHECK();
  return ah_free(ws);
}
int32_t ah_embedding_bwd_indexed(ah_ptr index, ah_ptr grad_out, ah_ptr grad_w, int64_t n_idx, int64_t dim, int64_t vocab, int32_t accumulate) {
  AH_REQUIRE_READY();
  AH_ARG(grad_w != 0 || vocab * dim == 0, "ah_embedding_bwd_indexed: null grad_w");
  if (!accumulate) { int32_t rc = ah_fill_f32(grad_w, 0.f, (uint64_t)(vocab * dim)); if (rc) return rc; }
  if (n_idx == 0 || dim == 0) return AH_OK;
  AH_ARG(ah_embedding_index_bytes(n_idx, vocab) > 0, "ah_embedding_bwd_indexed: sizes outside the indexed path");
  AH_ARG(index && grad_out, "ah_embedding_bwd_indexed: null operand");
  AH_ARG(dim % 4 == 0 && cdiv(dim, 256) <= 65535 && aligned16(grad_out) && aligned16(grad_w), "ah_embedding_bwd_indexed: rows must be 16-byte aligned multiples of 4 floats");
  return embedding_bwd_sorted(index, grad_out, grad_w, n_idx, dim, accumulate);
}

int32_t ah_embedding_bwd(ah_ptr idx, ah_ptr grad_out, ah_ptr grad_w, int64_t n_idx, int64_t dim, int64_t vocab, int32_t accumulate) {
  AH_REQUIRE_READY();
  AH_ARG(grad_w != 0 || vocab * dim == 0, "ah_embedding_bwd: null grad_w");
  if (!accumulate) { int32_t rc = ah_fill_f32(grad_w, 0.f, (uint64_t)(vocab * dim)); if (rc) return rc; }
  if (n_idx == 0 || dim == 0) return AH_OK;
  AH_ARG(idx && grad_out, "ah_embedding_bwd: null operand");
  if (ah_embedding_index_bytes(n_idx, vocab) > 0 && dim % 4 == 0 && cdiv(dim, 256) <= 65535 && aligned16(grad_out) && aligned16(grad_w)) {
    // fixed summation order: sort the positions by id, then ah_embedding_bwd_indexed
    ah_ptr index = 0;
    int32_t rc = ah_alloc((uint64_t)ah_embedding_index_bytes(n_idx, vocab), &index);
    if (rc) return rc;
    rc = ah_embedding_index(idx, n_idx, vocab, index);
    if (rc == AH_OK) rc = embedding_bwd_sorted(index, grad_out, grad_w, n_idx, dim, accumulate);
    int32_t rc2 = ah_free(index);
    return rc ? rc : rc2;
  }
  if (cdiv(n_idx, EB_POS) < (1ll << 31) && cdiv(dim, 1024) <= 65535)
    ah::launch_kernel(k_embedding_bwd_blocks, dim3((unsigned)cdiv(n_idx, EB_POS), (unsigned)cdiv(dim, 1024)), dim3(1024), 0, 
                       dp<const int32_t>(idx), dp<const float>(grad_out), dp<float>(grad_w), n_idx, dim, vocab);
  else
    ah::launch_kernel(k_embedding_bwd, dim3((unsigned)cdiv(n_idx, WPB)), dim3(TPB), 0, dp<const int32_t>(idx),
                       dp<const float>(grad_out), dp<float>(grad_w), n_idx, dim, vocab);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_pos_embedding_bwd(ah_ptr grad_out, ah_ptr grad_wpe, int64_t batch, int64_t T, int64_t dim, int32_t accumulate) {
  AH_REQUIRE_READY();
  int64_t td = T * dim;
  if (td == 0) return AH_OK;
  AH_ARG(grad_out && grad_wpe, "ah_pos_embedding_bwd: null operand");
  ah::launch_kernel(k_pos_embedding_bwd, dim3((unsigned)cdiv(td, TPB)), dim3(TPB), 0, dp<const float>(grad_out),
                     dp<float>(grad_wpe), batch, td, accumulate);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_layernorm(ah_ptr x, ah_ptr w, ah_ptr b, ah_ptr out, int64_t rows, int64_t dim, float eps, int32_t out_dtype, int32_t x_dtype) {
  AH_REQUIRE_READY();
  AH_ARG(out_dtype == AH_F32 || out_dtype == AH_BF16, "ah_layernorm: out dtype must be f32 or bf16");
  AH_ARG(x_dtype == AH_F32 || (x_dtype == AH_BF16 && out_dtype == AH_BF16), "ah_layernorm: x is f32, or bf16 with a bf16 result");
  if (rows == 0 || dim == 0) return AH_OK;
  AH_ARG(x && w && b && out, "ah_layernorm: null operand");
  AH_ARG(dim < (int64_t(1) << 30), "ah_layernorm: row too long");
  if (x_dtype == AH_BF16) return launch_ln<uint16_t, uint16_t>(x, w, b, out, rows, dim, eps);
  return out_dtype == AH_F32 ? launch_ln<float, float>(x, w, b, out, rows, dim, eps) : launch_ln<uint16_t, float>(x, w, b, out, rows, dim, eps);
}

// Blocks of a LayerNorm-backward launch = rows of its partial column sums; a function of the shape alone, because the caller
// sizes the partials by it (ah_layernorm_bwd_partials_bytes) and the column sums walk them.  The kernel is bound by the latency of
// a row's loads (a wave has one row in flight beyond the one it reduces), so as many blocks as stay resident together, and no
// more: a block beyond that runs alone in a second round.  Resident blocks per CU by registers, the least over the stream and
// gradient types of a row length: 4 up to 512 elements, 3 up to 768, 2 beyond (16384 x 768: 21.3 us with two blocks per CU of
// eight rows a wave, 19.5 with three of five or six, 24.4 with four; 8192 x 1024: 22.0 -> 16.1 us).
static int ln_bwd_blocks(int64_t rows, int64_t dim) {
  int64_t nblk = cdiv(rows, WPB * 4);             // >= 4 rows per wave amortise the partial write
  int64_t cap = (int64_t)num_cus() * (dim <= 512 ? 4 : dim <= 768 ? 3 : 2);
  if (nblk > cap) nblk = cap;
  return nblk < 1 ? 1 : (int)nblk;
}

// dx and the per-block partial column sums part[2][nblk][dim] (dw partials, then db partials)
static int32_t ln_bwd_launch(ah_ptr x, ah_ptr w, ah_ptr grad_out, int32_t grad_dtype, ah_ptr residual_grad, ah_ptr dx, ah_ptr dx_bf16,
                             float *part, int nblk, int64_t rows, int64_t dim, float eps, int32_t stream_dtype = AH_F32) {
  size_t lds = sizeof(float) * 2 * WPB * (size_t)dim;
  float *part_dw = part, *part_db = part + (size_t)nblk * dim;
  const unsigned sa = stream_dtype == AH_BF16 ? 8 : 16;       // bytes of four stream elements
  bool vec = dim % 4 == 0 && dim <= 2048 && x % sa == 0 && aligned16(w) && aligned16(dx) && (grad_out % 8 == 0) && (residual_grad % sa == 0) &&
             (dx_bf16 % 8 == 0) && (grad_dtype == AH_BF16 || aligned16(grad_out));
  if (stream_dtype == AH_BF16)
    AH_ARG(vec && grad_dtype == AH_BF16 && dx_bf16, "ah_layernorm_bwd: a bf16 stream needs bf16 gradients, a bf16 dx and rows of 4 k <= 2048 aligned elements");
  else
    AH_ARG(dx != 0, "ah_layernorm_bwd: null dx");
  if (vec) {
    int nvl = (int)cdiv(dim / 4, 64);
#define LNB_CASE(NV, GT, XT) ah::launch_kernel((k_layernorm_bwd_vec<NV, GT, XT>), dim3(nblk), dim3(TPB), lds, dp<const XT>(x), dp<const float>(w), \
      dp<const GT>(grad_out), dp<const XT>(residual_grad), dp<float>(dx), dp<uint16_t>(dx_bf16), part_dw, part_db, rows, (int)dim, eps)
#define LNB_SWITCH(GT, XT) switch (nvl) { case 1: LNB_CASE(1, GT, XT); break; case 2: LNB_CASE(2, GT, XT); break; case 3: LNB_CASE(3, GT, XT); break; \
      case 4: LNB_CASE(4, GT, XT); break; case 5: case 6: LNB_CASE(6, GT, XT); break; default: LNB_CASE(8, GT, XT); break; }
    if (stream_dtype == AH_BF16) { LNB_SWITCH(uint16_t, uint16_t) }
    else if (grad_dtype == AH_F32) { LNB_SWITCH(float, float) } else { LNB_SWITCH(uint16_t, float) }
#undef LNB_SWITCH
#undef LNB_CASE
  } else if (grad_dtype == AH_F32)
    ah::launch_kernel(k_layernorm_bwd<float>, dim3(nblk), dim3(TPB), lds, dp<const float>(x), dp<const float>(w),
                       dp<const float>(grad_out), dp<const float>(residual_grad), dp<float>(dx), dp<uint16_t>(dx_bf16), part_dw, part_db, rows, (int)dim, eps);
  else
    ah::launch_kernel(k_layernorm_bwd<uint16_t>, dim3(nblk), dim3(TPB), lds, dp<const float>(x), dp<const float>(w),
                       dp<const uint16_t>(grad_out), dp<const float>(residual_grad), dp<float>(dx), dp<uint16_t>(dx_bf16), part_dw, part_db, rows, (int)dim, eps);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_layernorm_bwd(ah_ptr x, ah_ptr w, ah_ptr grad_out, int32_t grad_dtype, ah_ptr residual_grad, ah_ptr dx, ah_ptr dx_bf16,
                         ah_ptr dw, ah_ptr db, int64_t rows, int64_t dim, float eps, int32_t accumulate, int32_t stream_dtype) {
  AH_REQUIRE_READY();
  AH_ARG(grad_dtype == AH_F32 || grad_dtype == AH_BF16, "ah_layernorm_bwd: grad dtype must be f32 or bf16");
  AH_ARG(stream_dtype == AH_F32 || stream_dtype == AH_BF16, "ah_layernorm_bwd: stream dtype must be f32 or bf16");
  if (dim == 0) return AH_OK;
  AH_ARG(dw && db, "ah_layernorm_bwd: null dw/db");
  if (rows == 0) {
    if (!accumulate) { int32_t rc = ah_fill_f32(dw, 0.f, (uint64_t)dim); if (rc) return rc; return ah_fill_f32(db, 0.f, (uint64_t)dim); }
    return AH_OK;
  }
  AH_ARG(x && w && grad_out && (dx || stream_dtype == AH_BF16), "ah_layernorm_bwd: null operand");
  AH_ARG(sizeof(float) * 2 * WPB * (size_t)dim <= 160 * 1024, "ah_layernorm_bwd: dim %lld too large for the LDS column accumulators", (long long)dim);
  const int nblk = ln_bwd_blocks(rows, dim);
  float *part = (float *)scratch(sizeof(float) * 2 * (size_t)nblk * (size_t)dim);
  if (!part) return fail(AH_ERR_OOM, "ah_layernorm_bwd: no scratch");
  int32_t rc = ln_bwd_launch(x, w, grad_out, grad_dtype, residual_grad, dx, dx_bf16, part, nblk, rows, dim, eps, stream_dtype);
  if (rc) return rc;
  ah::launch_kernel(k_colsum_partials, dim3((unsigned)cdiv(dim, 32)), dim3(1024), 0, part, part + (size_t)nblk * dim, nblk, (int)dim,
                     dp<float>(dw), dp<float>(db), accumulate);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int64_t ah_layernorm_bwd_partials_bytes(int64_t rows, int64_t dim) {
  if (rows <= 0 || dim <= 0 || !ready()) return 0;
  return (int64_t)sizeof(float) * 2 * ln_bwd_blocks(rows, dim) * dim;
}

int32_t ah_layernorm_bwd_deferred(ah_ptr x, ah_ptr w, ah_ptr grad_out, int32_t grad_dtype, ah_ptr residual_grad, ah_ptr dx, ah_ptr dx_bf16,
                                  ah_ptr partials, int64_t rows, int64_t dim, float eps, int32_t stream_dtype) {
  AH_REQUIRE_READY();
  AH_ARG(grad_dtype == AH_F32 || grad_dtype == AH_BF16, "ah_layernorm_bwd_deferred: grad dtype must be f32 or bf16");
  AH_ARG(stream_dtype == AH_F32 || stream_dtype == AH_BF16, "ah_layernorm_bwd_deferred: stream dtype must be f32 or bf16");
  AH_ARG(rows > 0 && dim > 0, "ah_layernorm_bwd_deferred: empty input [%lld, %lld]", (long long)rows, (long long)dim);
  AH_ARG(x && w && grad_out && (dx || stream_dtype == AH_BF16) && partials, "ah_layernorm_bwd_deferred: null operand");
  AH_ARG(partials % 4 == 0, "ah_layernorm_bwd_deferred: partials must be aligned to 4 bytes");
  AH_ARG(sizeof(float) * 2 * WPB * (size_t)dim <= 160 * 1024, "ah_layernorm_bwd_deferred: dim %lld too large for the LDS column accumulators", (long long)dim);
  return ln_bwd_launch(x, w, grad_out, grad_dtype, residual_grad, dx, dx_bf16, dp<float>(partials), ln_bwd_blocks(rows, dim), rows, dim, eps, stream_dtype);
}

int32_t ah_layernorm_colsums(const AhColsumJob *jobs, int32_t count) {
  AH_REQUIRE_READY();
  AH_ARG(count >= 0 && (count == 0 || jobs != nullptr), "ah_layernorm_colsums: bad job list (count %d)", count);
  for (int32_t first = 0; first < count; first += COLSUM_JOBS) {
    ColsumJobs tab;
    const int n = count - first < COLSUM_JOBS ? count - first : COLSUM_JOBS;
    int64_t max_dim = 0;
    for (int i = 0; i < n; i++) {
      const AhColsumJob &q = jobs[first + i];
      AH_ARG(q.rows > 0 && q.dim > 0 && q.dim < (1ll << 31), "ah_layernorm_colsums: job %d: empty input [%lld, %lld]", first + i, (long long)q.rows, (long long)q.dim);
      AH_ARG(q.partials && q.dw && q.db, "ah_layernorm_colsums: job %d: null operand", first + i);
      tab.j[i] = ColsumJob{dp<const float>(q.partials), dp<float>(q.dw), dp<float>(q.db), ln_bwd_blocks(q.rows, q.dim), (int)q.dim, q.accumulate, 0};
      if (q.dim > max_dim) max_dim = q.dim;
    }
    ah::launch_kernel(k_colsum_partials_batched, dim3((unsigned)cdiv(max_dim, 32), (unsigned)n), dim3(1024), 0, tab);
    AH_LAUNCH_CHECK();
  }
  return AH_OK;
}

int32_t ah_cross_entropy(ah_ptr logits, int32_t dtype, ah_ptr targets, ah_ptr loss_out, ah_ptr lse_out, int64_t n, int64_t c) {
  AH_REQUIRE_READY();
  AH_ARG(dtype == AH_F32 || dtype == AH_BF16, "ah_cross_entropy: logits dtype must be f32 or bf16");
  AH_ARG(loss_out != 0, "ah_cross_entropy: null loss_out");
  AH_ARG(n >= 0 && c >= 0, "ah_cross_entropy: negative extent [%lld, %lld]", (long long)n, (long long)c);
  if (n == 0 || c == 0) return ah_fill_f32(loss_out, NAN, 1);      // a mean over no rows (0 / 0), or of entries that do not exist (cpu_ref.ts:543-563)
  AH_ARG(logits && targets, "ah_cross_entropy: null operand");
  AH_ARG(n < (int64_t(1) << 31), "ah_cross_entropy: too many rows");
  float *rows = (float *)scratch(sizeof(float) * (size_t)n);
  if (!rows) return fail(AH_ERR_OOM, "ah_cross_entropy: no scratch");
  if (dtype == AH_F32)
    ah::launch_kernel(k_ce_fwd<float>, dim3((unsigned)n), dim3(TPB), 0, dp<const float>(logits), dp<const int32_t>(targets), rows, dp<float>(lse_out), c);
  else
    ah::launch_kernel(k_ce_fwd<uint16_t>, dim3((unsigned)n), dim3(CE_TPB), 0, dp<const uint16_t>(logits), dp<const int32_t>(targets), rows, dp<float>(lse_out), c);
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_mean_rows, dim3(1), dim3(TPB), 0, rows, n, dp<float>(loss_out));
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t ah_cross_entropy_bwd(ah_ptr logits, int32_t dtype, ah_ptr targets, ah_ptr lse, ah_ptr g_scalar, float g_mul, ah_ptr dlogits,
                             int64_t n, int64_t c) {
  AH_REQUIRE_READY();
  AH_ARG(dtype == AH_F32 || dtype == AH_BF16, "ah_cross_entropy_bwd: dtype must be f32 or bf16");
  if (n == 0 || c == 0) return AH_OK;
  AH_ARG(logits && targets && lse && dlogits, "ah_cross_entropy_bwd: null operand");
  AH_ARG(n <= 65535 * 1024ll, "ah_cross_entropy_bwd: too many rows");
  unsigned gx = (unsigned)cdiv(c, TPB * 8);
  if (gx < 1) gx = 1;
  // gridDim.y is limited to 65535: fold rows beyond that by launching in row chunks
  for (int64_t r0 = 0; r0 < n; r0 += 65535) {
    int64_t nr = n - r0 < 65535 ? n - r0 : 65535;
    size_t esz = dtype == AH_F32 ? 4 : 2;
    ah_ptr lg = logits + (uint64_t)(r0 * c) * esz, dl = dlogits + (uint64_t)(r0 * c) * esz;
    if (dtype == AH_F32)
      ah::launch_kernel(k_ce_bwd<float>, dim3(gx, (unsigned)nr), dim3(TPB), 0, dp<const float>(lg),
                         dp<const int32_t>(targets) + r0, dp<const float>(lse) + r0, dp<const float>(g_scalar), g_mul, dp<float>(dl), n, c);
    else
      ah::launch_kernel(k_ce_bwd<uint16_t>, dim3(gx, (unsigned)nr), dim3(TPB), 0, dp<const uint16_t>(lg),
                         dp<const int32_t>(targets) + r0, dp<const float>(lse) + r0, dp<const float>(g_scalar), g_mul, dp<uint16_t>(dl), n, c);
    AH_LAUNCH_CHECK();
  }
  return AH_OK;
}

int32_t ah_cross_entropy_fwd_bwd(ah_ptr logits, int32_t dtype, ah_ptr targets, ah_ptr loss_out, ah_ptr lse_out, ah_ptr g_scalar, float g_mul,
                                 ah_ptr dlogits, int64_t n, int64_t c) {
  AH_REQUIRE_READY();
  AH_ARG(dtype == AH_F32 || dtype == AH_BF16, "ah_cross_entropy_fwd_bwd: logits dtype must be f32 or bf16");
  AH_ARG(loss_out != 0, "ah_cross_entropy_fwd_bwd: null loss_out");
  AH_ARG(n >= 0 && c >= 0, "ah_cross_entropy_fwd_bwd: negative extent [%lld, %lld]", (long long)n, (long long)c);
  if (n == 0 || c == 0) return ah_fill_f32(loss_out, NAN, 1);      // as ah_cross_entropy; there is no gradient to write
  AH_ARG(logits && targets && lse_out && dlogits, "ah_cross_entropy_fwd_bwd: null operand");
  AH_ARG(n < (int64_t(1) << 31), "ah_cross_entropy_fwd_bwd: too many rows");
  const bool one_pass = dtype == AH_BF16 && (c & 7) == 0 && (c >> 3) <= (int64_t)CE_CHUNKS * CE_TPB && ((logits | dlogits) & 15u) == 0;
  if (!one_pass) {                // rows that do not fit the registers of a block, f32 logits, odd alignments: the two kernels
    int32_t rc = ah_cross_entropy(logits, dtype, targets, loss_out, lse_out, n, c);
    return rc ? rc : ah_cross_entropy_bwd(logits, dtype, targets, lse_out, g_scalar, g_mul, dlogits, n, c);
  }
  float *rows = (float *)scratch(sizeof(float) * (size_t)n);
  if (!rows) return fail(AH_ERR_OOM, "ah_cross_entropy_fwd_bwd: no scratch");
  ah::launch_kernel(k_ce_fwd_bwd, dim3((unsigned)n), dim3(CE_TPB), 0, dp<const uint16_t>(logits), dp<const int32_t>(targets), rows,
                     dp<float>(lse_out), dp<const float>(g_scalar), g_mul, dp<uint16_t>(dlogits), n, c);
  AH_LAUNCH_CHECK();
  ah::launch_kernel(k_mean_rows, dim3(1), dim3(TPB), 0, rows, n, dp<float>(loss_out));
  AH_LAUNCH_CHECK();
  return AH_OK;
}

}  // extern "C"
