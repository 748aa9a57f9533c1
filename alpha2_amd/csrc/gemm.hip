// GEMM on the gfx950 matrix cores.
//   fp32 (parity mode): v_mfma_f32_32x32x2_f32, 128x128x16 LDS tiles, 4 waves (2x2) of 64x64.
//   bf16 (fast mode)  : v_mfma_f32_32x32x16_bf16, BMxBNx32 LDS tiles double-buffered, fp32 accumulate.
// All three operand layouts the training step needs are handled (NN: dX = G W, NT: Y = X W^T,
// TN: dW = G^T X).  Epilogues fuse GELU (+ saved pre-activation), the residual add, gradient
// accumulation and the GELU derivative.
#include "gemm_common.h"
#include <cstdarg>
#include <vector>
#include <cstdio>

using namespace ah;

namespace {

// ================================================================ fp32 MFMA kernel
// LDS tiles are k-major: As[k][m], Bs[k][n]; a lane of the 32x32x2 MFMA reads As[2*kk + lane/32][m0 + lane%32].
constexpr int F_BM = 128, F_BN = 128, F_BK = 16, F_PAD = 4;

// Load a [rows x F_BK] tile of an operand into registers (2 float4 per thread).
//   KCONTIG = true : memory is [row][k] (k contiguous), thread -> (row = t/4 + 64*i, kq = t%4)
//   KCONTIG = false: memory is [k][row] (row contiguous), thread -> (k = t/32 + 8*i, r4 = t%32)
template <bool KCONTIG>
__device__ __forceinline__ void f32_load_tile(const float *__restrict__ base, int64_t ld, int row0, int k0, int rows, int K,
                                              bool vec, float4 (&v)[2]) {
  int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    int r, k;
    if (KCONTIG) { r = row0 + (t >> 2) + 64 * i; k = k0 + (t & 3) * 4; }
    else { k = k0 + (t >> 5) + 8 * i; r = row0 + (t & 31) * 4; }
    float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
    if (KCONTIG) {
      if (r < rows) {
        const float *p = base + (int64_t)r * ld + k;
        if (vec && k + 3 < K) x = *reinterpret_cast<const float4 *>(p);
        else { if (k < K) x.x = p[0]; if (k + 1 < K) x.y = p[1]; if (k + 2 < K) x.z = p[2]; if (k + 3 < K) x.w = p[3]; }
      }
    } else {
      if (k < K) {
        const float *p = base + (int64_t)k * ld + r;
        if (vec && r + 3 < rows) x = *reinterpret_cast<const float4 *>(p);
        else { if (r < rows) x.x = p[0]; if (r + 1 < rows) x.y = p[1]; if (r + 2 < rows) x.z = p[2]; if (r + 3 < rows) x.w = p[3]; }
      }
    }
    v[i] = x;
  }
}
template <bool KCONTIG>
__device__ __forceinline__ void f32_store_tile(float (*s)[F_BM + F_PAD], const float4 (&v)[2]) {
  int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    if (KCONTIG) {
      int r = (t >> 2) + 64 * i, k = (t & 3) * 4;
      s[k + 0][r] = v[i].x; s[k + 1][r] = v[i].y; s[k + 2][r] = v[i].z; s[k + 3][r] = v[i].w;
    } else {
      int k = (t >> 5) + 8 * i, r = (t & 31) * 4;
      *reinterpret_cast<float4 *>(&s[k][r]) = v[i];
    }
  }
}

template <int LAYOUT, int EPI, class OUT>
__global__ __launch_bounds__(256) void k_gemm_f32(GemmArgs g, int vec_a, int vec_b, int vec_c) {
  __shared__ __attribute__((aligned(16))) float As[2][F_BK][F_BM + F_PAD];
  __shared__ __attribute__((aligned(16))) float Bs[2][F_BK][F_BN + F_PAD];
  constexpr bool A_KC = (LAYOUT != AH_GEMM_TN);     // A is [M][K] except for TN ([K][M])
  constexpr bool B_KC = (LAYOUT == AH_GEMM_NT);     // B is [N][K] only for NT
  int bz = blockIdx.z;
  const float *A = (const float *)g.a + (int64_t)bz * g.sa;
  const float *B = (const float *)g.b + (int64_t)bz * g.sb;
  int64_t cbase = (int64_t)bz * g.sc;
  int m0 = blockIdx.y * F_BM, n0 = blockIdx.x * F_BN;
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  int lr = lane & 31, lk = lane >> 5;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

  float4 ra[2], rb[2];
  int nt = (g.K + F_BK - 1) / F_BK;
  f32_load_tile<A_KC>(A, g.lda, m0, 0, g.M, g.K, vec_a, ra);
  f32_load_tile<B_KC>(B, g.ldb, n0, 0, g.N, g.K, vec_b, rb);
  f32_store_tile<A_KC>(As[0], ra);
  f32_store_tile<B_KC>(Bs[0], rb);
  __syncthreads();
  for (int t = 0; t < nt; t++) {
    int cur = t & 1;
    if (t + 1 < nt) {
      f32_load_tile<A_KC>(A, g.lda, m0, (t + 1) * F_BK, g.M, g.K, vec_a, ra);
      f32_load_tile<B_KC>(B, g.ldb, n0, (t + 1) * F_BK, g.N, g.K, vec_b, rb);
    }
#pragma unroll
    for (int kk = 0; kk < F_BK / 2; kk++) {
      float a0 = As[cur][2 * kk + lk][wm + lr], a1 = As[cur][2 * kk + lk][wm + 32 + lr];
      float b0 = Bs[cur][2 * kk + lk][wn + lr], b1 = Bs[cur][2 * kk + lk][wn + 32 + lr];
      // operands swapped: the accumulator holds C^T tiles (rows = n, columns = m)
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(b0, a0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(b1, a0, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(b0, a1, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(b1, a1, acc[1][1], 0, 0, 0);
    }
    if (t + 1 < nt) {
      f32_store_tile<A_KC>(As[cur ^ 1], ra);
      f32_store_tile<B_KC>(Bs[cur ^ 1], rb);
    }
    __syncthreads();
  }
  // accumulator element e of a (transposed) 32x32 tile: n = 8*(e/4) + 4*(lane/32) + e%4, m = lane%32
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        int row = m0 + wm + 32 * i + lr;
        int col = n0 + wn + 32 * j + 8 * q + 4 * lk;
        epilogue4<EPI, OUT>(g, cbase, row, col, acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3], vec_c);
      }
}

// ================================================================ bf16 MFMA kernel (NT operands)
// Both operands are [rows][K] with K contiguous.  LDS tiles are [rows][BK] with an 80-byte row pitch
// (32 bf16 + 8 pad) so the 16-byte fragment reads of 8 consecutive rows hit 8 distinct bank groups.
// A lane of v_mfma_f32_32x32x16_bf16 supplies, for row lane%32, the 8 k-values 8*(lane/32)..+7.
constexpr int H_BK = 32, H_PITCH = 40;   // in bf16 elements

template <int ROWS>
__device__ __forceinline__ void h_load_tile(const uint16_t *__restrict__ base, int64_t ld, int row0, int k0, int rows, int K,
                                            uint4 (&v)[ROWS / 64]) {
  // ROWS x 32 bf16 = ROWS*4 chunks of 16 bytes; 256 threads -> ROWS/64 chunks each.
  int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < ROWS / 64; i++) {
    int r = row0 + (t >> 2) + 64 * i, k = k0 + (t & 3) * 8;
    uint4 x = make_uint4(0, 0, 0, 0);
    if (r < rows && k < K) x = *reinterpret_cast<const uint4 *>(base + (int64_t)r * ld + k);   // K % 8 == 0 is required
    v[i] = x;
  }
}
template <int ROWS>
__device__ __forceinline__ void h_store_tile(uint16_t *s, const uint4 (&v)[ROWS / 64]) {
  int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < ROWS / 64; i++) {
    int r = (t >> 2) + 64 * i, k = (t & 3) * 8;
    *reinterpret_cast<uint4 *>(s + r * H_PITCH + k) = v[i];
  }
}

// BM x BN block tile, 4 waves as WGM x WGN grid; each wave owns (BM/WGM) x (BN/WGN).
template <int BM, int BN, int WGM, int WGN, int EPI, class OUT>
__global__ __launch_bounds__(256) void k_gemm_bf16_nt(GemmArgs g, int vec_c) {
  constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t *As = smem;                                   // [2][BM][H_PITCH]
  uint16_t *Bs = smem + 2 * BM * H_PITCH;                // [2][BN][H_PITCH]
  int bz = blockIdx.z;
  const uint16_t *A = (const uint16_t *)g.a + (int64_t)bz * g.sa;
  const uint16_t *B = (const uint16_t *)g.b + (int64_t)bz * g.sb;
  int64_t cbase = (int64_t)bz * g.sc;
  // Tile order: consecutive blocks walk down M inside one N column so the B (weight) tile stays hot in L2.
  int tiles_m = (g.M + BM - 1) / BM;
  int bid = blockIdx.x;
  int m0 = (bid % tiles_m) * BM, n0 = (bid / tiles_m) * BN;
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int wm = (wave / WGN) * WM, wn = (wave % WGN) * WN;
  int lr = lane & 31, lk = lane >> 5;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

  uint4 ra[BM / 64], rb[BN / 64];
  int nt = (g.K + H_BK - 1) / H_BK;
  h_load_tile<BM>(A, g.lda, m0, 0, g.M, g.K, ra);
  h_load_tile<BN>(B, g.ldb, n0, 0, g.N, g.K, rb);
  h_store_tile<BM>(As, ra);
  h_store_tile<BN>(Bs, rb);
  __syncthreads();
  for (int t = 0; t < nt; t++) {
    int cur = t & 1;
    if (t + 1 < nt) {
      h_load_tile<BM>(A, g.lda, m0, (t + 1) * H_BK, g.M, g.K, ra);
      h_load_tile<BN>(B, g.ldb, n0, (t + 1) * H_BK, g.N, g.K, rb);
    }
    const uint16_t *as = As + cur * BM * H_PITCH, *bs = Bs + cur * BN * H_PITCH;
#pragma unroll
    for (int kk = 0; kk < H_BK / 16; kk++) {
      bf16x8 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) fa[i] = *reinterpret_cast<const bf16x8 *>(as + (wm + 32 * i + lr) * H_PITCH + kk * 16 + lk * 8);
#pragma unroll
      for (int j = 0; j < TN; j++) fb[j] = *reinterpret_cast<const bf16x8 *>(bs + (wn + 32 * j + lr) * H_PITCH + kk * 16 + lk * 8);
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);   // C^T tile
    }
    if (t + 1 < nt) {
      h_store_tile<BM>(As + (cur ^ 1) * BM * H_PITCH, ra);
      h_store_tile<BN>(Bs + (cur ^ 1) * BN * H_PITCH, rb);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        int row = m0 + wm + 32 * i + lr;
        int col = n0 + wn + 32 * j + 8 * q + 4 * lk;
        epilogue4<EPI, OUT>(g, cbase, row, col, acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3], vec_c);
      }
}

// 16-bit [R][C] -> [C][R] through a 64x64 LDS tile (used to bring NN / TN operands into NT form)
__global__ void k_transpose_u16(const uint16_t *__restrict__ in, int64_t ld_in, uint16_t *__restrict__ out, int64_t ld_out, int R, int C) {
  __shared__ uint16_t tile[64][66];
  int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  for (int j = threadIdx.y; j < 64; j += blockDim.y) {
    int r = r0 + j, c = c0 + threadIdx.x;
    tile[j][threadIdx.x] = (r < R && c < C) ? in[(int64_t)r * ld_in + c] : (uint16_t)0;
  }
  __syncthreads();
  for (int j = threadIdx.y; j < 64; j += blockDim.y) {
    int c = c0 + j, r = r0 + threadIdx.x;
    if (r < R && c < C) out[(int64_t)c * ld_out + r] = tile[threadIdx.x][j];
  }
}

template <int BM, int BN, int WGM, int WGN, int EPI, class OUT>
int32_t launch_bf16_nt_t(const GemmArgs &ga, int batch, int vec_c) {
  size_t lds = sizeof(uint16_t) * 2 * (size_t)(BM + BN) * H_PITCH;
  int64_t tiles = cdiv(ga.M, BM) * cdiv(ga.N, BN);
  dim3 grid((unsigned)tiles, 1, (unsigned)batch);
  auto kfn = k_gemm_bf16_nt<BM, BN, WGM, WGN, EPI, OUT>;
  if (lds > 64 * 1024) {
    static bool raised = false;      // per instantiation: the attribute only needs setting once
    if (!raised) { AH_HIP(hipFuncSetAttribute((const void *)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); raised = true; }
  }
  note_gemm_kernel("k_gemm_bf16_nt<%d, %d, %d, %d, %d, %s>", BM, BN, WGM, WGN, EPI, sizeof(OUT) == 4 ? "float" : "unsigned short");
  note_gemm_split(1);
  ah::launch_kernel(kfn, grid, dim3(256), lds, ga, vec_c);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
int32_t run_bf16_nt(const GemmArgs &ga, int batch, int out_dtype, int vec_c) {
  // Fallback kernel for shapes the direct kernel does not take (K % 64 != 0, unaligned C): one tile size.
  bool f32 = out_dtype == AH_F32;
  switch (ga.epi) {
    case AH_EPI_NONE: return f32 ? launch_bf16_nt_t<128, 128, 2, 2, AH_EPI_NONE, float>(ga, batch, vec_c)
                                 : launch_bf16_nt_t<128, 128, 2, 2, AH_EPI_NONE, uint16_t>(ga, batch, vec_c);
    case AH_EPI_ACCUM: return launch_bf16_nt_t<128, 128, 2, 2, AH_EPI_ACCUM, float>(ga, batch, vec_c);
    case AH_EPI_RESIDUAL: return f32 ? launch_bf16_nt_t<128, 128, 2, 2, AH_EPI_RESIDUAL, float>(ga, batch, vec_c)
                                     : launch_bf16_nt_t<128, 128, 2, 2, AH_EPI_RESIDUAL, uint16_t>(ga, batch, vec_c);
    case AH_EPI_GELU: return launch_bf16_nt_t<128, 128, 2, 2, AH_EPI_GELU, uint16_t>(ga, batch, vec_c);
    case AH_EPI_GELU_GRAD: return launch_bf16_nt_t<128, 128, 2, 2, AH_EPI_GELU_GRAD, uint16_t>(ga, batch, vec_c);
    case AH_EPI_MUL_AUX: return launch_bf16_nt_t<128, 128, 2, 2, AH_EPI_MUL_AUX, uint16_t>(ga, batch, vec_c);
    default: return launch_bf16_nt_t<128, 128, 2, 2, AH_EPI_GELU_BWD, uint16_t>(ga, batch, vec_c);
  }
}

template <int LAYOUT, int EPI, class OUT>
int32_t launch_f32_t(const GemmArgs &ga, int batch, int vec_a, int vec_b, int vec_c) {
  dim3 grid((unsigned)cdiv(ga.N, F_BN), (unsigned)cdiv(ga.M, F_BM), (unsigned)batch);
  note_gemm_kernel("k_gemm_f32<%d, %d, %s>", LAYOUT, EPI, sizeof(OUT) == 4 ? "float" : "unsigned short");
  note_gemm_split(1);
  ah::launch_kernel((k_gemm_f32<LAYOUT, EPI, OUT>), grid, dim3(256), 0, ga, vec_a, vec_b, vec_c);
  AH_LAUNCH_CHECK();
  return AH_OK;
}
template <int LAYOUT>
int32_t launch_f32(const GemmArgs &ga, int batch, int out_dtype, int vec_a, int vec_b, int vec_c) {
  switch (ga.epi) {
    case AH_EPI_NONE: return out_dtype == AH_F32 ? launch_f32_t<LAYOUT, AH_EPI_NONE, float>(ga, batch, vec_a, vec_b, vec_c)
                                                 : launch_f32_t<LAYOUT, AH_EPI_NONE, uint16_t>(ga, batch, vec_a, vec_b, vec_c);
    case AH_EPI_ACCUM: return launch_f32_t<LAYOUT, AH_EPI_ACCUM, float>(ga, batch, vec_a, vec_b, vec_c);
    case AH_EPI_GELU: return launch_f32_t<LAYOUT, AH_EPI_GELU, float>(ga, batch, vec_a, vec_b, vec_c);
    case AH_EPI_RESIDUAL: return launch_f32_t<LAYOUT, AH_EPI_RESIDUAL, float>(ga, batch, vec_a, vec_b, vec_c);
    case AH_EPI_GELU_GRAD: return launch_f32_t<LAYOUT, AH_EPI_GELU_GRAD, float>(ga, batch, vec_a, vec_b, vec_c);
    case AH_EPI_MUL_AUX: return launch_f32_t<LAYOUT, AH_EPI_MUL_AUX, float>(ga, batch, vec_a, vec_b, vec_c);
    default: return launch_f32_t<LAYOUT, AH_EPI_GELU_BWD, float>(ga, batch, vec_a, vec_b, vec_c);
  }
}

}  // namespace

namespace ah {
static char g_last_kernel[96] = "";
static int g_last_split = 1;
void note_gemm_kernel(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_kernel, sizeof(g_last_kernel), fmt, ap);
  va_end(ap);
}
void note_gemm_split(int nsplit) { g_last_split = nsplit; }
}  // namespace ah

namespace {
// A plan holds the device table of its problems.  Where it pays (see split_tail), the problems at the end of the launch
// are each two entries, one per half of k: the first writes (or accumulates into) C, the second the plan's workspace, which
// k_grouped_join then adds to C.
struct JoinPart { float *c; float *ws; int M, N; int64_t ldc; };
struct GroupPlan {
  ah_ptr table; int count, blocks, layout, out_dtype; bool live;
  ah_ptr parts, ws; int nparts;
  ah_ptr sumsq;                        // 4 floats per block of the launch, then JOIN_BLOCKS per k-split problem (ah_gemm_grouped_run_sumsq)
  int ndescs; int64_t ws_bytes;        // what ah_gemm_grouped_update checks a new descriptor list against:
  std::vector<int64_t> shape;          // m, n, k, lda, ldb, ldc of every problem
};
std::vector<int64_t> group_shape(const AhGemm *descs, int count) {
  std::vector<int64_t> v;
  for (int i = 0; i < count; i++) { const AhGemm &q = descs[i]; v.insert(v.end(), {q.m, q.n, q.k, q.lda, q.ldb, q.ldc}); }
  return v;
}
std::vector<GroupPlan> g_plans;      // plan id = g_plan_base + index + 1
uint64_t g_plan_base = 0;            // ids handed out in earlier lives of the library (before an ah_shutdown): never valid again
GroupPlan *find_plan(uint64_t id) {
  if (id <= g_plan_base || id - g_plan_base > g_plans.size()) return nullptr;
  GroupPlan &p = g_plans[id - g_plan_base - 1];
  return p.live ? &p : nullptr;
}

// C += ws, ws = 0 for every k-split problem of a grouped launch: block (x, y) walks the float4s of part y.  The workspace
// is left all zero, so the second halves of an ACCUMULATING run (whose epilogue adds to what it finds) store into it just
// as those of a plain run do.
constexpr int JOIN_BLOCKS = 128;     // blocks per k-split problem
// With SUMSQ, block (x, y) also leaves the sum of the squares of the sums it stored in sumsq[JOIN_BLOCKS y + x].
template <bool SUMSQ>
__global__ __launch_bounds__(256) void k_grouped_join(const JoinPart *__restrict__ parts, float *__restrict__ sumsq) {
  const JoinPart p = parts[blockIdx.y];
  const int nq = p.N >> 2;
  const int64_t total = (int64_t)p.M * nq;
  float ss = 0.f;
  for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < total; q += (int64_t)gridDim.x * 256) {
    const int64_t row = q / nq;
    const int col = (int)(q - row * nq) * 4;
    float4 *dst = (float4 *)(p.c + row * p.ldc + col), *src = (float4 *)(p.ws + row * p.N + col);
    const float4 w = *src;
    float4 v = *dst;
    v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
    *dst = v;
    *src = make_float4(0.f, 0.f, 0.f, 0.f);
    if (SUMSQ) ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
  }
  if (SUMSQ) {
    __shared__ float part[4];
    ss = ah::wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    if (threadIdx.x == 0) sumsq[blockIdx.y * JOIN_BLOCKS + blockIdx.x] = (part[0] + part[1]) + (part[2] + part[3]);
  }
}

// *inout += the sum of the n partial sums (n a multiple of 4), added up in f64 in an order that depends on n only.
__global__ __launch_bounds__(256) void k_grouped_sumsq_final(const float *__restrict__ partial, int n, float *__restrict__ inout) {
  __shared__ double sh[4];
  const float4 *p4 = reinterpret_cast<const float4 *>(partial);
  const int n4 = n >> 2;
  double t = 0.0;
#pragma unroll 8
  for (int i = threadIdx.x; i < n4; i += 256) {      // (unrolled: the loads of a thread are in flight together)
    const float4 v = p4[i];
    t += ((double)v.x + (double)v.y) + ((double)v.z + (double)v.w);
  }
  t = ah::wave_sum_d(t);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = t;
  __syncthreads();
  if (threadIdx.x == 0) *inout = (float)((double)*inout + ((sh[0] + sh[1]) + (sh[2] + sh[3])));
}

constexpr int GROUP_ROUND = 256;     // tiles that run at a time: one per CU

// The launch runs its 256 x 256 tiles one per CU, in rounds of 256; all tiles of a weight-gradient group take the same
// time, so a last round of t < 256 tiles costs a whole round.  Cutting the problems that make up that round in two along
// k turns it into 2 t half-length tiles, which still run at once when t <= 128: the round then costs half.  Chooses whole
// problems from the end of the list whose tiles add up to between t and 128 and returns their indices (ascending), or
// nothing when no such choice exists.
std::vector<int> split_tail(const AhGemm *descs, int count, int64_t blocks) {
  std::vector<int> chosen;
  const int64_t tail = blocks % GROUP_ROUND;
  if (descs[0].out_dtype != AH_F32 || tail == 0 || tail > GROUP_ROUND / 2) return chosen;
  int64_t sum = 0;
  for (int i = count - 1; i >= 0 && sum < tail; i--) {
    const AhGemm &q = descs[i];
    const int64_t t = cdiv(q.m, 256) * cdiv(q.n, 256);
    if (q.k % 128 != 0 || q.n % 4 != 0 || sum + t > GROUP_ROUND / 2) continue;
    chosen.insert(chosen.begin(), i);
    sum += t;
  }
  if (sum < tail) chosen.clear();
  return chosen;
}
}  // namespace

namespace ah {
// ah_shutdown frees every device allocation, the plans' tables and workspaces among them: their ids must stop working.
void gemm_plans_forget() {
  g_plan_base += g_plans.size();
  g_plans.clear();
}
}  // namespace ah

extern "C" {

// Validates a descriptor list and builds the launch's tables from it: `tab` (one entry per problem, the problems of a short last
// round as two entries each at the end) and `parts` (what k_grouped_join adds to what).  The second halves write consecutive
// pieces of a workspace that starts at ws_base (0 while only its size, *ws_bytes, is wanted).
static int32_t grouped_tables(const char *who, const AhGemm *descs, int32_t count, ah_ptr ws_base, std::vector<GemmGroupEntry> &tab,
                              std::vector<JoinPart> &parts, int64_t *blocks_out, int64_t *ws_bytes) {
  AH_ARG(descs != nullptr && count > 0 && count <= 4096, "%s: bad descriptor list (count %d)", who, count);
  tab.assign((size_t)count, GemmGroupEntry{});
  parts.clear();
  int64_t blocks = 0;
  const int layout = descs[0].layout, out_dtype = descs[0].out_dtype;
  AH_ARG(layout >= AH_GEMM_NN && layout <= AH_GEMM_TN, "%s: bad layout %d", who, layout);
  AH_ARG(out_dtype == AH_F32 || out_dtype == AH_BF16, "%s: output must be f32 or bf16", who);
  const bool akm = layout == AH_GEMM_TN, bkm = layout != AH_GEMM_NT;
  const int osz = out_dtype == AH_F32 ? 4 : 2;
  for (int i = 0; i < count; i++) {
    const AhGemm &q = descs[i];
    if (q.layout != layout || q.out_dtype != out_dtype || q.in_dtype != AH_BF16 || q.batch != 1 ||
        (q.epilogue != AH_EPI_NONE && q.epilogue != AH_EPI_ACCUM))
      return fail(AH_ERR_UNSUPPORTED, "%s: problem %d: a group shares one layout and output type, takes bf16 operands, "
                                      "batch 1 and the NONE / ACCUM epilogues", who, i);
    AH_ARG(q.m > 0 && q.n > 0 && q.k >= 64 && q.k % 64 == 0 && q.m < (1ll << 31) && q.n < (1ll << 31) && q.k < (1ll << 31),
           "%s: problem %d: extents m=%lld n=%lld k=%lld (k must be a positive multiple of 64)", who, i, (long long)q.m,
           (long long)q.n, (long long)q.k);
    AH_ARG(q.a != 0 && q.b != 0 && q.c != 0, "%s: problem %d: null operand", who, i);
    int64_t a_cols = akm ? q.m : q.k, b_cols = bkm ? q.n : q.k;
    AH_ARG(q.lda >= a_cols && q.ldb >= b_cols && q.ldc >= q.n, "matmul shape mismatch: problem %d: lda/ldb/ldc too small", i);
    bool ok = aligned16(q.a) && aligned16(q.b) && q.lda % 8 == 0 && q.ldb % 8 == 0 && (!akm || q.m % 8 == 0) && (!bkm || q.n % 8 == 0) &&
              (q.c % (4 * osz)) == 0 && q.ldc % 4 == 0;
    AH_ARG(ok, "%s: problem %d: operands need 16-byte aligned rows and a vector-aligned C", who, i);
    int64_t a_span = (akm ? (int64_t)64 : q.m) * q.lda * 2, b_span = (bkm ? (int64_t)64 : q.n) * q.ldb * 2;
    AH_ARG(a_span < (1ll << 32) && b_span < (1ll << 32), "%s: problem %d: operand spans more than 4 GiB", who, i);
    AH_ARG(q.ldc < (1 << 22), "%s: problem %d: ldc %lld too large (128 rows of C must span less than 2 GiB)", who, i, (long long)q.ldc);
    GemmGroupEntry &e = tab[(size_t)i];
    e.a = dp<const void>(q.a); e.b = dp<const void>(q.b); e.c = dp<void>(q.c);
    e.M = (int)q.m; e.N = (int)q.n; e.K = (int)q.k; e.tile_start = (int)blocks;
    e.lda = q.lda; e.ldb = q.ldb; e.ldc = q.ldc;
    blocks += cdiv(q.m, 256) * cdiv(q.n, 256);
    AH_ARG(blocks < (1ll << 31), "%s: too many tiles", who);
  }
  // the problems that make up a short last round are cut in two along k: they move to the end of the table as pairs of
  // entries, the second of which writes the workspace
  const std::vector<int> chosen = split_tail(descs, count, blocks);
  *ws_bytes = 0;
  if (!chosen.empty()) {
    for (int i : chosen) *ws_bytes += descs[i].m * descs[i].n * 4;
    std::vector<GemmGroupEntry> cut_tab;
    std::vector<bool> cut((size_t)count, false);
    for (int i : chosen) cut[(size_t)i] = true;
    int64_t nblocks = 0;
    auto push = [&](GemmGroupEntry e) {
      e.tile_start = (int)nblocks;
      nblocks += cdiv(e.M, 256) * cdiv(e.N, 256);
      cut_tab.push_back(e);
    };
    for (int i = 0; i < count; i++)
      if (!cut[(size_t)i]) push(tab[(size_t)i]);
    char *ws = dp<char>(ws_base);
    for (int i : chosen) {
      GemmGroupEntry lo = tab[(size_t)i], hi = lo;
      lo.K = hi.K = lo.K / 2;
      lo.partial = hi.partial = 1;
      hi.a = (const char *)lo.a + (akm ? (int64_t)lo.K * lo.lda : (int64_t)lo.K) * 2;
      hi.b = (const char *)lo.b + (bkm ? (int64_t)lo.K * lo.ldb : (int64_t)lo.K) * 2;
      hi.c = ws;
      hi.ldc = lo.N;
      parts.push_back(JoinPart{(float *)lo.c, (float *)ws, lo.M, lo.N, lo.ldc});
      ws += (int64_t)lo.M * lo.N * 4;
      push(lo);
      push(hi);
    }
    tab.swap(cut_tab);
    blocks = nblocks;
  }
  *blocks_out = blocks;
  return AH_OK;
}

int32_t ah_gemm_grouped_plan(const AhGemm *descs, int32_t count, uint64_t *plan_out) {
  AH_REQUIRE_READY();
  AH_ARG(plan_out != nullptr, "ah_gemm_grouped_plan: null plan_out");
  std::vector<GemmGroupEntry> tab;
  std::vector<JoinPart> parts;
  int64_t blocks = 0, ws_bytes = 0;
  int32_t rc = grouped_tables("ah_gemm_grouped_plan", descs, count, 0, tab, parts, &blocks, &ws_bytes);      // sizes first
  if (rc) return rc;
  GroupPlan plan{0, (int)tab.size(), (int)blocks, descs[0].layout, descs[0].out_dtype, true, 0, 0, (int)parts.size(), 0, count, ws_bytes,
                 group_shape(descs, count)};
  if (ws_bytes > 0) {
    rc = ah_alloc((size_t)ws_bytes, &plan.ws);
    if (rc) return rc;
    rc = ah_fill_f32(plan.ws, 0.f, (uint64_t)(ws_bytes / 4));           // the workspace is all zero between runs (see k_grouped_join)
    if (rc == AH_OK) rc = grouped_tables("ah_gemm_grouped_plan", descs, count, plan.ws, tab, parts, &blocks, &ws_bytes);
    if (rc == AH_OK) rc = ah_alloc(parts.size() * sizeof(JoinPart), &plan.parts);
    if (rc == AH_OK) rc = ah_upload(plan.parts, parts.data(), parts.size() * sizeof(JoinPart));
  }
  if (rc == AH_OK) rc = ah_alloc(tab.size() * sizeof(GemmGroupEntry), &plan.table);
  if (rc == AH_OK) rc = ah_upload(plan.table, tab.data(), tab.size() * sizeof(GemmGroupEntry));
  if (rc == AH_OK && plan.out_dtype == AH_F32) rc = ah_alloc(((size_t)blocks * 4 + parts.size() * JOIN_BLOCKS) * sizeof(float), &plan.sumsq);
  if (rc) {
    if (plan.sumsq) ah_free(plan.sumsq);
    if (plan.ws) ah_free(plan.ws);
    if (plan.parts) ah_free(plan.parts);
    if (plan.table) ah_free(plan.table);
    return rc;
  }
  g_plans.push_back(plan);
  *plan_out = g_plan_base + g_plans.size();
  return AH_OK;
}

int32_t ah_gemm_grouped_update(uint64_t plan, const AhGemm *descs, int32_t count) {
  AH_REQUIRE_READY();
  AH_ARG(find_plan(plan) != nullptr, "ah_gemm_grouped_update: unknown plan %llu", (unsigned long long)plan);
  const GroupPlan &p = *find_plan(plan);
  std::vector<GemmGroupEntry> tab;
  std::vector<JoinPart> parts;
  int64_t blocks = 0, ws_bytes = 0;
  int32_t rc = grouped_tables("ah_gemm_grouped_update", descs, count, p.ws, tab, parts, &blocks, &ws_bytes);
  if (rc) return rc;
  if (count != p.ndescs || descs[0].layout != p.layout || descs[0].out_dtype != p.out_dtype || (int)tab.size() != p.count ||
      (int)blocks != p.blocks || (int)parts.size() != p.nparts || ws_bytes != p.ws_bytes || group_shape(descs, count) != p.shape)
    return fail(AH_ERR_ARG, "ah_gemm_grouped_update: the problems do not have the shapes the plan was made for");
  if (!parts.empty()) {
    rc = ah_upload(p.parts, parts.data(), parts.size() * sizeof(JoinPart));
    if (rc) return rc;
  }
  return ah_upload(p.table, tab.data(), tab.size() * sizeof(GemmGroupEntry));
}

// The launches of a plan; with sumsq_inout also the sum of the squares of everything they leave in the C matrices.
static int32_t grouped_run(const char *who, uint64_t plan, int32_t epilogue, ah_ptr sumsq_inout) {
  AH_REQUIRE_READY();
  AH_ARG(find_plan(plan) != nullptr, "%s: unknown plan %llu", who, (unsigned long long)plan);
  const GroupPlan &p = *find_plan(plan);
  AH_ARG(epilogue == AH_EPI_NONE || (epilogue == AH_EPI_ACCUM && p.out_dtype == AH_F32), "%s: epilogue %d is not provided for this plan", who, epilogue);
  const bool sums = sumsq_inout != 0;
  if (sums && p.out_dtype != AH_F32) return fail(AH_ERR_UNSUPPORTED, "%s: the sum of squares is provided for f32 outputs", who);
  const GemmGroupEntry *tab = dp<const GemmGroupEntry>(p.table);
  float *ss = sums ? dp<float>(p.sumsq) : nullptr;
  int32_t rc;
  switch (p.layout) {
    case AH_GEMM_NT: rc = gemm_bf16_dma_nt_grouped(tab, p.count, p.blocks, epilogue, p.out_dtype, ss); break;
    case AH_GEMM_NN: rc = gemm_bf16_dma_nn_grouped(tab, p.count, p.blocks, epilogue, p.out_dtype, ss); break;
    default: rc = gemm_bf16_dma_tn_grouped(tab, p.count, p.blocks, epilogue, p.out_dtype, ss);
  }
  if (rc != AH_OK) return rc;
  if (p.nparts > 0) {
    if (sums) ah::launch_kernel(k_grouped_join<true>, dim3(JOIN_BLOCKS, (unsigned)p.nparts), dim3(256), 0, dp<const JoinPart>(p.parts), ss + (size_t)p.blocks * 4);
    else ah::launch_kernel(k_grouped_join<false>, dim3(JOIN_BLOCKS, (unsigned)p.nparts), dim3(256), 0, dp<const JoinPart>(p.parts), (float *)nullptr);
    AH_LAUNCH_CHECK();
    ah::note_gemm_split(2);
  }
  if (sums) {
    ah::launch_kernel(k_grouped_sumsq_final, dim3(1), dim3(256), 0, (const float *)ss, p.blocks * 4 + p.nparts * JOIN_BLOCKS, dp<float>(sumsq_inout));
    AH_LAUNCH_CHECK();
  }
  return AH_OK;
}

int32_t ah_gemm_grouped_run(uint64_t plan, int32_t epilogue) { return grouped_run("ah_gemm_grouped_run", plan, epilogue, 0); }

int32_t ah_gemm_grouped_run_sumsq(uint64_t plan, int32_t epilogue, ah_ptr sumsq_inout) {
  AH_ARG(sumsq_inout != 0 && sumsq_inout % 4 == 0, "ah_gemm_grouped_run_sumsq: sumsq_inout must be an f32 on the device");
  return grouped_run("ah_gemm_grouped_run_sumsq", plan, epilogue, sumsq_inout);
}

int32_t ah_gemm_grouped_destroy(uint64_t plan) {
  AH_REQUIRE_READY();
  AH_ARG(find_plan(plan) != nullptr, "ah_gemm_grouped_destroy: unknown plan %llu", (unsigned long long)plan);
  GroupPlan &p = *find_plan(plan);
  p.live = false;
  if (p.sumsq) ah_free(p.sumsq);
  p.sumsq = 0;
  if (p.nparts > 0) {
    ah_free(p.parts);
    ah_free(p.ws);
    p.nparts = 0;
  }
  return ah_free(p.table);
}

int32_t ah_gemm_last_kernel(char *name, int32_t capacity, int32_t *nsplit) {
  AH_ARG(name != nullptr && capacity > 0, "ah_gemm_last_kernel: no output buffer");
  snprintf(name, (size_t)capacity, "%s", g_last_kernel);
  if (nsplit) *nsplit = g_last_split;
  return AH_OK;
}

int32_t ah_gemm_planes(const AhGemm *p, int64_t c_plane_cols, int64_t c_plane_stride, int64_t a_plane_k, int64_t a_plane_stride, int32_t dry_run) {
  AH_REQUIRE_READY();
  AH_ARG(p != nullptr, "ah_gemm_planes: null descriptor");
  const AhGemm &q = *p;
  AH_ARG(q.layout == AH_GEMM_NN || q.layout == AH_GEMM_NT, "ah_gemm_planes: layout NN or NT (A row-major [m, k])");
  AH_ARG(c_plane_cols >= 0 && a_plane_k >= 0 && (c_plane_cols > 0 || a_plane_k > 0), "ah_gemm_planes: no planes given");
  AH_ARG(q.m > 0 && q.n > 0 && q.k > 0 && q.m < (1ll << 31) && q.n < (1ll << 31) && q.k < (1ll << 31), "ah_gemm_planes: bad extent");
  AH_ARG(q.a != 0 && q.b != 0 && q.c != 0, "ah_gemm_planes: null operand");
  if (q.in_dtype != AH_BF16 || q.out_dtype != AH_BF16 || q.epilogue != AH_EPI_NONE || q.batch != 1)
    return fail(AH_ERR_UNSUPPORTED, "ah_gemm_planes: one plain product of bf16 operands with a bf16 result");
  const bool bkm = q.layout == AH_GEMM_NN;
  if (c_plane_cols > 0) {
    AH_ARG(q.n % c_plane_cols == 0 && q.ldc >= c_plane_cols && c_plane_stride % 4 == 0,
           "ah_gemm_planes: n = %lld is not whole planes of %lld columns, or ldc / the plane stride do not fit", (long long)q.n, (long long)c_plane_cols);
    AH_ARG(q.n == c_plane_cols || c_plane_stride >= (q.m - 1) * q.ldc + c_plane_cols,
           "ah_gemm_planes: planes of C %lld elements apart overlap (m = %lld rows of stride %lld)", (long long)c_plane_stride, (long long)q.m, (long long)q.ldc);
  } else {
    AH_ARG(q.ldc >= q.n, "matmul shape mismatch: ldc %lld too small for n=%lld", (long long)q.ldc, (long long)q.n);
  }
  if (a_plane_k > 0) {
    AH_ARG(q.k % a_plane_k == 0 && q.k / a_plane_k <= 3 && q.lda >= a_plane_k && a_plane_stride % 8 == 0 && a_plane_stride >= 0,
           "ah_gemm_planes: k = %lld is not 1 to 3 whole planes of %lld, or lda / the plane stride do not fit", (long long)q.k, (long long)a_plane_k);
  } else {
    AH_ARG(q.lda >= q.k, "matmul shape mismatch: lda %lld too small for k=%lld", (long long)q.lda, (long long)q.k);
  }
  AH_ARG(q.ldb >= (bkm ? q.n : q.k), "matmul shape mismatch: ldb %lld too small", (long long)q.ldb);
  // what the large-tile kernel asks of its operands (the checks ah_gemm makes before it takes that kernel)
  const bool fits = aligned16(q.a) && aligned16(q.b) && q.lda % 8 == 0 && q.ldb % 8 == 0 && (!bkm || q.n % 8 == 0) && q.k % 64 == 0 &&
                    q.c % 8 == 0 && q.ldc % 4 == 0 && (a_plane_k == 0 || a_plane_k % 64 == 0) && (c_plane_cols == 0 || c_plane_cols % 128 == 0);
  GemmArgs ga;
  ga.a = dp<const void>(q.a); ga.b = dp<const void>(q.b); ga.c = dp<void>(q.c);
  ga.aux = nullptr; ga.aux_out = nullptr;
  ga.M = (int)q.m; ga.N = (int)q.n; ga.K = (int)q.k;
  ga.lda = q.lda; ga.ldb = q.ldb; ga.ldc = q.ldc;
  ga.sa = ga.sb = ga.sc = 0;
  ga.epi = AH_EPI_NONE;
  ga.ksplit = (int)q.k; ga.nsplit = 1;
  ga.sumsq = nullptr;
  if (c_plane_cols > 0) { ga.c_plane_n = (int)c_plane_cols; ga.c_plane_adj = c_plane_stride - c_plane_cols; }
  if (a_plane_k > 0) { ga.a_plane_tiles = (int)(a_plane_k / 64); ga.a_plane_adj = (a_plane_stride - a_plane_k) * 2; }
  if (!fits || !ah::gemm_bf16_takes_large_tile(ga, q.layout))
    return fail(AH_ERR_UNSUPPORTED, "ah_gemm_planes: m=%lld n=%lld k=%lld does not run on the large-tile kernel", (long long)q.m, (long long)q.n, (long long)q.k);
  if (dry_run) return AH_OK;
  return ah::gemm_bf16_direct(ga, q.layout, 1, AH_BF16);
}

int32_t ah_gemm(const AhGemm *p) {
  AH_REQUIRE_READY();
  AH_ARG(p != nullptr, "ah_gemm: null descriptor");
  const AhGemm &q = *p;
  AH_ARG(q.layout >= AH_GEMM_NN && q.layout <= AH_GEMM_TN, "ah_gemm: bad layout %d", q.layout);
  AH_ARG(q.in_dtype == AH_F32 || q.in_dtype == AH_BF16, "ah_gemm: operands must be f32 or bf16");
  AH_ARG(q.out_dtype == AH_F32 || q.out_dtype == AH_BF16, "ah_gemm: output must be f32 or bf16");
  AH_ARG(q.epilogue >= AH_EPI_NONE && q.epilogue <= AH_EPI_MUL_AUX, "ah_gemm: bad epilogue %d", q.epilogue);
  AH_ARG(q.m >= 0 && q.n >= 0 && q.k >= 0 && q.batch >= 0, "ah_gemm: negative extent");
  AH_ARG(q.m < (1ll << 31) && q.n < (1ll << 31) && q.k < (1ll << 31) && q.batch <= 65535, "ah_gemm: extent too large");
  if (q.m == 0 || q.n == 0 || q.batch == 0) return AH_OK;
  AH_ARG(q.c != 0, "ah_gemm: null C");
  AH_ARG(q.k == 0 || (q.a != 0 && q.b != 0), "ah_gemm: null operand");
  // minimum leading dimensions for the stated layout
  int64_t a_cols = q.layout == AH_GEMM_TN ? q.m : q.k, b_cols = q.layout == AH_GEMM_NT ? q.k : q.n;
  AH_ARG(q.lda >= a_cols && q.ldb >= b_cols && q.ldc >= q.n, "matmul shape mismatch: lda/ldb/ldc (%lld,%lld,%lld) too small for m=%lld n=%lld k=%lld",
         (long long)q.lda, (long long)q.ldb, (long long)q.ldc, (long long)q.m, (long long)q.n, (long long)q.k);
  const bool gelu_like = q.epilogue == AH_EPI_GELU || q.epilogue == AH_EPI_GELU_BWD || q.epilogue == AH_EPI_GELU_GRAD || q.epilogue == AH_EPI_MUL_AUX;
  if (gelu_like || q.epilogue == AH_EPI_RESIDUAL)
    AH_ARG(q.aux != 0, "ah_gemm: epilogue %d needs aux", q.epilogue);
  // epilogue / output-type combinations: NONE -> f32 or bf16; ACCUM -> f32; RESIDUAL -> f32, or bf16 from bf16 operands (aux
  // then bf16 too); GELU, GELU_BWD -> the operand type
  bool combo = q.epilogue == AH_EPI_NONE || ((q.epilogue == AH_EPI_ACCUM || q.epilogue == AH_EPI_RESIDUAL) && q.out_dtype == AH_F32) ||
               (q.epilogue == AH_EPI_RESIDUAL && q.in_dtype == AH_BF16 && q.out_dtype == AH_BF16) || (gelu_like && q.out_dtype == q.in_dtype);
  if (!combo) return fail(AH_ERR_UNSUPPORTED, "ah_gemm: epilogue %d with operands of dtype %d and output dtype %d is not provided", q.epilogue, q.in_dtype, q.out_dtype);

  GemmArgs ga;
  ga.a = dp<const void>(q.a); ga.b = dp<const void>(q.b); ga.c = dp<void>(q.c);
  ga.aux = dp<const void>(q.aux); ga.aux_out = dp<void>(q.aux);
  ga.M = (int)q.m; ga.N = (int)q.n; ga.K = (int)q.k;
  ga.lda = q.lda; ga.ldb = q.ldb; ga.ldc = q.ldc;
  ga.sa = q.stride_a; ga.sb = q.stride_b; ga.sc = q.stride_c;
  ga.epi = q.epilogue;
  ga.ksplit = (int)q.k; ga.nsplit = 1;
  ga.sumsq = nullptr;
  int batch = (int)q.batch;

  // 4-wide epilogue accesses need 16-byte (f32) / 8-byte (bf16) aligned rows of C and aux
  int osz = q.out_dtype == AH_F32 ? 4 : 2;
  int vec_c = ((q.c % (4 * osz)) == 0) && (q.ldc % 4 == 0) && (q.stride_c % 4 == 0);
  if (q.epilogue == AH_EPI_RESIDUAL) vec_c = vec_c && (q.aux % (4 * osz) == 0);
  if (gelu_like) vec_c = vec_c && (q.aux % (4 * osz) == 0);
  if (q.in_dtype == AH_F32) {
    int vec_a = aligned16(q.a) && (q.lda % 4 == 0) && (q.stride_a % 4 == 0);
    int vec_b = aligned16(q.b) && (q.ldb % 4 == 0) && (q.stride_b % 4 == 0);
    auto run_f32 = [&](const GemmArgs &g, int nb, int vc) -> int32_t {
      switch (q.layout) {
        case AH_GEMM_NN: return launch_f32<AH_GEMM_NN>(g, nb, q.out_dtype, vec_a, vec_b, vc);
        case AH_GEMM_NT: return launch_f32<AH_GEMM_NT>(g, nb, q.out_dtype, vec_a, vec_b, vc);
        default: return launch_f32<AH_GEMM_TN>(g, nb, q.out_dtype, vec_a, vec_b, vc);
      }
    };
    // Split-K for a long contraction with too few output tiles to fill the chip (weight gradients: K = tokens): the
    // slices run as batch entries of the same kernel (batch strides step along K) into a workspace [slices][M][N], which
    // is then summed in fixed order.
    int64_t tiles = cdiv(q.m, F_BM) * cdiv(q.n, F_BN);
    if (batch == 1 && q.out_dtype == AH_F32 && (q.epilogue == AH_EPI_NONE || q.epilogue == AH_EPI_ACCUM) && tiles < num_cus() && q.k >= 2048 &&
        (q.m * q.n) % 4 == 0 && q.n % 4 == 0 && vec_c) {
      int s = (int)cdiv(2ll * num_cus(), tiles);
      if (s > 32) s = 32;
      while (s > 1 && (q.k % (s * 4) != 0 || q.k / s < 512)) s--;
      if (s > 1) {
        ah_ptr ws = 0;
        int32_t rc = ah_alloc((uint64_t)s * q.m * q.n * 4, &ws);
        if (rc) return rc;
        GemmArgs gs = ga;
        int64_t ks = q.k / s;
        gs.K = (int)ks; gs.ksplit = (int)ks;
        gs.sa = q.layout == AH_GEMM_TN ? ks * q.lda : ks;
        gs.sb = q.layout == AH_GEMM_NT ? ks : ks * q.ldb;
        gs.c = dp<void>(ws); gs.ldc = q.n; gs.sc = q.m * q.n; gs.epi = AH_EPI_NONE;
        rc = run_f32(gs, s, 1);
        if (rc == AH_OK) rc = ah::splitk_reduce(dp<const float>(ws), (float *)ga.c, s, ga.M, ga.N, ga.ldc, q.epilogue == AH_EPI_ACCUM);
        note_gemm_split(s);
        int32_t rf = ah_free(ws);
        return rc ? rc : rf;
      }
    }
    return run_f32(ga, batch, vec_c);
  }

  AH_ARG(q.k % 8 == 0, "ah_gemm: bf16 contraction length %lld must be a multiple of 8", (long long)q.k);
  ah_ptr zeros = 0;
  if (q.k == 0) {
    // A product over an empty contraction is all zeros (cpu_ref.ts:166-258 sums no terms), and the epilogue applies to that.
    // It runs as an A B^T product with k = 64 whose operand rows all alias one stretch of 64 zeros (leading dimensions and
    // batch strides 0), so every output type, epilogue and batch goes through the kernels it always goes through.
    const uint64_t zbytes = 64 * 2;
    int32_t rz = ah_alloc(zbytes, &zeros);
    if (rz) return rz;
    rz = ah_fill_i32(zeros, 0, zbytes / 4);
    if (rz) { ah_free(zeros); return rz; }
    ga.a = ga.b = dp<const void>(zeros);
    ga.lda = ga.ldb = 0; ga.sa = ga.sb = 0;
    ga.K = 64; ga.ksplit = 64;
    int32_t rc0 = vec_c ? ah::gemm_bf16_direct(ga, AH_GEMM_NT, batch, q.out_dtype) : run_bf16_nt(ga, batch, q.out_dtype, vec_c);
    int32_t rf = ah_free(zeros);      // stream-ordered: reusable only by later work
    return rc0 ? rc0 : rf;
  }
  {
    // direct kernel: every operand row (k-contiguous) or row group (k-major) must be 16-byte addressable
    bool akm = q.layout == AH_GEMM_TN, bkm = q.layout != AH_GEMM_NT;
    bool ok = aligned16(q.a) && aligned16(q.b) && q.lda % 8 == 0 && q.ldb % 8 == 0 && q.stride_a % 8 == 0 && q.stride_b % 8 == 0 &&
              (!akm || q.m % 8 == 0) && (!bkm || q.n % 8 == 0);
    ok = ok && vec_c && q.k % 64 == 0;
    if (ok) return ah::gemm_bf16_direct(ga, q.layout, batch, q.out_dtype);
  }
  // fallback for unaligned shapes: bring the operands into K-contiguous form with explicit transposes
  AH_ARG(batch == 1 || q.layout == AH_GEMM_NT, "ah_gemm: batched bf16 with unaligned operands is supported for the NT layout only");
  ah_ptr ta = 0, tb = 0;
  int32_t rc = AH_OK;
  if (q.layout == AH_GEMM_TN) {           // A is [K][M] -> [M][K]
    int64_t ldt = (q.k + 7) & ~7ll;
    rc = ah_alloc((uint64_t)q.m * ldt * 2, &ta);
    if (rc) return rc;
    ah::launch_kernel(k_transpose_u16, dim3((unsigned)cdiv(q.m, 64), (unsigned)cdiv(q.k, 64)), dim3(64, 4), 0, 
                       (const uint16_t *)ga.a, q.lda, dp<uint16_t>(ta), ldt, (int)q.k, (int)q.m);
    AH_LAUNCH_CHECK();
    ga.a = dp<const void>(ta); ga.lda = ldt;
  }
  if (q.layout != AH_GEMM_NT) {           // B is [K][N] -> [N][K]
    int64_t ldt = (q.k + 7) & ~7ll;
    rc = ah_alloc((uint64_t)q.n * ldt * 2, &tb);
    if (rc) { if (ta) ah_free(ta); return rc; }
    ah::launch_kernel(k_transpose_u16, dim3((unsigned)cdiv(q.n, 64), (unsigned)cdiv(q.k, 64)), dim3(64, 4), 0, 
                       (const uint16_t *)ga.b, q.ldb, dp<uint16_t>(tb), ldt, (int)q.k, (int)q.n);
    AH_LAUNCH_CHECK();
    ga.b = dp<const void>(tb); ga.ldb = ldt;
  }
  if (!(((uintptr_t)ga.a & 15u) == 0 && ((uintptr_t)ga.b & 15u) == 0 && ga.lda % 8 == 0 && ga.ldb % 8 == 0 && ga.sa % 8 == 0 && ga.sb % 8 == 0)) {
    if (ta) ah_free(ta);
    if (tb) ah_free(tb);
    return fail(AH_ERR_ARG, "ah_gemm: bf16 operands need 16-byte aligned rows (lda, ldb, batch strides multiples of 8)");
  }
  rc = run_bf16_nt(ga, batch, q.out_dtype, vec_c);
  if (ta) ah_free(ta);       // stream-ordered: reusable only by later work
  if (tb) ah_free(tb);
  return rc;
}

}  // extern "C"
