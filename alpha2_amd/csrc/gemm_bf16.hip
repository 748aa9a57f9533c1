// bf16 GEMM on v_mfma_f32_32x32x16_bf16 for all three operand layouts of the training step.
//
// Block tile BM x BN x 64 on WGM x WGN waves, fp32 accumulators, LDS double-buffered.  Global loads run one k-tile
// ahead in registers so HBM / L2 latency is covered by a tile of MFMA work.
//   k-contiguous operand ([row][K] in memory): LDS tile [rows][64 + 8]; a fragment is one 16-byte read; the
//     144-byte pitch puts 8 consecutive rows on 8 distinct bank groups.
//   k-major operand ([K][row] in memory: W for dX = G W, G and X for dW = G^T X): the tile is copied as it lies,
//     LDS [64][rows + 32], and fragments come from ds_read_b64_tr_b16, the gfx950 LDS transpose read: within 16
//     lanes, lane j receives for q = 0..3 element [j % 4] of the 8 bytes addressed by lane 4q + j/4, so 16 lanes
//     pointing at a 4(k) x 16(row) block each get 4 consecutive k of "their" row.
// Addressing: one uniform 64-bit base per operand and k-tile (SGPRs) plus a 32-bit per-thread offset per chunk, so
// the loads need no per-chunk 64-bit pointers or predicates: rows past the edge are clamped onto the last valid row
// (their products land in accumulator rows / columns the epilogue never stores) and K is a multiple of 64.
#include "gemm_common.h"

using namespace ah;

namespace {

constexpr int G_BK = 64, G_PK = 72;      // k tile; k-contiguous LDS pitch (bf16 elements)
constexpr int G_KPAD = 32;               // k-major LDS pitch = rows + 32: consecutive k rows 64 bytes apart modulo 256
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // a native vector (not the HIP struct) so staging arrays stay in VGPRs

template <int ROWS, bool KMAJOR, int NT> struct TileGeom {
  static constexpr int PITCH = KMAJOR ? ROWS + G_KPAD : G_PK;
  static constexpr int ELEMS = KMAJOR ? G_BK * (ROWS + G_KPAD) : ROWS * G_PK;
  static constexpr int CHUNKS = ROWS * G_BK / 8 / NT;       // 16-byte chunks per thread and k-tile
};

// per-thread byte offsets of this thread's chunks relative to (operand base + k-tile start)
template <int ROWS, bool KMAJOR, int NT>
__device__ __forceinline__ void g_offsets(int64_t ld, int row0, int rows, uint32_t (&off)[TileGeom<ROWS, KMAJOR, NT>::CHUNKS]) {
  int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < TileGeom<ROWS, KMAJOR, NT>::CHUNKS; i++) {
    int c = t + NT * i;
    if (!KMAJOR) {
      int r = min(row0 + (c >> 3), rows - 1);
      off[i] = (uint32_t)(((int64_t)r * ld + (c & 7) * 8) * 2);
    } else {
      int r = min(row0 + (c % (ROWS / 8)) * 8, rows - 8);
      off[i] = (uint32_t)(((int64_t)(c / (ROWS / 8)) * ld + r) * 2);
    }
  }
}
template <int N>
__device__ __forceinline__ void g_load(const char *__restrict__ base, const uint32_t (&off)[N], u32x4 (&v)[N]) {
#pragma unroll
  for (int i = 0; i < N; i++) v[i] = *reinterpret_cast<const u32x4 *>(base + off[i]);
}
template <int ROWS, bool KMAJOR, int NT>
__device__ __forceinline__ void g_store(uint16_t *s, const u32x4 (&v)[TileGeom<ROWS, KMAJOR, NT>::CHUNKS]) {
  int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < TileGeom<ROWS, KMAJOR, NT>::CHUNKS; i++) {
    int c = t + NT * i;
    if (!KMAJOR) *reinterpret_cast<u32x4 *>(s + (c >> 3) * G_PK + (c & 7) * 8) = v[i];
    else *reinterpret_cast<u32x4 *>(s + (c / (ROWS / 8)) * (ROWS + G_KPAD) + (c % (ROWS / 8)) * 8) = v[i];
  }
}
// LDS element offset of this lane's fragment for tile rows [r0, r0+32), k-slice 0 (add kk * KSTEP per slice)
template <int ROWS, bool KMAJOR>
__device__ __forceinline__ int g_frag_base(int r0, int lane) {
  if (!KMAJOR) return (r0 + (lane & 31)) * G_PK + (lane >> 5) * 8;
  int j = lane & 15, g = lane >> 4;                  // 16-lane group g: rows r0 + 16*(g&1).., k half g>>1
  return ((g >> 1) * 8 + (j >> 2)) * (ROWS + G_KPAD) + r0 + (g & 1) * 16 + (j & 3) * 4;
}
template <int ROWS, bool KMAJOR>
__device__ __forceinline__ bf16x8 g_frag(const uint16_t *s, int base, int kk) {
  if (!KMAJOR) {
    return *reinterpret_cast<const bf16x8 *>(s + base + kk * 16);
  } else {
    typedef __attribute__((address_space(3))) bf16x4 lds_v4;
    const uint16_t *p = s + base + kk * 16 * (ROWS + G_KPAD);
    bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4 *)p);
    bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4 *)(p + 4 * (ROWS + G_KPAD)));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
}

// split-K: slice y writes its partial tile (plain f32 stores) to workspace[y][M][N]; this kernel then sums the slices
// in fixed order into C (deterministic, unlike atomic accumulation).
__global__ void k_splitk_reduce(const float *__restrict__ ws, float *__restrict__ c, int nsplit, int M, int N, int64_t ldc, int accumulate) {
  int64_t n4 = (int64_t)M * N / 4;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
    float4 s = reinterpret_cast<const float4 *>(ws)[i];
    for (int k = 1; k < nsplit; k++) {
      float4 v = reinterpret_cast<const float4 *>(ws + (int64_t)k * M * N)[i];
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    int64_t e = i * 4, row = e / N, col = e % N;
    float4 *dst = reinterpret_cast<float4 *>(c + row * ldc + col);
    if (accumulate) { float4 o = *dst; s.x += o.x; s.y += o.y; s.z += o.z; s.w += o.w; }
    *dst = s;
  }
}

template <int BM, int BN, int WGM, int WGN, bool AKM, bool BKM>
__global__ __launch_bounds__(64 * WGM * WGN) void k_gemm_bf16(GemmArgs g, int out_f32) {
  constexpr int NT = 64 * WGM * WGN, WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
  typedef TileGeom<BM, AKM, NT> GA;
  typedef TileGeom<BN, BKM, NT> GB;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t *As = smem;                       // [2][GA::ELEMS]
  uint16_t *Bs = smem + 2 * GA::ELEMS;       // [2][GB::ELEMS]
  // blockIdx.y = split-K slice: this block contracts k in [y * ksplit, (y + 1) * ksplit)
  const int64_t k_first = (int64_t)blockIdx.y * g.ksplit;
  const char *A = (const char *)((const uint16_t *)g.a + (int64_t)blockIdx.z * g.sa + (AKM ? k_first * g.lda : k_first));
  const char *B = (const char *)((const uint16_t *)g.b + (int64_t)blockIdx.z * g.sb + (BKM ? k_first * g.ldb : k_first));
  int64_t cbase = (int64_t)blockIdx.z * g.sc;
  // Tile order: consecutive block ids walk down M inside one N column, so the blocks resident at the same time
  // (and the 8 XCD L2s they are dealt to round-robin) share one B tile and stream disjoint A tiles.
  int tiles_m = (g.M + BM - 1) / BM;
  int m0 = (blockIdx.x % tiles_m) * BM, n0 = (blockIdx.x / tiles_m) * BN;
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int wm = (wave / WGN) * WM, wn = (wave % WGN) * WN;
  // bytes to advance per k-tile: 64 elements along a k-contiguous row, 64 rows of a k-major operand
  const int64_t a_step = AKM ? (int64_t)G_BK * g.lda * 2 : (int64_t)G_BK * 2;
  const int64_t b_step = BKM ? (int64_t)G_BK * g.ldb * 2 : (int64_t)G_BK * 2;

  uint32_t offa[GA::CHUNKS], offb[GB::CHUNKS];
  g_offsets<BM, AKM, NT>(g.lda, m0, g.M, offa);
  g_offsets<BN, BKM, NT>(g.ldb, n0, g.N, offb);
  int fa_base[TM], fb_base[TN];
#pragma unroll
  for (int i = 0; i < TM; i++) fa_base[i] = g_frag_base<BM, AKM>(wm + 32 * i, lane);
#pragma unroll
  for (int j = 0; j < TN; j++) fb_base[j] = g_frag_base<BN, BKM>(wn + 32 * j, lane);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

  // Staging registers for the one k-tile in flight between global memory and LDS.
  u32x4 ra[GA::CHUNKS], rb[GB::CHUNKS];
  const int nt = g.ksplit / G_BK, last = nt - 1;
  bf16x8 fa[2][TM], fb[2][TN];       // fragments of the current and the next k-slice

  auto read_frags = [&](int buf, int kk, int set) {
    const uint16_t *as = As + buf * GA::ELEMS, *bs = Bs + buf * GB::ELEMS;
#pragma unroll
    for (int i = 0; i < TM; i++) fa[set][i] = g_frag<BM, AKM>(as, fa_base[i], kk);
#pragma unroll
    for (int j = 0; j < TN; j++) fb[set][j] = g_frag<BN, BKM>(bs, fb_base[j], kk);
  };
  auto mfma_slice = [&](int set) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);   // operands swapped: C^T tile
  };
  // One k-tile (4 slices of 16).  Entering, LDS buffer `buf` holds tile t, fragment set 0 holds its slice 0, and the
  // staging registers hold (or are receiving) tile t + 1.  The fragments of slice kk + 1 are read while the MFMAs of
  // slice kk issue.  After slice 1 the staged tile goes to the other LDS buffer (free since the barrier that ended
  // tile t - 1) and the loads of tile t + 2 start, so a load has a whole tile of MFMA work to land.  The barrier sits
  // before the last slice: its MFMAs cover the LDS latency of the next tile's first fragments.  Tiles past the last
  // are clamped onto it (loaded and stored, never consumed), which keeps the steady state branch-free.
  auto tile = [&](int buf, int t) {
    read_frags(buf, 1, 1);
    mfma_slice(0);
    __builtin_amdgcn_sched_barrier(0);
    read_frags(buf, 2, 0);
    mfma_slice(1);
    __builtin_amdgcn_sched_barrier(0);
    g_store<BM, AKM, NT>(As + (buf ^ 1) * GA::ELEMS, ra);
    g_store<BN, BKM, NT>(Bs + (buf ^ 1) * GB::ELEMS, rb);
    g_load(A + min(t + 2, last) * a_step, offa, ra);
    g_load(B + min(t + 2, last) * b_step, offb, rb);
    __builtin_amdgcn_sched_barrier(0);
    read_frags(buf, 3, 1);
    mfma_slice(0);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    read_frags(buf ^ 1, 0, 0);
    mfma_slice(1);
    __builtin_amdgcn_sched_barrier(0);
  };

  g_load(A, offa, ra);
  g_load(B, offb, rb);
  g_store<BM, AKM, NT>(As, ra);
  g_store<BN, BKM, NT>(Bs, rb);
  g_load(A + min(1, last) * a_step, offa, ra);
  g_load(B + min(1, last) * b_step, offb, rb);
  __syncthreads();
  read_frags(0, 0, 0);
  int t = 0;
  for (; t + 2 <= nt; t += 2) {
    tile(0, t);
    tile(1, t + 1);
  }
  if (t < nt) tile(0, t);
  int r0 = m0 + wm, c0 = n0 + wn;
  if (g.nsplit > 1) {     // g.c is the split-K workspace [nsplit][M][N] here
    store_tiles<AH_EPI_NONE, float, TM, TN>(g, (int64_t)blockIdx.y * g.M * g.N, r0, c0, lane, acc);
    return;
  }
  switch (g.epi) {      // one uniform branch per kernel; only the combinations the dispatcher admits
    case AH_EPI_NONE:
      if (out_f32) store_tiles<AH_EPI_NONE, float, TM, TN>(g, cbase, r0, c0, lane, acc);
      else store_tiles<AH_EPI_NONE, uint16_t, TM, TN>(g, cbase, r0, c0, lane, acc);
      break;
    case AH_EPI_ACCUM: store_tiles<AH_EPI_ACCUM, float, TM, TN>(g, cbase, r0, c0, lane, acc); break;
    case AH_EPI_RESIDUAL:
      if (out_f32) store_tiles<AH_EPI_RESIDUAL, float, TM, TN>(g, cbase, r0, c0, lane, acc);
      else store_tiles<AH_EPI_RESIDUAL, uint16_t, TM, TN>(g, cbase, r0, c0, lane, acc);
      break;
    case AH_EPI_GELU: store_tiles<AH_EPI_GELU, uint16_t, TM, TN>(g, cbase, r0, c0, lane, acc); break;
    case AH_EPI_GELU_GRAD: store_tiles<AH_EPI_GELU_GRAD, uint16_t, TM, TN>(g, cbase, r0, c0, lane, acc); break;
    case AH_EPI_MUL_AUX: store_tiles<AH_EPI_MUL_AUX, uint16_t, TM, TN>(g, cbase, r0, c0, lane, acc); break;
    default: store_tiles<AH_EPI_GELU_BWD, uint16_t, TM, TN>(g, cbase, r0, c0, lane, acc); break;
  }
}

template <int BM, int BN, int WGM, int WGN, bool AKM, bool BKM>
int32_t launch(const GemmArgs &ga, int batch, int out_dtype) {
  constexpr int NT = 64 * WGM * WGN;
  size_t lds = sizeof(uint16_t) * 2 * (size_t)(TileGeom<BM, AKM, NT>::ELEMS + TileGeom<BN, BKM, NT>::ELEMS);
  int64_t tiles = cdiv(ga.M, BM) * cdiv(ga.N, BN);
  dim3 grid((unsigned)tiles, (unsigned)ga.nsplit, (unsigned)batch);
  auto kfn = k_gemm_bf16<BM, BN, WGM, WGN, AKM, BKM>;
  if (lds > 64 * 1024) {
    static bool raised = false;      // per instantiation: the attribute only needs setting once
    if (!raised) { AH_HIP(hipFuncSetAttribute((const void *)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); raised = true; }
  }
  note_gemm_kernel("k_gemm_bf16<%d, %d, %d, %d, %s, %s>", BM, BN, WGM, WGN, AKM ? "true" : "false", BKM ? "true" : "false");
  note_gemm_split(ga.nsplit);
  ah::launch_kernel(kfn, grid, dim3(NT), lds, ga, out_dtype == AH_F32 ? 1 : 0);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

// Large outputs go to the kernel fed by global->LDS loads (gemm_bf16_dma.inc): half the L2 traffic and a third of the
// LDS traffic per flop of the 128x128 tile.  It holds one block per CU, so what matters is how evenly the tiles fill
// whole rounds of CUs: take 256 x 256, 256 x 192 or 256 x 128 tiles, whichever wastes least of its last round, and keep the
// 128x128 tile of this file (two blocks per CU, finer grain) when neither fills 70 %.  Returns the tile width, 0 = the
// 128x128 kernel.  A product with planes only gets tile widths that divide a plane of C, and always gets one.
int pick_large_tile(const GemmArgs &ga, int batch, bool akm, bool bkm) {
  if (!(ga.M >= 256 && ga.N >= 128 && ga.ldc < (1 << 22))) return 0;      // (its epilogue addresses 128 rows of C with 31-bit byte offsets)
  const int64_t cus = num_cus(), per = (int64_t)batch * ga.nsplit;
  auto fill = [&](int bn) {
    if (ga.c_plane_n > 0 && ga.c_plane_n % bn != 0) return 0.0;
    int64_t t = cdiv(ga.M, 256) * cdiv(ga.N, bn) * per;
    double useful = (double)ga.N / (double)(cdiv(ga.N, bn) * bn);        // columns of edge tiles that exist
    return useful * (double)t / (double)(cdiv(t, cus) * cus);
  };
  // (narrower tiles read more from LDS per flop: measured ~3 % and ~8 % slower per flop than the 256-wide one; with two
  // k-major operands, whose transposing LDS reads run at half rate, the 128-wide tile is ~35 % slower per flop)
  double f256 = ga.N >= 256 ? fill(256) : 0.0, f192 = 0.97 * fill(192), f128 = (akm && bkm ? 0.65 : 0.92) * fill(128);
  int bn = f256 >= f192 && f256 >= f128 ? 256 : f192 >= f128 ? 192 : 128;
  const double best = bn == 256 ? f256 : bn == 192 ? f192 : f128;
  if (ga.c_plane_n > 0 || ga.a_plane_adj != 0) return best > 0.0 ? bn : 0;      // planes exist on this kernel only: taken however few tiles there are
  return best >= 0.7 ? bn : 0;
}

template <bool AKM, bool BKM>
int32_t run(const GemmArgs &ga, int batch, int out_dtype) {
  const int bn = pick_large_tile(ga, batch, AKM, BKM);
  if (bn) return AKM ? gemm_bf16_dma_tn(ga, batch, out_dtype, bn) : BKM ? gemm_bf16_dma_nn(ga, batch, out_dtype, bn) : gemm_bf16_dma_nt(ga, batch, out_dtype, bn);
  if (ga.c_plane_n > 0 || ga.a_plane_adj != 0) return fail(AH_ERR_UNSUPPORTED, "ah_gemm_planes: this shape does not run on the large-tile kernel");
  return launch<128, 128, 2, 2, AKM, BKM>(ga, batch, out_dtype);
}

}  // namespace

namespace ah {

bool gemm_bf16_takes_large_tile(const GemmArgs &ga, int layout) {
  return pick_large_tile(ga, 1, layout == AH_GEMM_TN, layout != AH_GEMM_NT) != 0;
}

// Preconditions (checked by the caller): K % 64 == 0; operands 16-byte aligned with lda/ldb/strides % 8 == 0;
// M % 8 == 0 (N % 8 == 0) when A (B) is k-major; C/aux rows vector-aligned; a provided epilogue/output combination.
int32_t splitk_reduce(const float *ws, float *c, int nsplit, int M, int N, int64_t ldc, bool accumulate) {
  int64_t n4 = (int64_t)M * N / 4;
  int blocks = (int)(cdiv(n4, 256) < 4096 ? cdiv(n4, 256) : 4096);
  ah::launch_kernel(k_splitk_reduce, dim3(blocks), dim3(256), 0, ws, c, nsplit, M, N, ldc, accumulate ? 1 : 0);
  AH_LAUNCH_CHECK();
  return AH_OK;
}

int32_t gemm_bf16_direct(const GemmArgs &ga, int layout, int batch, int out_dtype) {
  // per-thread offsets are 32-bit byte offsets from the operand base
  int64_t a_span = (layout == AH_GEMM_TN ? (int64_t)64 : (int64_t)ga.M) * ga.lda * 2;
  int64_t b_span = (layout == AH_GEMM_NT ? (int64_t)ga.N : (int64_t)64) * ga.ldb * 2;
  if (a_span >= (int64_t(1) << 32) || b_span >= (int64_t(1) << 32))
    return fail(AH_ERR_ARG, "ah_gemm: bf16 operand spans more than 4 GiB per batch entry");
  // Split-K for long contractions with few output tiles (the weight gradients dW = G^T X: K = tokens).
  GemmArgs gs = ga;
  int64_t tiles = cdiv(ga.M, 128) * cdiv(ga.N, 128), want = 3ll * num_cus();
  ah_ptr ws = 0;
  if (batch == 1 && out_dtype == AH_F32 && (ga.epi == AH_EPI_NONE || ga.epi == AH_EPI_ACCUM) && tiles < want && ga.K >= 2048 && ga.N % 4 == 0) {
    int s = (int)cdiv(want, tiles);
    while (s > 1 && (ga.K % (s * G_BK) != 0 || ga.K / s < 512)) s--;
    if (s > 1) {
      int32_t rc = ah_alloc((uint64_t)s * ga.M * ga.N * 4, &ws);
      if (rc) return rc;
      gs.nsplit = s; gs.ksplit = ga.K / s;
      gs.c = dp<void>(ws); gs.ldc = ga.N; gs.epi = AH_EPI_NONE;
    }
  }
  int32_t rc = layout == AH_GEMM_NT ? run<false, false>(gs, batch, out_dtype)
             : layout == AH_GEMM_NN ? run<false, true>(gs, batch, out_dtype) : run<true, true>(gs, batch, out_dtype);
  if (ws) {
    if (rc == AH_OK) rc = splitk_reduce(dp<const float>(ws), (float *)ga.c, gs.nsplit, ga.M, ga.N, ga.ldc, ga.epi == AH_EPI_ACCUM);
    int32_t rf = ah_free(ws);      // stream-ordered: reusable only by later work
    if (rc == AH_OK) rc = rf;
  }
  return rc;
}

}  // namespace ah
