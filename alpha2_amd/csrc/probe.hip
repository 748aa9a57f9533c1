// Measurement aids that are not ops: what the matrix pipes of this part sustain, so that a kernel's rate can be read
// against the hardware's own ceiling under its power limit and not only against the published peak.
#include "common.h"

namespace {
using namespace ah;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint32_t scramble(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// Every wave issues `iters` x 8 independent 32x32x16 bf16 MFMAs on operands held in registers: no LDS, no memory traffic
// (the guarded store is never taken).  RANDOM: four operand register sets of different pseudo-random values of the size
// of activations and weights; otherwise all zeros, which toggle no bits in the multipliers.
template <bool RANDOM>
__global__ __launch_bounds__(256) void k_probe_mfma_bf16(float *out, int iters) {
  bf16x8 a[4], b[4];
#pragma unroll
  for (int s = 0; s < 4; s++)
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t r = scramble(blockIdx.x * 977u + threadIdx.x * 131u + s * 17u + i);
      a[s][i] = (__bf16)(RANDOM ? ((int)(r & 0xffff) - 32768) * (0.02f / 32768.f) : 0.f);
      b[s][i] = (__bf16)(RANDOM ? ((int)(r >> 16) - 32768) * (1.0f / 32768.f) : 0.f);
    }
  f32x16 c[8];
#pragma unroll
  for (int j = 0; j < 8; j++)
#pragma unroll
    for (int e = 0; e < 16; e++) c[j][e] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int j = 0; j < 8; j++) c[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j & 3], b[(j + (j >> 2)) & 3], c[j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++)
#pragma unroll
    for (int e = 0; e < 16; e++) s += c[j][e];
  if (s == 12345.678f) out[threadIdx.x & 63] = s;
}

// Issue rates of one SIMD.  Every wave runs `iters` x 32 groups of instructions on eight independent register chains (no
// memory traffic, the guarded store is never taken); a group is KIND 0: one v_fma_f32, 1: one v_exp_f32, 2: one v_exp_f32 and
// three v_fma_f32, 3: one 32x32x16 bf16 MFMA (two accumulators alternate), 4 / 5: that MFMA followed by 8 / 16 v_fma_f32.
// Inline assembly, so that the compiler neither merges nor reorders what is being timed.
template <int KIND>
__global__ __launch_bounds__(1024) void k_probe_issue(float *out, int iters, float a, float b) {
  float x[8];
#pragma unroll
  for (int i = 0; i < 8; i++) x[i] = 0.001f * (float)(threadIdx.x + i);
  f32x16 acc0, acc1;
  bf16x8 fa, fb;
#pragma unroll
  for (int e = 0; e < 16; e++) { acc0[e] = 0.f; acc1[e] = 0.f; }
#pragma unroll
  for (int i = 0; i < 8; i++) { fa[i] = (__bf16)(0.01f * (float)(threadIdx.x & 63)); fb[i] = (__bf16)(0.02f * (float)i); }
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int g = 0; g < 32; g++) {
      if (KIND == 0) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[g & 7]) : "v"(a), "v"(b));
      if (KIND == 1 || KIND == 2) asm volatile("v_exp_f32 %0, %0" : "+v"(x[g & 7]));
      if (KIND == 2) {
#pragma unroll
        for (int i = 1; i < 4; i++) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[(g + 2 * i) & 7]) : "v"(a), "v"(b));
      }
      if (KIND >= 3) {
        if (g & 1) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc1) : "v"(fa), "v"(fb));
        else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc0) : "v"(fa), "v"(fb));
#pragma unroll
        for (int i = 0; i < (KIND == 4 ? 8 : KIND == 5 ? 16 : 0); i++) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[i & 7]) : "v"(a), "v"(b));
      }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) s += x[i];
#pragma unroll
  for (int e = 0; e < 16; e++) s += acc0[e] + acc1[e];
  if (s == 12345.678f) out[threadIdx.x & 63] = s;
}
}  // namespace

extern "C" int32_t ah_probe_issue(int32_t kind, int32_t waves_per_simd, int32_t iters, double *groups_per_simd_out) {
  AH_REQUIRE_READY();
  AH_ARG(kind >= 0 && kind <= 5 && waves_per_simd >= 1 && waves_per_simd <= (kind >= 3 ? 2 : 4) && iters >= 1 && iters <= 200000,
         "ah_probe_issue: kind 0-5, 1-4 waves per SIMD (1-2 with an MFMA in the group), 1-200000 iterations");
  float *out = (float *)scratch(256);
  if (out == nullptr) return fail(AH_ERR_OOM, "ah_probe_issue: no scratch");
  const dim3 grid((unsigned)num_cus()), block((unsigned)(256 * waves_per_simd));       // one workgroup per CU, its waves spread over the four SIMDs
  switch (kind) {
    case 0: ah::launch_kernel(k_probe_issue<0>, grid, block, 0, out, (int)iters, 0.999f, 0.001f); break;
    case 1: ah::launch_kernel(k_probe_issue<1>, grid, block, 0, out, (int)iters, 0.999f, 0.001f); break;
    case 2: ah::launch_kernel(k_probe_issue<2>, grid, block, 0, out, (int)iters, 0.999f, 0.001f); break;
    case 3: ah::launch_kernel(k_probe_issue<3>, grid, block, 0, out, (int)iters, 0.999f, 0.001f); break;
    case 4: ah::launch_kernel(k_probe_issue<4>, grid, block, 0, out, (int)iters, 0.999f, 0.001f); break;
    default: ah::launch_kernel(k_probe_issue<5>, grid, block, 0, out, (int)iters, 0.999f, 0.001f); break;
  }
  AH_LAUNCH_CHECK();
  if (groups_per_simd_out) *groups_per_simd_out = (double)iters * 32.0 * waves_per_simd;
  return AH_OK;
}

extern "C" int32_t ah_probe_mfma_bf16(int32_t waves_per_simd, int32_t iters, int32_t random_operands, double *flops_out) {
  AH_REQUIRE_READY();
  AH_ARG(waves_per_simd >= 1 && waves_per_simd <= 4 && iters >= 1 && iters <= 200000, "ah_probe_mfma_bf16: 1-4 waves per SIMD, 1-200000 iterations");
  float *out = (float *)scratch(256);
  if (out == nullptr) return fail(AH_ERR_OOM, "ah_probe_mfma_bf16: no scratch");
  const int blocks = num_cus() * waves_per_simd;      // 4 waves each: one per SIMD and round
  if (random_operands) ah::launch_kernel(k_probe_mfma_bf16<true>, dim3((unsigned)blocks), dim3(256), 0, out, (int)iters);
  else ah::launch_kernel(k_probe_mfma_bf16<false>, dim3((unsigned)blocks), dim3(256), 0, out, (int)iters);
  AH_LAUNCH_CHECK();
  if (flops_out) *flops_out = (double)blocks * 4.0 * iters * 8.0 * 2.0 * 32 * 32 * 16;
  return AH_OK;
}
