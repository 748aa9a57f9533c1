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
}  // namespace

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
