// Shared host/device helpers for libalpha_hip (gfx950 only, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stddef.h>
#include <tuple>
#include <utility>
#include "../../include/alpha_hip.h"

namespace ah {

// ---- host-side context (defined in runtime.hip) -------------------------------------------------
hipStream_t stream();
bool        ready();
int32_t     fail(int32_t code, const char *fmt, ...);
int32_t     hip_fail(hipError_t e, const char *what);
void        count_op();
int         num_cus();
// Scratch for two-stage reductions: a library-owned device buffer of at least `bytes` bytes that stays
// valid until the next call that asks for scratch on the same stream (calls are stream-ordered).  There is ONE buffer,
// ordered by the main stream: between ah_side_begin and ah_side_end it is refused (nullptr), as is growing it while a
// graph or step plan exists.
void       *scratch(size_t bytes);
int         current_device();                     // the device ah_init was called with
int32_t     static_partials_init(int device);     // reduce.hip: device address of its static scratch array (called by ah_init)
void        gemm_plans_forget();                  // gemm.hip: every grouped-GEMM plan id becomes unknown (called by ah_shutdown)

// Every kernel of the library is launched through launch_kernel(): the arguments are converted to the kernel's parameter
// types and handed, as an array of pointers to them, to launch_raw (runtime.hip).  Outside a step plan that is
// hipLaunchKernel on the library stream.  Inside one (ah_step_begin .. ah_step_end) the launch is recorded into the
// stream capture, or -- when a plan exists -- compared with the plan's next kernel node: same kernel, same grid means
// "skip, the graph will run it", with the node's parameters rewritten if any argument differs.
void launch_raw(const void *func, dim3 grid, dim3 block, unsigned shmem, void **args, const uint32_t *sizes, int nargs);
template <class... KArgs, class... Args, size_t... I>
inline void launch_impl(void (*kernel)(KArgs...), dim3 grid, dim3 block, unsigned shmem, std::index_sequence<I...>, Args &&...args) {
  std::tuple<KArgs...> vals{static_cast<KArgs>(std::forward<Args>(args))...};
  void *ptrs[sizeof...(KArgs) + 1] = {(void *)&std::get<I>(vals)..., nullptr};
  const uint32_t sizes[sizeof...(KArgs) + 1] = {(uint32_t)sizeof(KArgs)..., 0u};
  launch_raw(reinterpret_cast<const void *>(kernel), grid, block, shmem, ptrs, sizes, (int)sizeof...(KArgs));
}
template <class... KArgs, class... Args>
inline void launch_kernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, unsigned shmem, Args &&...args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "kernel argument count");
  launch_impl(kernel, grid, block, shmem, std::index_sequence_for<KArgs...>{}, std::forward<Args>(args)...);
}
// A point where the host needs the stream's results or touches it outside a kernel launch (download, sync, events):
// inside a step plan the work recorded so far is launched first.  Returns AH_OK or an error code.
int32_t step_boundary(const char *what);
bool    step_active();

#define AH_REQUIRE_READY() do { if (!ah::ready()) return ah::fail(AH_ERR_STATE, "%s: ah_init has not been called", __func__); } while (0)
#define AH_HIP(expr) do { hipError_t _e = (expr); if (_e != hipSuccess) return ah::hip_fail(_e, #expr); } while (0)
#define AH_ARG(cond, ...) do { if (!(cond)) return ah::fail(AH_ERR_ARG, __VA_ARGS__); } while (0)
#define AH_LAUNCH_CHECK() do { hipError_t _e = hipGetLastError(); if (_e != hipSuccess) return ah::hip_fail(_e, __func__); ah::count_op(); } while (0)

template <class T> static inline T *dp(ah_ptr p) { return reinterpret_cast<T *>(static_cast<uintptr_t>(p)); }
static inline bool aligned16(ah_ptr p) { return (p & 15u) == 0; }
static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- device helpers -----------------------------------------------------------------------------
typedef __hip_bfloat16 bf16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
// f32 -> bf16, round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950)
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2_t v;
  v[0] = (__bf16)lo; v[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return (uint16_t)(pack_bf16x2(f, 0.f) & 0xffffu); }

template <class T> struct Io;
template <> struct Io<float> {
  static __device__ __forceinline__ float ld(const float *p, size_t i) { return p[i]; }
  static __device__ __forceinline__ void  st(float *p, size_t i, float v) { p[i] = v; }
};
template <> struct Io<uint16_t> {   // bf16 storage
  static __device__ __forceinline__ float ld(const uint16_t *p, size_t i) { return bf16_bits_to_f32(p[i]); }
  static __device__ __forceinline__ void  st(uint16_t *p, size_t i, float v) { p[i] = f32_to_bf16_bits(v); }
};

// wave64 butterfly reductions
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// tanh-approximation GELU and its derivative (cpu_ref.ts:422-427; ops.ts:405-417) on the gate
// s = sigmoid(2u) = (1 + tanh u) / 2 with u = sqrt(2/pi) (x + 0.044715 x^3):  gelu(x) = x s and
// gelu'(x) = s + x s (1 - s) 2u'.  Two hardware transcendentals, no branches, absolute error at fp32 rounding level; a
// value + derivative pair costs 9 simple operations (the epilogues of the big GEMM tiles run one wave per SIMD, where
// every instruction costs 4 cycles, and cannot afford libm's tanhf: its register footprint on top of 256 live
// accumulators spills).
__device__ __forceinline__ float gelu_gate_s(float x, float x2) {
  const float k2 = 0.7978845608028654f * 2.0f * 1.4426950408889634f;      // 2 sqrt(2/pi) log2(e)
  float z = x * __builtin_fmaf(x2, -k2 * 0.044715f, -k2);
  return __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(z) + 1.0f);
}
__device__ __forceinline__ float gelu_f(float x) { return x * gelu_gate_s(x, x * x); }
// value and derivative from one gate evaluation
__device__ __forceinline__ void gelu_both_f(float x, float &val, float &grad) {
  const float k = 0.7978845608028654f;
  float x2 = x * x, s = gelu_gate_s(x, x2);
  float h = x * s;
  float d = __builtin_fmaf(x2, 6.0f * k * 0.044715f, 2.0f * k);           // 2 du/dx
  val = h;
  grad = __builtin_fmaf(h * d, 1.0f - s, s);
}
__device__ __forceinline__ float gelu_grad_f(float x) {
  float v, d;
  gelu_both_f(x, v, d);
  return d;
}

}  // namespace ah
