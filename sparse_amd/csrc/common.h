// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "sparse_hip.h"

namespace sparse {

// ---- error plumbing ---------------------------------------------------------
void set_error(const char* fmt, ...);
int hip_fail(hipError_t err, const char* what);

#define SP_REQUIRE(cond, ...)              \
  do {                                     \
    if (!(cond)) {                         \
      sparse::set_error(__VA_ARGS__);      \
      return SPARSE_HIP_EINVAL;            \
    }                                      \
  } while (0)

#define SP_HIP(call)                                         \
  do {                                                       \
    hipError_t _e = (call);                                  \
    if (_e != hipSuccess) return sparse::hip_fail(_e, #call); \
  } while (0)

#define SP_LAUNCH_CHECK(name)                                    \
  do {                                                           \
    hipError_t _e = hipGetLastError();                           \
    if (_e != hipSuccess) return sparse::hip_fail(_e, name);      \
  } while (0)

// Brackets one kernel launch with an event pair while profiling is enabled.
struct ProfScope {
  ProfScope(int kernel, hipStream_t stream);
  ~ProfScope();
  int kernel_;
  hipStream_t stream_;
  hipEvent_t start_;
};

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
inline size_t elem_size(int dtype) { return dtype == SPARSE_HIP_BF16 ? 2 : 4; }
inline bool valid_dtype(int dtype) { return dtype == SPARSE_HIP_F32 || dtype == SPARSE_HIP_BF16; }

// ---- vector types -----------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

struct __attribute__((aligned(16))) u32x4 {
  uint32_t x, y, z, w;
};

// ---- bf16 <-> fp32 ----------------------------------------------------------
// Round-to-nearest-even, the rounding torch applies when it stores fp32 into bf16.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}
// fp32 value after a round trip through bf16.
__device__ __forceinline__ float round_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// Storage traits: T is float or uint16_t (bf16 bits).
template <typename T>
struct Elem;
template <>
struct Elem<float> {
  static constexpr int dtype = SPARSE_HIP_F32;
  __device__ static __forceinline__ float load(const float* p) { return *p; }
  __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
  __device__ static __forceinline__ float round(float v) { return v; }
};
template <>
struct Elem<uint16_t> {
  static constexpr int dtype = SPARSE_HIP_BF16;
  __device__ static __forceinline__ float load(const uint16_t* p) { return bf16_bits_to_f32(*p); }
  __device__ static __forceinline__ void store(uint16_t* p, float v) { *p = f32_to_bf16_bits(v); }
  __device__ static __forceinline__ float round(float v) { return round_bf16(v); }
};

// SiLU and sigmoid evaluated in fp32, as ATen does for reduced-precision inputs.
__device__ __forceinline__ float silu_f32(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float sigmoid_f32(float v) { return 1.0f / (1.0f + expf(-v)); }

// ---- wavefront (64 lanes) reductions ---------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

}  // namespace sparse
