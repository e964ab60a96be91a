// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "sparse_hip.h"

// The kernels here are written for one target.  Two things in them are outside what the language
// guarantees and hold on gfx950 (and its gfx9 family) only: the raw `s_waitcnt` immediates below use the
// gfx9 encoding (vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8), and the hand-off between
// workgroups in the decode kernel relies on device-scope (sc1) stores being written through to memory
// and acknowledged only then.  Compiling the device code for anything else must fail here.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "libsparse_hip's kernels are gfx950 code: s_waitcnt immediates and the sc1 write-through hand-off assume it"
#endif

namespace sparse {

// s_waitcnt immediates, gfx9 encoding, expcnt and lgkmcnt left at "do not wait" (7 and 15).
constexpr int kWaitVmcnt0 = 0x0F70;    // vmcnt(0)
constexpr int kWaitVmcnt20 = 0x4F74;   // vmcnt(20): 20 = 0b01'0100 -> bits 15:14 = 01, bits 3:0 = 0100
static_assert((kWaitVmcnt0 & 0xC00F) == 0 && (kWaitVmcnt0 & 0x0F70) == 0x0F70, "vmcnt(0), nothing else waited for");
static_assert((((kWaitVmcnt20 >> 14) & 3) << 4 | (kWaitVmcnt20 & 15)) == 20 && (kWaitVmcnt20 & 0x0F70) == 0x0F70,
              "vmcnt(20), nothing else waited for");

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

// Times one kernel launch while profiling is enabled.  Either the scope records an event
// before and after the launch (the interval then contains the dispatch latency of the launch,
// 2-3 us), or the launch site asks for the pair with `dispatch_events` and hands it to
// hipExtLaunchKernelGGL, which stamps the events with the dispatch's own begin and end.
struct ProfScope {
  ProfScope(int kernel, hipStream_t stream, bool dispatch_events = false);
  ~ProfScope();
  bool active() const { return start_ != nullptr && stop_ != nullptr; }
  int kernel_;
  hipStream_t stream_;
  hipEvent_t start_, stop_;  // stop_ is set only for dispatch events
};

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
inline size_t elem_size(int dtype) { return dtype == SPARSE_HIP_F32 ? 4 : 2; }
inline bool valid_dtype(int dtype) {
  return dtype == SPARSE_HIP_F32 || dtype == SPARSE_HIP_BF16 || dtype == SPARSE_HIP_F16;
}
inline bool is_16bit(int dtype) { return dtype == SPARSE_HIP_BF16 || dtype == SPARSE_HIP_F16; }

// ---- vector types -----------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef _Float16 f16_t;  // IEEE half: the storage tag of fp16 tensors (bf16 tensors are tagged uint16_t)
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

struct __attribute__((aligned(16))) u32x4 {
  uint32_t x, y, z, w;
};

// ---- bf16 <-> fp32 ----------------------------------------------------------
// Round-to-nearest-even, the rounding torch applies when it stores fp32 into bf16; gfx950
// converts in hardware (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}
// Two values at once, `lo` in bits 0..15.
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
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

// IEEE half: round-to-nearest-even conversions in hardware, as torch's.
template <>
struct Elem<f16_t> {
  static constexpr int dtype = SPARSE_HIP_F16;
  __device__ static __forceinline__ float load(const f16_t* p) { return static_cast<float>(*p); }
  __device__ static __forceinline__ void store(f16_t* p, float v) { *p = static_cast<f16_t>(v); }
  __device__ static __forceinline__ float round(float v) { return static_cast<float>(static_cast<f16_t>(v)); }
};

// The two 16-bit formats as the MFMA kernels see them: tensors are raw uint16_t there, and a format is
// its conversions plus its matrix instruction.  Operand fragments are 16 bytes either way (bf16x8 is the
// carrier type; the fp16 instruction takes the same bits as f16x8).
struct Bf16 {
  static constexpr int dtype = SPARSE_HIP_BF16;
  __device__ static __forceinline__ float from_bits(uint16_t b) { return bf16_bits_to_f32(b); }
  __device__ static __forceinline__ uint16_t bits(float f) { return f32_to_bf16_bits(f); }
  __device__ static __forceinline__ float round(float f) { return round_bf16(f); }
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) { return f32x2_to_bf16x2_bits(lo, hi); }
  __device__ static __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
struct Fp16 {
  static constexpr int dtype = SPARSE_HIP_F16;
  __device__ static __forceinline__ float from_bits(uint16_t b) {
    return static_cast<float>(__builtin_bit_cast(f16_t, b));
  }
  __device__ static __forceinline__ uint16_t bits(float f) { return __builtin_bit_cast(uint16_t, static_cast<f16_t>(f)); }
  __device__ static __forceinline__ float round(float f) { return static_cast<float>(static_cast<f16_t>(f)); }
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    return static_cast<uint32_t>(bits(lo)) | (static_cast<uint32_t>(bits(hi)) << 16);
  }
  __device__ static __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
// storage tag -> format
template <typename T> struct FormatOf;
template <> struct FormatOf<uint16_t> { typedef Bf16 type; };
template <> struct FormatOf<f16_t> { typedef Fp16 type; };

// SiLU and sigmoid evaluated in fp32, as ATen does for reduced-precision inputs.  SiLU runs
// once per intermediate element, so it uses the hardware exp2 and reciprocal (a few fp32
// ulp, far below the bf16 rounding that follows).
__device__ __forceinline__ float silu_f32(float v) {
  return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * v));
}
__device__ __forceinline__ float sigmoid_f32(float v) { return 1.0f / (1.0f + expf(-v)); }

// ---- wavefront (64 lanes) reductions ---------------------------------------
// Data-parallel-primitive moves instead of LDS permutes: four shifts inside each row of
// 16 lanes leave the row total in its lane 15, two row broadcasts carry the totals up to
// lane 63, and a read of lane 63 hands the result to every lane.  All 64 lanes must be
// active.  A lane whose source falls outside its row, or whose row is masked off, gets
// `identity`.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_move(float identity, float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(__float_as_int(identity), __float_as_int(v), kCtrl, kRowMask, 0xf, false));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0x111, 0xf>(0.f, v);  // row_shr:1
  v += dpp_move<0x112, 0xf>(0.f, v);  // row_shr:2
  v += dpp_move<0x114, 0xf>(0.f, v);  // row_shr:4
  v += dpp_move<0x118, 0xf>(0.f, v);  // row_shr:8
  v += dpp_move<0x142, 0xa>(0.f, v);  // row_bcast:15 into rows 1 and 3
  v += dpp_move<0x143, 0xc>(0.f, v);  // row_bcast:31 into rows 2 and 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
template <int kCtrl, int kRowMask>
__device__ __forceinline__ int dpp_move_int(int identity, int v) {
  return __builtin_amdgcn_update_dpp(identity, v, kCtrl, kRowMask, 0xf, false);
}
__device__ __forceinline__ int wave_min_int(int v) {
  constexpr int kMax = 0x7fffffff;
  v = min(v, dpp_move_int<0x111, 0xf>(kMax, v));
  v = min(v, dpp_move_int<0x112, 0xf>(kMax, v));
  v = min(v, dpp_move_int<0x114, 0xf>(kMax, v));
  v = min(v, dpp_move_int<0x118, 0xf>(kMax, v));
  v = min(v, dpp_move_int<0x142, 0xa>(kMax, v));
  v = min(v, dpp_move_int<0x143, 0xc>(kMax, v));
  return __builtin_amdgcn_readlane(v, 63);
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0x111, 0xf>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x112, 0xf>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x114, 0xf>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x118, 0xf>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x142, 0xa>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x143, 0xc>(-INFINITY, v));
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

}  // namespace sparse
