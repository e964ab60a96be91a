// Routing-scout predictor (Linear -> BatchNorm (eval) -> ReLU -> Linear -> softmax) for decode-size
// calls, in two launches: the hidden layer as one workgroup per hidden unit over all token rows, the
// head as one workgroup per token.  The predictor's parameters are fp32 with the BatchNorm folded into
// the first Linear by the host; the token rows come in the activations' storage type and are widened to
// fp32 on the way in, as the reference's `x.float()` does.
#include "common.h"

namespace sparse {

constexpr int kRsThreads = 256;
constexpr int kRsMaxTokens = SPARSE_HIP_DECODE_MAX_TOKENS;

template <typename T>
__device__ __forceinline__ void rs_load8(const T* p, float (&v)[8]);
template <>
__device__ __forceinline__ void rs_load8<float>(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <>
__device__ __forceinline__ void rs_load8<uint16_t>(const uint16_t* p, float (&v)[8]) {
  const u32x4 a = *reinterpret_cast<const u32x4*>(p);
  v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
  v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
  v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xffff0000u);
  v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xffff0000u);
}
template <>
__device__ __forceinline__ void rs_load8<f16_t>(const f16_t* p, float (&v)[8]) {
  const f16x8 a = *reinterpret_cast<const f16x8*>(p);
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = static_cast<float>(a[j]);
}

// hidden[t, j] = relu(b1[j] + <x[t, :], w1[j, :]>), one workgroup per hidden unit j.
template <typename T>
__global__ __launch_bounds__(kRsThreads) void rs_hidden_kernel(const T* __restrict__ x, const float* __restrict__ w1,
                                                               const float* __restrict__ b1, int Ttok, int H, int D,
                                                               float* __restrict__ hidden) {
  const int j = blockIdx.x;
  const float* w = w1 + static_cast<size_t>(j) * H;
  float acc[kRsMaxTokens];
#pragma unroll
  for (int i = 0; i < kRsMaxTokens; ++i) acc[i] = 0.f;
  for (int h = threadIdx.x * 8; h < H; h += kRsThreads * 8) {
    float wv[8];
    rs_load8<float>(w + h, wv);
#pragma unroll
    for (int i = 0; i < kRsMaxTokens; ++i) {
      if (i < Ttok) {
        float xv[8];
        rs_load8<T>(x + static_cast<size_t>(i) * H + h, xv);
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[i] = fmaf(xv[k], wv[k], acc[i]);
      }
    }
  }
  __shared__ float red[kRsThreads / 64][kRsMaxTokens];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < kRsMaxTokens; ++i) {
    if (i < Ttok) {
      const float s = wave_sum(acc[i]);
      if (lane == 0) red[wave][i] = s;
    }
  }
  __syncthreads();
  if (static_cast<int>(threadIdx.x) < Ttok) {
    float s = b1[j];
#pragma unroll
    for (int wv = 0; wv < kRsThreads / 64; ++wv) s += red[wv][threadIdx.x];
    hidden[static_cast<size_t>(threadIdx.x) * D + j] = fmaxf(s, 0.f);
  }
}

// pred[t, :] = softmax(b2 + w2 hidden[t, :]), one workgroup per token; wavefront w takes experts
// w, w + 4, ...
__global__ __launch_bounds__(kRsThreads) void rs_head_kernel(const float* __restrict__ hidden,
                                                             const float* __restrict__ w2,
                                                             const float* __restrict__ b2, int D, int E,
                                                             float* __restrict__ pred) {
  __shared__ float s_logit[SPARSE_HIP_MAX_EXPERTS];
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* hrow = hidden + static_cast<size_t>(t) * D;
  for (int e = wave; e < E; e += kRsThreads / 64) {
    const float* w = w2 + static_cast<size_t>(e) * D;
    float acc = 0.f;
    for (int d = lane * 4; d < D; d += 256) {
      const float4 a = *reinterpret_cast<const float4*>(w + d), b = *reinterpret_cast<const float4*>(hrow + d);
      acc = fmaf(a.x, b.x, acc);
      acc = fmaf(a.y, b.y, acc);
      acc = fmaf(a.z, b.z, acc);
      acc = fmaf(a.w, b.w, acc);
    }
    const float s = wave_sum(acc);
    if (lane == 0) s_logit[e] = s + b2[e];
  }
  __syncthreads();
  if (wave == 0) {
    float v[SPARSE_HIP_MAX_EXPERTS / 64];
    float m = -INFINITY;
#pragma unroll
    for (int q = 0; q < SPARSE_HIP_MAX_EXPERTS / 64; ++q) {
      const int e = lane + 64 * q;
      v[q] = e < E ? s_logit[e] : -INFINITY;
      m = fmaxf(m, v[q]);
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < SPARSE_HIP_MAX_EXPERTS / 64; ++q) {
      v[q] = (lane + 64 * q) < E ? expf(v[q] - m) : 0.f;
      sum += v[q];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int q = 0; q < SPARSE_HIP_MAX_EXPERTS / 64; ++q) {
      const int e = lane + 64 * q;
      if (e < E) pred[static_cast<size_t>(t) * E + e] = v[q] / sum;
    }
  }
}

}  // namespace sparse

using namespace sparse;

extern "C" int sparse_hip_rs_predict(const void* x_dev, int dtype, int T, int H, const float* w1_dev,
                                     const float* b1_dev, int D, const float* w2_dev, const float* b2_dev, int E,
                                     float* hidden_ws_dev, float* pred_dev, void* stream) {
  SP_REQUIRE(valid_dtype(dtype), "rs_predict: unknown dtype %d", dtype);
  SP_REQUIRE(T >= 1 && T <= kRsMaxTokens, "rs_predict: T=%d outside [1,%d]", T, kRsMaxTokens);
  SP_REQUIRE(H > 0 && H % 8 == 0, "rs_predict: H=%d must be a positive multiple of 8", H);
  SP_REQUIRE(D > 0 && D % 4 == 0, "rs_predict: hidden width D=%d must be a positive multiple of 4", D);
  SP_REQUIRE(E >= 1 && E <= SPARSE_HIP_MAX_EXPERTS, "rs_predict: E=%d outside [1,%d]", E, SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(x_dev && w1_dev && b1_dev && w2_dev && b2_dev && hidden_ws_dev && pred_dev, "rs_predict: NULL pointer");
  SP_REQUIRE(((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(w1_dev) |
               reinterpret_cast<uintptr_t>(w2_dev) | reinterpret_cast<uintptr_t>(hidden_ws_dev)) & 15) == 0,
             "rs_predict: pointers must be 16-byte aligned");
  hipStream_t st = as_stream(stream);
  if (dtype == SPARSE_HIP_F32) {
    hipLaunchKernelGGL((rs_hidden_kernel<float>), dim3(D), dim3(kRsThreads), 0, st, static_cast<const float*>(x_dev),
                       w1_dev, b1_dev, T, H, D, hidden_ws_dev);
  } else if (dtype == SPARSE_HIP_F16) {
    hipLaunchKernelGGL((rs_hidden_kernel<f16_t>), dim3(D), dim3(kRsThreads), 0, st, static_cast<const f16_t*>(x_dev),
                       w1_dev, b1_dev, T, H, D, hidden_ws_dev);
  } else {
    hipLaunchKernelGGL((rs_hidden_kernel<uint16_t>), dim3(D), dim3(kRsThreads), 0, st,
                       static_cast<const uint16_t*>(x_dev), w1_dev, b1_dev, T, H, D, hidden_ws_dev);
  }
  SP_LAUNCH_CHECK("rs_hidden_kernel");
  hipLaunchKernelGGL(rs_head_kernel, dim3(T), dim3(kRsThreads), 0, st, hidden_ws_dev, w2_dev, b2_dev, D, E, pred_dev);
  SP_LAUNCH_CHECK("rs_head_kernel");
  return SPARSE_HIP_OK;
}
