// Routing-scout predictors on the device, fp32 arithmetic throughout (the reference feeds them
// `x.float()`).
//  * The plain predictor (Linear -> BatchNorm (eval) -> ReLU -> Linear -> softmax) in two launches: the
//    hidden layer as one workgroup per hidden unit and block of 32 token rows, the head as one workgroup
//    per token.  Parameters are fp32 with the BatchNorm folded into the first Linear by the host; the
//    token rows come in the activations' storage type and are widened on the way in.
//  * The building blocks of the deeper residual predictor (LayerNorm, Linear + GELU, pre-norm residual
//    units, LayerNorm, Linear, softmax): a dense layer with an optional activation and residual input,
//    a LayerNorm and a row softmax, which the host strings together.
#include <type_traits>

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

enum { kRsActNone = 0, kRsActRelu = 1, kRsActGelu = 2 };

__device__ __forceinline__ float rs_act(float v, int act) {
  if (act == kRsActRelu) return fmaxf(v, 0.f);
  if (act == kRsActGelu) return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));   // the exact form, nn.GELU's default
  return v;
}

// hidden[t, j] = act(b1[j] + <x[t, :], w1[j, :]>) (+ residual[t, j]), one workgroup per output unit j and
// block of kRsMaxTokens token rows (blockIdx.y).
template <typename T>
__global__ __launch_bounds__(kRsThreads) void rs_hidden_kernel(const T* __restrict__ x_all, const float* __restrict__ w1,
                                                               const float* __restrict__ b1, int Ttok_all, int H, int D,
                                                               float* __restrict__ hidden_all, int act,
                                                               const float* __restrict__ residual_all) {
  const int j = blockIdx.x;
  const int t0 = blockIdx.y * kRsMaxTokens;
  const int Ttok = min(kRsMaxTokens, Ttok_all - t0);
  const T* x = x_all + static_cast<size_t>(t0) * H;
  float* hidden = hidden_all + static_cast<size_t>(t0) * D;
  const float* residual = residual_all != nullptr ? residual_all + static_cast<size_t>(t0) * D : nullptr;
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
    s = rs_act(s, act);
    if (residual != nullptr) s += residual[static_cast<size_t>(threadIdx.x) * D + j];
    hidden[static_cast<size_t>(threadIdx.x) * D + j] = s;
  }
}

// out[t, :H] = (x[t, :H] - mean) / sqrt(var + eps) * gamma + beta, biased variance, one workgroup per token;
// rows of x are ld_in apart, rows of out ld_out, and out[t, H:ld_out] is set to zero.
template <typename T>
__global__ __launch_bounds__(kRsThreads) void rs_layernorm_kernel(const T* __restrict__ x, int H, int ld_in, int ld_out,
                                                                  const float* __restrict__ gamma,
                                                                  const float* __restrict__ beta, float eps,
                                                                  float* __restrict__ out) {
  __shared__ float red[2][kRsThreads / 64];
  const T* row = x + static_cast<size_t>(blockIdx.x) * ld_in;
  float* orow = out + static_cast<size_t>(blockIdx.x) * ld_out;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float sum = 0.f;
  for (int h = threadIdx.x; h < H; h += kRsThreads) sum += Elem<T>::load(row + h);
  sum = wave_sum(sum);
  if (lane == 0) red[0][wave] = sum;
  __syncthreads();
  const float mean = (red[0][0] + red[0][1] + red[0][2] + red[0][3]) / static_cast<float>(H);
  float sq = 0.f;
  for (int h = threadIdx.x; h < H; h += kRsThreads) {
    const float d = Elem<T>::load(row + h) - mean;
    sq = fmaf(d, d, sq);
  }
  sq = wave_sum(sq);
  if (lane == 0) red[1][wave] = sq;
  __syncthreads();
  const float rstd = rsqrtf((red[1][0] + red[1][1] + red[1][2] + red[1][3]) / static_cast<float>(H) + eps);
  for (int h = threadIdx.x; h < ld_out; h += kRsThreads)
    orow[h] = h < H ? (Elem<T>::load(row + h) - mean) * rstd * gamma[h] + beta[h] : 0.f;
}

// out[t, :] = [ float(x[t, :H]) | the token's K routing weights, rescaled to sum 1, at its K expert ids
// among E columns | zeros up to ld ], one workgroup per token.
template <typename T>
__global__ __launch_bounds__(kRsThreads) void rs_features_kernel(const T* __restrict__ x, int H,
                                                                 const int64_t* __restrict__ topi,
                                                                 const T* __restrict__ topv, int K, int E, int ld,
                                                                 float* __restrict__ out) {
  const T* row = x + static_cast<size_t>(blockIdx.x) * H;
  float* orow = out + static_cast<size_t>(blockIdx.x) * ld;
  for (int h = threadIdx.x; h < H; h += kRsThreads) orow[h] = Elem<T>::load(row + h);
  for (int h = H + threadIdx.x; h < ld; h += kRsThreads) orow[h] = 0.f;
  __syncthreads();
  if (threadIdx.x == 0) {
    const int64_t* ti = topi + static_cast<size_t>(blockIdx.x) * K;
    const T* tv = topv + static_cast<size_t>(blockIdx.x) * K;
    float sum = 0.f;
    for (int k = 0; k < K; ++k) sum += Elem<T>::load(tv + k);
    sum = fmaxf(sum, 1e-12f);
    for (int k = 0; k < K; ++k) {
      const int64_t e = ti[k];
      if (e >= 0 && e < E) orow[H + e] += Elem<T>::load(tv + k) / sum;
    }
  }
}

// out[t, :] = softmax(in[t, :]), one wavefront per row of at most SPARSE_HIP_MAX_EXPERTS entries.
__global__ __launch_bounds__(kRsThreads) void rs_softmax_kernel(const float* __restrict__ in, int Ttok, int E,
                                                                float* __restrict__ out) {
  const int t = blockIdx.x * (kRsThreads / 64) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= Ttok) return;
  float v[SPARSE_HIP_MAX_EXPERTS / 64];
  float m = -INFINITY;
#pragma unroll
  for (int q = 0; q < SPARSE_HIP_MAX_EXPERTS / 64; ++q) {
    const int e = lane + 64 * q;
    v[q] = e < E ? in[static_cast<size_t>(t) * E + e] : -INFINITY;
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
    if (e < E) out[static_cast<size_t>(t) * E + e] = v[q] / sum;
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

template <typename Launch>
static int rs_by_dtype(int dtype, Launch&& launch) {
  if (dtype == SPARSE_HIP_F32) launch(static_cast<const float*>(nullptr));
  else if (dtype == SPARSE_HIP_F16) launch(static_cast<const f16_t*>(nullptr));
  else launch(static_cast<const uint16_t*>(nullptr));
  return SPARSE_HIP_OK;
}

static int rs_dense_launch(const void* x_dev, int dtype, int T, int H, const float* w_dev, const float* b_dev, int D,
                           int act, const float* residual_dev, float* out_dev, hipStream_t st) {
  const dim3 grid(D, (T + kRsMaxTokens - 1) / kRsMaxTokens);
  rs_by_dtype(dtype, [&](auto tag) {
    typedef typename std::remove_cv<typename std::remove_pointer<decltype(tag)>::type>::type TT;
    hipLaunchKernelGGL((rs_hidden_kernel<TT>), grid, dim3(kRsThreads), 0, st, static_cast<const TT*>(x_dev), w_dev,
                       b_dev, T, H, D, out_dev, act, residual_dev);
  });
  SP_LAUNCH_CHECK("rs_hidden_kernel");
  return SPARSE_HIP_OK;
}

extern "C" int sparse_hip_rs_predict(const void* x_dev, int dtype, int T, int H, const float* w1_dev,
                                     const float* b1_dev, int D, const float* w2_dev, const float* b2_dev, int E,
                                     float* hidden_ws_dev, float* pred_dev, void* stream) {
  SP_REQUIRE(valid_dtype(dtype), "rs_predict: unknown dtype %d", dtype);
  SP_REQUIRE(T >= 1 && T <= 65535 * kRsMaxTokens, "rs_predict: T=%d outside [1,%d]", T, 65535 * kRsMaxTokens);
  SP_REQUIRE(H > 0 && H % 8 == 0, "rs_predict: H=%d must be a positive multiple of 8", H);
  SP_REQUIRE(D > 0 && D % 4 == 0, "rs_predict: hidden width D=%d must be a positive multiple of 4", D);
  SP_REQUIRE(E >= 1 && E <= SPARSE_HIP_MAX_EXPERTS, "rs_predict: E=%d outside [1,%d]", E, SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(x_dev && w1_dev && b1_dev && w2_dev && b2_dev && hidden_ws_dev && pred_dev, "rs_predict: NULL pointer");
  SP_REQUIRE(((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(w1_dev) |
               reinterpret_cast<uintptr_t>(w2_dev) | reinterpret_cast<uintptr_t>(hidden_ws_dev)) & 15) == 0,
             "rs_predict: pointers must be 16-byte aligned");
  hipStream_t st = as_stream(stream);
  const int rc = rs_dense_launch(x_dev, dtype, T, H, w1_dev, b1_dev, D, kRsActRelu, nullptr, hidden_ws_dev, st);
  if (rc != SPARSE_HIP_OK) return rc;
  hipLaunchKernelGGL(rs_head_kernel, dim3(T), dim3(kRsThreads), 0, st, hidden_ws_dev, w2_dev, b2_dev, D, E, pred_dev);
  SP_LAUNCH_CHECK("rs_head_kernel");
  return SPARSE_HIP_OK;
}

extern "C" int sparse_hip_rs_dense(const void* x_dev, int dtype, int T, int H, const float* w_dev, const float* b_dev,
                                   int D, int act, const float* residual_dev, float* out_dev, void* stream) {
  SP_REQUIRE(valid_dtype(dtype), "rs_dense: unknown dtype %d", dtype);
  SP_REQUIRE(T >= 1 && T <= 65535 * kRsMaxTokens, "rs_dense: T=%d outside [1,%d]", T, 65535 * kRsMaxTokens);
  SP_REQUIRE(H > 0 && H % 8 == 0, "rs_dense: input width %d must be a positive multiple of 8", H);
  SP_REQUIRE(D >= 1, "rs_dense: output width %d", D);
  SP_REQUIRE(act == kRsActNone || act == kRsActRelu || act == kRsActGelu, "rs_dense: activation %d is not 0 (none), 1 (ReLU) or 2 (GELU)", act);
  SP_REQUIRE(x_dev && w_dev && b_dev && out_dev, "rs_dense: NULL pointer");
  SP_REQUIRE(((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(w_dev)) & 15) == 0,
             "rs_dense: input and weights must be 16-byte aligned");
  SP_REQUIRE(static_cast<const void*>(out_dev) != x_dev, "rs_dense: output must not be the input");
  return rs_dense_launch(x_dev, dtype, T, H, w_dev, b_dev, D, act, residual_dev, out_dev, as_stream(stream));
}

extern "C" int sparse_hip_rs_layernorm(const void* x_dev, int dtype, int T, int H, int ld_in, int ld_out,
                                       const float* gamma_dev, const float* beta_dev, float eps, float* out_dev,
                                       void* stream) {
  SP_REQUIRE(valid_dtype(dtype), "rs_layernorm: unknown dtype %d", dtype);
  SP_REQUIRE(T >= 1 && H >= 1, "rs_layernorm: T=%d H=%d", T, H);
  SP_REQUIRE(ld_in >= H && ld_out >= H, "rs_layernorm: row strides %d, %d below the width %d", ld_in, ld_out, H);
  SP_REQUIRE(eps >= 0.f, "rs_layernorm: eps must not be negative");
  SP_REQUIRE(x_dev && gamma_dev && beta_dev && out_dev, "rs_layernorm: NULL pointer");
  SP_REQUIRE(static_cast<const void*>(out_dev) != x_dev, "rs_layernorm: output must not be the input");
  hipStream_t st = as_stream(stream);
  rs_by_dtype(dtype, [&](auto tag) {
    typedef typename std::remove_cv<typename std::remove_pointer<decltype(tag)>::type>::type TT;
    hipLaunchKernelGGL((rs_layernorm_kernel<TT>), dim3(T), dim3(kRsThreads), 0, st, static_cast<const TT*>(x_dev), H,
                       ld_in, ld_out, gamma_dev, beta_dev, eps, out_dev);
  });
  SP_LAUNCH_CHECK("rs_layernorm_kernel");
  return SPARSE_HIP_OK;
}

extern "C" int sparse_hip_rs_features(const void* x_dev, int dtype, int T, int H, const int64_t* topi_dev,
                                      const void* topv_dev, int K, int E, int ld, float* out_dev, void* stream) {
  SP_REQUIRE(valid_dtype(dtype), "rs_features: unknown dtype %d", dtype);
  SP_REQUIRE(T >= 1 && H >= 1 && K >= 1, "rs_features: T=%d H=%d K=%d", T, H, K);
  SP_REQUIRE(E >= 1 && E <= SPARSE_HIP_MAX_EXPERTS, "rs_features: E=%d outside [1,%d]", E, SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(ld >= H + E, "rs_features: row stride %d below H + E = %d", ld, H + E);
  SP_REQUIRE(x_dev && topi_dev && topv_dev && out_dev, "rs_features: NULL pointer");
  hipStream_t st = as_stream(stream);
  rs_by_dtype(dtype, [&](auto tag) {
    typedef typename std::remove_cv<typename std::remove_pointer<decltype(tag)>::type>::type TT;
    hipLaunchKernelGGL((rs_features_kernel<TT>), dim3(T), dim3(kRsThreads), 0, st, static_cast<const TT*>(x_dev), H,
                       topi_dev, static_cast<const TT*>(topv_dev), K, E, ld, out_dev);
  });
  SP_LAUNCH_CHECK("rs_features_kernel");
  return SPARSE_HIP_OK;
}

extern "C" int sparse_hip_rs_softmax(const float* in_dev, int T, int E, float* out_dev, void* stream) {
  SP_REQUIRE(T >= 1, "rs_softmax: T=%d", T);
  SP_REQUIRE(E >= 1 && E <= SPARSE_HIP_MAX_EXPERTS, "rs_softmax: E=%d outside [1,%d]", E, SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(in_dev && out_dev, "rs_softmax: NULL pointer");
  hipLaunchKernelGGL(rs_softmax_kernel, dim3((T + kRsThreads / 64 - 1) / (kRsThreads / 64)), dim3(kRsThreads), 0,
                     as_stream(stream), in_dev, T, E, out_dev);
  SP_LAUNCH_CHECK("rs_softmax_kernel");
  return SPARSE_HIP_OK;
}
