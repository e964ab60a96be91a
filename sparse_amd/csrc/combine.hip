// Un-permute + weighted-sum combine.  Rows in `parts` already carry their route weight;
// the sum over a token's K rows runs in ascending expert id (== ascending permuted
// row) with a rounding to the storage type after every add, then the shared-expert
// row is added the same way.
#include "common.h"

namespace sparse {

constexpr int kCombThreads = 256;

template <typename T>
__global__ __launch_bounds__(kCombThreads) void combine_kernel(const T* __restrict__ parts,
                                                               const int32_t* __restrict__ inv_perm,
                                                               const T* __restrict__ shared, int K, int H,
                                                               T* __restrict__ out) {
  const int hb = (H / 8 + kCombThreads - 1) / kCombThreads;
  const int t = blockIdx.x / hb;
  const int h = ((blockIdx.x - t * hb) * kCombThreads + threadIdx.x) * 8;
  if (h >= H) return;

  int32_t pos[SPARSE_HIP_MAX_TOPK];
#pragma unroll
  for (int k = 0; k < SPARSE_HIP_MAX_TOPK; ++k) pos[k] = (k < K) ? inv_perm[static_cast<size_t>(t) * K + k] : 0x7fffffff;
  // insertion sort, ascending (K <= 16)
#pragma unroll
  for (int i = 1; i < SPARSE_HIP_MAX_TOPK; ++i) {
#pragma unroll
    for (int j = i; j > 0; --j) {
      const int32_t lo = min(pos[j - 1], pos[j]), hi = max(pos[j - 1], pos[j]);
      pos[j - 1] = lo;
      pos[j] = hi;
    }
  }

  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
#pragma unroll
  for (int k = 0; k < SPARSE_HIP_MAX_TOPK; ++k) {
    if (k < K) {
      const T* row = parts + static_cast<size_t>(pos[k]) * H + h;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = Elem<T>::round(acc[j] + Elem<T>::load(row + j));
    }
  }
  if (shared != nullptr) {
    const T* row = shared + static_cast<size_t>(t) * H + h;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = Elem<T>::round(acc[j] + Elem<T>::load(row + j));
  }
  T* o = out + static_cast<size_t>(t) * H + h;
#pragma unroll
  for (int j = 0; j < 8; ++j) Elem<T>::store(o + j, acc[j]);
}

// The same sum for a decode call whose shared down projection was left as `nparts` fp32
// partial sums [nparts][T][H]: the shared value is bf16(bf16(p_0 + p_1 + ...) * bf16(sigmoid(
// gate[t]))) (no factor without a gate), exactly what the one-workgroup down projection
// stores, and is added after the routed parts.
template <typename T16>
__global__ __launch_bounds__(kCombThreads) void combine_split_kernel(
    const T16* __restrict__ parts, const int32_t* __restrict__ inv_perm, const float* __restrict__ sums,
    int nparts, const T16* __restrict__ gate, int T, int K, int H, T16* __restrict__ out) {
  const int hb = (H / 8 + kCombThreads - 1) / kCombThreads;
  const int t = blockIdx.x / hb;
  const int h = ((blockIdx.x - t * hb) * kCombThreads + threadIdx.x) * 8;
  if (h >= H) return;

  int32_t pos[SPARSE_HIP_MAX_TOPK];
#pragma unroll
  for (int k = 0; k < SPARSE_HIP_MAX_TOPK; ++k) pos[k] = (k < K) ? inv_perm[static_cast<size_t>(t) * K + k] : 0x7fffffff;
#pragma unroll
  for (int i = 1; i < SPARSE_HIP_MAX_TOPK; ++i) {
#pragma unroll
    for (int j = i; j > 0; --j) {
      const int32_t lo = min(pos[j - 1], pos[j]), hi = max(pos[j - 1], pos[j]);
      pos[j - 1] = lo;
      pos[j] = hi;
    }
  }

  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
#pragma unroll
  for (int k = 0; k < SPARSE_HIP_MAX_TOPK; ++k) {
    if (k < K) {
      const T16* row = parts + static_cast<size_t>(pos[k]) * H + h;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = Elem<T16>::round(acc[j] + Elem<T16>::load(row + j));
    }
  }
  const float* src = sums + static_cast<size_t>(t) * H + h;
  const size_t part_stride = static_cast<size_t>(T) * H;
  float sh[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) sh[j] = src[j];
  for (int p = 1; p < nparts; ++p) {
#pragma unroll
    for (int j = 0; j < 8; ++j) sh[j] += src[p * part_stride + j];
  }
  const bool gated = gate != nullptr;
  const float scale = gated ? Elem<T16>::round(sigmoid_f32(Elem<T16>::load(gate + t))) : 1.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float v = Elem<T16>::round(sh[j]);
    if (gated) v = v * scale;
    acc[j] = Elem<T16>::round(acc[j] + Elem<T16>::round(v));
  }
  T16* o = out + static_cast<size_t>(t) * H + h;
#pragma unroll
  for (int j = 0; j < 8; ++j) Elem<T16>::store(o + j, acc[j]);
}

}  // namespace sparse

using namespace sparse;

extern "C" int sparse_hip_combine_split(const void* parts_dev, const int32_t* inv_perm_dev, const void* split_ws_dev,
                                        int nparts, const void* shared_gate_dev, int dtype, int T, int K, int H,
                                        void* out_dev, void* stream) {
  SP_REQUIRE(is_16bit(dtype), "combine_split: dtype must be bf16 or fp16");
  SP_REQUIRE(T >= 0 && H > 0 && H % 8 == 0, "combine_split: bad shape T=%d H=%d", T, H);
  SP_REQUIRE(K >= 1 && K <= SPARSE_HIP_MAX_TOPK, "combine_split: K=%d outside [1,%d]", K, SPARSE_HIP_MAX_TOPK);
  SP_REQUIRE(nparts >= 1 && nparts <= 16, "combine_split: nparts=%d outside [1,16]", nparts);
  SP_REQUIRE(parts_dev && inv_perm_dev && split_ws_dev && out_dev, "combine_split: NULL pointer");
  if (T == 0) return SPARSE_HIP_OK;
  const int64_t nblk = static_cast<int64_t>((H / 8 + kCombThreads - 1) / kCombThreads) * T;
  SP_REQUIRE(nblk < (1ll << 31), "combine_split: grid too large");
  ProfScope prof(SPARSE_HIP_K_COMBINE, as_stream(stream));
  if (dtype == SPARSE_HIP_F16) {
    hipLaunchKernelGGL((combine_split_kernel<f16_t>), dim3(static_cast<unsigned>(nblk)), dim3(kCombThreads), 0,
                       as_stream(stream), static_cast<const f16_t*>(parts_dev), inv_perm_dev,
                       static_cast<const float*>(split_ws_dev), nparts, static_cast<const f16_t*>(shared_gate_dev), T, K,
                       H, static_cast<f16_t*>(out_dev));
  } else {
    hipLaunchKernelGGL((combine_split_kernel<uint16_t>), dim3(static_cast<unsigned>(nblk)), dim3(kCombThreads), 0,
                       as_stream(stream), static_cast<const uint16_t*>(parts_dev), inv_perm_dev,
                       static_cast<const float*>(split_ws_dev), nparts, static_cast<const uint16_t*>(shared_gate_dev), T,
                       K, H, static_cast<uint16_t*>(out_dev));
  }
  SP_LAUNCH_CHECK("combine_split_kernel");
  return SPARSE_HIP_OK;
}

extern "C" int sparse_hip_combine(const void* parts_dev, const int32_t* inv_perm_dev, const void* shared_dev,
                                  int dtype, int T, int K, int H, void* out_dev, void* stream) {
  SP_REQUIRE(valid_dtype(dtype), "combine: unknown dtype %d", dtype);
  SP_REQUIRE(T >= 0 && H > 0 && H % 8 == 0, "combine: bad shape T=%d H=%d", T, H);
  SP_REQUIRE(K >= 1 && K <= SPARSE_HIP_MAX_TOPK, "combine: K=%d outside [1,%d]", K, SPARSE_HIP_MAX_TOPK);
  SP_REQUIRE(parts_dev && inv_perm_dev && out_dev, "combine: NULL pointer");
  if (T == 0) return SPARSE_HIP_OK;
  const int64_t nblk = static_cast<int64_t>((H / 8 + kCombThreads - 1) / kCombThreads) * T;
  SP_REQUIRE(nblk < (1ll << 31), "combine: grid too large");
  dim3 grid(static_cast<unsigned>(nblk));
  ProfScope prof(SPARSE_HIP_K_COMBINE, as_stream(stream));
  if (dtype == SPARSE_HIP_BF16) {
    hipLaunchKernelGGL((combine_kernel<uint16_t>), grid, dim3(kCombThreads), 0, as_stream(stream),
                       static_cast<const uint16_t*>(parts_dev), inv_perm_dev,
                       static_cast<const uint16_t*>(shared_dev), K, H, static_cast<uint16_t*>(out_dev));
  } else if (dtype == SPARSE_HIP_F16) {
    hipLaunchKernelGGL((combine_kernel<f16_t>), grid, dim3(kCombThreads), 0, as_stream(stream),
                       static_cast<const f16_t*>(parts_dev), inv_perm_dev, static_cast<const f16_t*>(shared_dev), K, H,
                       static_cast<f16_t*>(out_dev));
  } else {
    hipLaunchKernelGGL((combine_kernel<float>), grid, dim3(kCombThreads), 0, as_stream(stream),
                       static_cast<const float*>(parts_dev), inv_perm_dev, static_cast<const float*>(shared_dev),
                       K, H, static_cast<float*>(out_dev));
  }
  SP_LAUNCH_CHECK("combine_kernel");
  return SPARSE_HIP_OK;
}
