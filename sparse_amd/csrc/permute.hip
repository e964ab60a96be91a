// Token x K expansion and stable bucketing by expert id, staged in LDS.
//
// A block owns 256 consecutive tokens.  Inside a block the rank of item (t, k) among
// the items of its expert is the number of earlier tokens of the block that picked
// the same expert (a token picks an expert at most once), read off a per-expert
// token bitmap in LDS with popcounts.  Across blocks the ranks are offset by the
// per-block histograms of a first pass.  The result is the (expert id, t*K+k)
// order of a stable sort, with no atomics on positions, so it is deterministic.
#include "permute_device.h"

#include <mutex>

namespace sparse {

// Per-block histograms of the entry point that allocates nothing: one copy of this array
// per GPU, held until the process ends.  Host code never passes the array's name to a
// kernel (on the host it is a stand-in, not a device address); it asks the runtime for
// the address on the current device once and keeps it.
constexpr int kPermStaticBlocks = SPARSE_HIP_PERMUTE_STATIC_MAX_TOKENS / kPermThreads;
static __device__ __align__(256) int32_t scratch[kPermStaticBlocks * SPARSE_HIP_MAX_EXPERTS];

constexpr int kPermMaxDevices = 64;
static std::mutex g_scratch_mu;
static int32_t* g_scratch_ptr[kPermMaxDevices] = {nullptr};

// Device address of `scratch` on the current device (looked up on the first call there).
static int static_scratch(int32_t** out) {
  int dev = -1;
  SP_HIP(hipGetDevice(&dev));
  SP_REQUIRE(dev >= 0 && dev < kPermMaxDevices, "permute_build_static: device ordinal %d outside [0,%d)", dev,
             kPermMaxDevices);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    SP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    SP_REQUIRE(p != nullptr, "permute_build_static: hipGetSymbolAddress returned NULL");
    g_scratch_ptr[dev] = static_cast<int32_t*>(p);
  }
  *out = g_scratch_ptr[dev];
  return SPARSE_HIP_OK;
}

__global__ __launch_bounds__(kPermThreads) void permute_count_kernel(const int64_t* __restrict__ topi, int T,
                                                                     int K, int E,
                                                                     int32_t* __restrict__ block_counts) {
  __shared__ int32_t hist[SPARSE_HIP_MAX_EXPERTS];
  for (int e = threadIdx.x; e < E; e += kPermThreads) hist[e] = 0;
  __syncthreads();
  const int t = blockIdx.x * kPermThreads + threadIdx.x;
  if (t < T) {
    for (int k = 0; k < K; ++k) {
      const int64_t e = topi[static_cast<size_t>(t) * K + k];
      if (e >= 0 && e < E) atomicAdd(&hist[e], 1);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kPermThreads)
    block_counts[static_cast<size_t>(blockIdx.x) * E + e] = hist[e];
}

template <bool kSingleBlock>
__global__ __launch_bounds__(kPermThreads) void permute_scatter_kernel(
    const int64_t* __restrict__ topi, int T, int K, int E, const int32_t* __restrict__ block_counts,
    int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm, int32_t* __restrict__ seg_offsets,
    int32_t* __restrict__ active_eids, int32_t* __restrict__ n_active) {
  permute_scatter_block<kSingleBlock>(topi, T, K, E, block_counts, blockIdx.x, gridDim.x, perm, inv_perm,
                                      seg_offsets, active_eids, n_active);
}

}  // namespace sparse

using namespace sparse;

extern "C" {

size_t sparse_hip_permute_ws_bytes(int T, int K, int E) {
  (void)K;
  if (T <= 0 || E <= 0) return 0;
  const size_t nb = (static_cast<size_t>(T) + kPermThreads - 1) / kPermThreads;
  return nb * static_cast<size_t>(E) * sizeof(int32_t);
}

}  // extern "C"

static int permute_build_impl(const int64_t* topi_dev, int T, int K, int E, int32_t* perm_dev,
                              int32_t* inv_perm_dev, int32_t* seg_offsets_dev, int32_t* active_eids_dev,
                              int32_t* n_active_dev, void* ws_dev, void* stream) {
  SP_REQUIRE(T >= 1, "permute_build: T=%d must be >= 1", T);
  SP_REQUIRE(E >= 1 && E <= SPARSE_HIP_MAX_EXPERTS, "permute_build: E=%d outside [1,%d]", E,
             SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(K >= 1 && K <= SPARSE_HIP_MAX_TOPK && K <= E, "permute_build: K=%d outside [1,min(%d,E)]", K,
             SPARSE_HIP_MAX_TOPK);
  SP_REQUIRE(static_cast<int64_t>(T) * K < (1ll << 31), "permute_build: T*K overflows int32");
  SP_REQUIRE(topi_dev && perm_dev && inv_perm_dev && seg_offsets_dev && active_eids_dev && n_active_dev,
             "permute_build: NULL pointer");
  hipStream_t st = as_stream(stream);
  const int nb = (T + kPermThreads - 1) / kPermThreads;
  ProfScope prof(SPARSE_HIP_K_PERMUTE, st);
  if (nb == 1) {
    hipLaunchKernelGGL((permute_scatter_kernel<true>), dim3(1), dim3(kPermThreads), 0, st, topi_dev, T, K, E,
                       static_cast<const int32_t*>(nullptr), perm_dev, inv_perm_dev, seg_offsets_dev,
                       active_eids_dev, n_active_dev);
    SP_LAUNCH_CHECK("permute_scatter_kernel<single>");
    return SPARSE_HIP_OK;
  }
  SP_REQUIRE(ws_dev != nullptr, "permute_build: workspace is NULL for T=%d", T);
  int32_t* counts = static_cast<int32_t*>(ws_dev);
  hipLaunchKernelGGL(permute_count_kernel, dim3(nb), dim3(kPermThreads), 0, st, topi_dev, T, K, E, counts);
  SP_LAUNCH_CHECK("permute_count_kernel");
  hipLaunchKernelGGL((permute_scatter_kernel<false>), dim3(nb), dim3(kPermThreads), 0, st, topi_dev, T, K, E,
                     counts, perm_dev, inv_perm_dev, seg_offsets_dev, active_eids_dev, n_active_dev);
  SP_LAUNCH_CHECK("permute_scatter_kernel");
  return SPARSE_HIP_OK;
}

extern "C" {

int sparse_hip_permute_build(const int64_t* topi_dev, int T, int K, int E, int32_t* perm_dev,
                             int32_t* inv_perm_dev, int32_t* seg_offsets_dev, int32_t* active_eids_dev,
                             int32_t* n_active_dev, void* ws_dev, void* stream) {
  return permute_build_impl(topi_dev, T, K, E, perm_dev, inv_perm_dev, seg_offsets_dev, active_eids_dev,
                            n_active_dev, ws_dev, stream);
}

int sparse_hip_permute_build_static(const int64_t* topi_dev, int T, int K, int E, int32_t* perm_dev,
                                    int32_t* inv_perm_dev, int32_t* seg_offsets_dev, int32_t* active_eids_dev,
                                    int32_t* n_active_dev, void* stream) {
  SP_REQUIRE(T <= SPARSE_HIP_PERMUTE_STATIC_MAX_TOKENS,
             "permute_build_static: T=%d exceeds the built-in scratch (at most %d tokens); use "
             "sparse_hip_permute_build with a workspace",
             T, SPARSE_HIP_PERMUTE_STATIC_MAX_TOKENS);
  int32_t* counts = nullptr;
  const int rc = static_scratch(&counts);
  if (rc != SPARSE_HIP_OK) return rc;
  // The counting pass writes every histogram entry the scatter pass reads (blocks < ceil(T/256),
  // experts < E), so nothing of an earlier call's contents is ever read and nothing needs clearing.
  return permute_build_impl(topi_dev, T, K, E, perm_dev, inv_perm_dev, seg_offsets_dev, active_eids_dev,
                            n_active_dev, counts, stream);
}

}  // extern "C"
