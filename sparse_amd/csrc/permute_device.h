// Device-side body of the stable expert bucketing, shared by the stand-alone permute
// kernels and the fused decode router.
#pragma once
#include "common.h"

namespace sparse {

constexpr int kPermThreads = 256;
constexpr int kMaskWords = kPermThreads / 32;

// Scatter pass of one 256-thread block over tokens [block*256, block*256+256).
// `block` / `num_blocks` stand for blockIdx.x / gridDim.x so that a fused kernel can run
// the pass as a single block.  With kSingleBlock the per-expert totals come from the
// block's own token bitmaps, otherwise from the histograms of the counting pass.
template <bool kSingleBlock>
__device__ __forceinline__ void permute_scatter_block(
    const int64_t* __restrict__ topi, int T, int K, int E, const int32_t* __restrict__ block_counts, int block,
    int num_blocks, int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm, int32_t* __restrict__ seg_offsets,
    int32_t* __restrict__ active_eids, int32_t* __restrict__ n_active) {
  __shared__ uint32_t mask[SPARSE_HIP_MAX_EXPERTS][kMaskWords];
  __shared__ int32_t scan_tot[SPARSE_HIP_MAX_EXPERTS];  // inclusive scan of per-expert totals
  __shared__ int32_t scan_act[SPARSE_HIP_MAX_EXPERTS];  // inclusive scan of (total > 0)
  __shared__ int32_t base[SPARSE_HIP_MAX_EXPERTS];      // first row of this block's items of e

  const int tid = threadIdx.x;
  for (int i = tid; i < E * kMaskWords; i += kPermThreads) (&mask[0][0])[i] = 0u;
  __syncthreads();

  const int t = block * kPermThreads + tid;
  int64_t my_e[SPARSE_HIP_MAX_TOPK];
  if (t < T) {
#pragma unroll
    for (int k = 0; k < SPARSE_HIP_MAX_TOPK; ++k) {
      if (k < K) {
        const int64_t e = topi[static_cast<size_t>(t) * K + k];
        my_e[k] = e;
        if (e >= 0 && e < E) atomicOr(&mask[e][tid >> 5], 1u << (tid & 31));
      }
    }
  }
  __syncthreads();

  // per-expert totals and the number of items in earlier blocks
  int32_t total = 0, before = 0;
  if (tid < E) {
    if (kSingleBlock) {
#pragma unroll
      for (int w = 0; w < kMaskWords; ++w) total += __popc(mask[tid][w]);
    } else {
      // eight histograms at a time: the loads do not depend on one another, and taken one by one each
      // would cost its own trip to the L2
      constexpr int kBatch = 8;
      for (int b0 = 0; b0 < num_blocks; b0 += kBatch) {
        int32_t c[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u)
          c[u] = (b0 + u < num_blocks) ? block_counts[static_cast<size_t>(b0 + u) * E + tid] : 0;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          total += c[u];
          if (b0 + u < block) before += c[u];
        }
      }
    }
  }
  scan_tot[tid] = (tid < E) ? total : 0;
  scan_act[tid] = (tid < E && total > 0) ? 1 : 0;
  __syncthreads();
  // Hillis-Steele inclusive scans over the 256 entries
  for (int off = 1; off < kPermThreads; off <<= 1) {
    int32_t a = 0, b = 0;
    if (tid >= off) {
      a = scan_tot[tid - off];
      b = scan_act[tid - off];
    }
    __syncthreads();
    scan_tot[tid] += a;
    scan_act[tid] += b;
    __syncthreads();
  }
  if (tid < E) {
    const int32_t excl = scan_tot[tid] - total;
    base[tid] = excl + before;
    if (block == 0) {
      seg_offsets[tid] = excl;
      if (tid == E - 1) seg_offsets[E] = scan_tot[tid];
      if (total > 0) active_eids[scan_act[tid] - 1] = tid;
      if (tid == E - 1) n_active[0] = scan_act[tid];
    }
  }
  __syncthreads();

  if (t < T) {
    const int word = tid >> 5;
    const uint32_t below = (1u << (tid & 31)) - 1u;
#pragma unroll
    for (int k = 0; k < SPARSE_HIP_MAX_TOPK; ++k) {
      if (k < K) {
        const int64_t e = my_e[k];
        if (e >= 0 && e < E) {
          int32_t rank = __popc(mask[e][word] & below);
          for (int w = 0; w < word; ++w) rank += __popc(mask[e][w]);
          const int32_t f = t * K + k;
          const int32_t pos = base[e] + rank;
          perm[pos] = f;
          inv_perm[f] = pos;
        }
      }
    }
  }
}

}  // namespace sparse
