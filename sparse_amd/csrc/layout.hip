// Weight layout conversion (row-major <-> tiled) and the plain copy kernel used to
// calibrate HBM traffic counters.
#include "common.h"

namespace sparse {

// Element offset of (row, k) of an [R, K] matrix in the tiled layout.
__host__ __device__ inline size_t tiled_offset(int row, int k, int K) {
  return static_cast<size_t>(row >> 4) * 16 * K + static_cast<size_t>(k >> 6) * 1024 + ((k >> 3) & 1) * 512 +
         ((k >> 4) & 3) * 128 + (row & 15) * 8 + (k & 7);
}

template <typename T, bool kToTiled>
__global__ __launch_bounds__(256) void tile_weight_kernel(const T* __restrict__ src, T* __restrict__ dst, int R,
                                                          int K) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;  // row-major index
  if (i >= static_cast<size_t>(R) * K) return;
  const int row = static_cast<int>(i / K), k = static_cast<int>(i - static_cast<size_t>(row) * K);
  const size_t t = tiled_offset(row, k, K);
  if (kToTiled) {
    dst[t] = src[i];
  } else {
    dst[i] = src[t];
  }
}

__global__ __launch_bounds__(256) void calib_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                         size_t n16) {
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n16;
       i += static_cast<size_t>(gridDim.x) * 256)
    dst[i] = src[i];
}

}  // namespace sparse

using namespace sparse;

extern "C" {

int sparse_hip_tile_weight(const void* src_dev, void* dst_dev, int rows, int cols, int dtype, int to_tiled,
                           void* stream) {
  SP_REQUIRE(valid_dtype(dtype), "tile_weight: unknown dtype %d", dtype);
  SP_REQUIRE(rows > 0 && rows % 16 == 0 && cols > 0 && cols % 64 == 0,
             "tile_weight: rows=%d must be a multiple of 16 and cols=%d a multiple of 64", rows, cols);
  SP_REQUIRE(src_dev && dst_dev && src_dev != dst_dev, "tile_weight: NULL or aliased pointers");
  const size_t n = static_cast<size_t>(rows) * cols;
  const unsigned grid = static_cast<unsigned>((n + 255) / 256);
  hipStream_t st = as_stream(stream);
  if (is_16bit(dtype)) {
    if (to_tiled)
      hipLaunchKernelGGL((tile_weight_kernel<uint16_t, true>), dim3(grid), dim3(256), 0, st,
                         static_cast<const uint16_t*>(src_dev), static_cast<uint16_t*>(dst_dev), rows, cols);
    else
      hipLaunchKernelGGL((tile_weight_kernel<uint16_t, false>), dim3(grid), dim3(256), 0, st,
                         static_cast<const uint16_t*>(src_dev), static_cast<uint16_t*>(dst_dev), rows, cols);
  } else {
    if (to_tiled)
      hipLaunchKernelGGL((tile_weight_kernel<float, true>), dim3(grid), dim3(256), 0, st,
                         static_cast<const float*>(src_dev), static_cast<float*>(dst_dev), rows, cols);
    else
      hipLaunchKernelGGL((tile_weight_kernel<float, false>), dim3(grid), dim3(256), 0, st,
                         static_cast<const float*>(src_dev), static_cast<float*>(dst_dev), rows, cols);
  }
  SP_LAUNCH_CHECK("tile_weight_kernel");
  return SPARSE_HIP_OK;
}

int sparse_hip_calib_copy(const void* src_dev, void* dst_dev, size_t bytes, void* stream) {
  SP_REQUIRE(src_dev && dst_dev && bytes >= 16 && bytes % 16 == 0, "calib_copy: bytes=%zu must be a multiple of 16",
             bytes);
  SP_REQUIRE(((reinterpret_cast<uintptr_t>(src_dev) | reinterpret_cast<uintptr_t>(dst_dev)) & 15) == 0,
             "calib_copy: pointers must be 16-byte aligned");
  hipLaunchKernelGGL(calib_copy_kernel, dim3(2048), dim3(256), 0, as_stream(stream),
                     static_cast<const u32x4*>(src_dev), static_cast<u32x4*>(dst_dev), bytes / 16);
  SP_LAUNCH_CHECK("calib_copy_kernel");
  return SPARSE_HIP_OK;
}

}  // extern "C"
