// Tile geometry shared by the two prefill-size FFN kernels (one tile per workgroup, and persistent
// workgroups over queues of tiles).
#pragma once

#include <stdint.h>

namespace sparse {

constexpr int kPfBM = 128;        // rows per tile
constexpr int kPfBR = 256;        // weight rows per tile
constexpr int kPfBK = 64;         // k slab
constexpr int kPfThreads = 256;
constexpr int kPfRowBytes = kPfBK * 2;  // LDS row of one k slab (16-byte chunks swizzled by row)
constexpr int kPfLdsA = kPfBM * kPfRowBytes;
constexpr int kPfStages = 3;            // activation slabs resident in LDS
constexpr int kPfXcds = 8;

struct PfTile {
  int32_t slot;  // weight slot of the segment's expert; -1: a tile of the shared expert
  int32_t r0;    // first (permuted) row of the tile
  int32_t rows;  // rows in the tile (0: idle)
  int32_t bn;    // column tile
};

}  // namespace sparse
