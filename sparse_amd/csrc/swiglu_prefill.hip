// Prefill-time grouped SwiGLU expert FFN (bf16): the MFMA grouped-GEMM path.
//
// C[p, n] = sum_k A[p, k] * W[n, k] per expert segment.  A workgroup (4 waves) owns a
// 128-row x 256-weight-row tile; wave w owns all 128 rows and 64 of the weight rows
// (four by two 32x32x16 MFMA tiles, 128 accumulator registers), which keeps LDS reads at
// 6 fragments per 8 MFMAs.  For the gate/up projection the 256 weight rows are 128 gate
// rows and the 128 matching up rows, and a wave's two column tiles are the gate and
// the up tile of the same 32 neurons, so SiLU(gate)*up is a lane-local epilogue.
// Tiles go HBM -> registers -> LDS in 64-wide k slabs (one LDS buffer, the next slab
// is prefetched into registers while the current one is multiplied); LDS rows are
// padded to 144 bytes so 16-byte fragment reads are bank-conflict free.
//
// Block ids are dealt to the eight XCDs round-robin by the hardware; the kernel
// re-maps them so that an XCD works through whole experts, m-tiles of one weight tile
// adjacent in time, which keeps a weight tile in that XCD's L2 while it is reused.
//
// MFMA 32x32x16 bf16 operand layout (lane l, c = l & 31, g = l >> 5):
//   A: row c, k = g*8 .. g*8+7     B: column c, k = g*8 .. g*8+7
//   D: column c, rows 8*i + 4*g + j for register 4*i + j
#include "common.h"

namespace sparse {

constexpr int kPfBM = 128;        // rows per tile
constexpr int kPfBR = 256;        // weight rows per tile
constexpr int kPfBK = 64;         // k slab
constexpr int kPfThreads = 256;
constexpr int kPfRowBytes = kPfBK * 2 + 16;  // padded LDS row
constexpr int kPfLdsA = kPfBM * kPfRowBytes;
constexpr int kPfLdsB = kPfBR * kPfRowBytes;
constexpr int kPfXcds = 8;

struct PrefillArgs {
  const uint16_t* slab;
  uint64_t slot_stride;  // elements
  uint64_t mat_offset;   // elements
  uint64_t mat2_offset;  // elements
  const int32_t* expert_slot;
  const int32_t* perm;
  const int32_t* seg_offsets;
  const uint16_t* topv;
  const uint16_t* act;
  uint16_t* out;
  int32_t topk;
  int32_t Kdim;
  int32_t Ndim;       // output columns (neurons for gate-up, hidden for down)
  int32_t ntiles_n;
  int32_t max_mtiles;
  int32_t shared;
  int32_t T;
  const uint16_t* w_s;
  const uint16_t* w2_s;
  const uint16_t* gate_s;
  sparse_hip_seglist segs;
};

template <bool kGateUp>
__global__ __launch_bounds__(kPfThreads, 2) void prefill_ffn_kernel(const PrefillArgs a) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[kPfLdsA + kPfLdsB];
  __shared__ float s_scale[kPfBM];
  __shared__ int32_t s_seg[5];  // eid, first row, rows, n-tile, slot

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int fc = lane & 31, fg = lane >> 5;

  // ---- XCD-aware tile lookup -------------------------------------------------
  if (tid == 0) {
    const int nblk = gridDim.x;
    const int per_xcd = (nblk + kPfXcds - 1) / kPfXcds;
    const int logical = (blockIdx.x % kPfXcds) * per_xcd + blockIdx.x / kPfXcds;
    int eid = -1, r0 = 0, M = 0, bn = 0, slot_id = 0;
    if (a.shared) {
      // n-tile major, m fastest
      const int mt = (a.T + kPfBM - 1) / kPfBM;
      if (logical < mt * a.ntiles_n) {
        bn = logical / mt;
        const int bm = logical - bn * mt;
        eid = 0;
        r0 = bm * kPfBM;
        M = min(kPfBM, a.T - r0);
      }
    } else {
      int nseg = a.segs.n;
      if (a.segs.eids_dev != nullptr) nseg = min(nseg, a.segs.count_dev[0]);
      int left = logical;
      for (int s = 0; s < nseg; ++s) {
        const int e = (a.segs.eids_dev != nullptr) ? a.segs.eids_dev[s] : a.segs.eids[s];
        const int b = a.seg_offsets[e], m = a.seg_offsets[e + 1] - b;
        const int mt = (m + kPfBM - 1) / kPfBM;
        const int nt = mt * a.ntiles_n;
        if (left < nt) {
          bn = left / mt;
          const int bm = left - bn * mt;
          eid = e;
          slot_id = (a.segs.eids_dev != nullptr) ? a.expert_slot[e] : a.segs.slots[s];
          r0 = b + bm * kPfBM;
          M = min(kPfBM, m - bm * kPfBM);
          break;
        }
        left -= nt;
      }
    }
    s_seg[0] = eid;
    s_seg[1] = r0;
    s_seg[2] = M;
    s_seg[3] = bn;
    s_seg[4] = slot_id;
  }
  __syncthreads();
  const int eid = s_seg[0], r0 = s_seg[1], M = s_seg[2], bn = s_seg[3];
  if (eid < 0) return;

  const int Kdim = a.Kdim, Ndim = a.Ndim;
  const uint16_t *w0, *w1 = nullptr;
  if (a.shared) {
    w0 = a.w_s;
    w1 = a.w2_s;
  } else {
    const uint16_t* slot = a.slab + static_cast<uint64_t>(s_seg[4]) * a.slot_stride;
    w0 = slot + a.mat_offset;
    w1 = slot + a.mat2_offset;
  }
  // first output column of this tile
  const int n0 = bn * (kGateUp ? kPfBR / 2 : kPfBR);

  // per-row epilogue scale (down projection only)
  if (!kGateUp && tid < kPfBM) {
    float sc = 1.f;
    if (tid < M) {
      const int p = r0 + tid;
      if (a.shared) {
        if (a.gate_s != nullptr) sc = round_bf16(sigmoid_f32(bf16_bits_to_f32(a.gate_s[p])));
      } else {
        sc = bf16_bits_to_f32(a.topv[a.perm[p]]);
      }
    }
    s_scale[tid] = sc;
  }

  // ---- loader mapping: 32 rows x 8 sixteen-byte chunks per pass ---------------
  const int lrow = tid >> 3, lchunk = tid & 7;
  const uint16_t* aptr[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = min(lrow + 32 * i, M - 1);
    const int p = r0 + m;
    size_t row;
    if (a.shared || !kGateUp) {
      row = static_cast<size_t>(p);
    } else {
      row = static_cast<size_t>(a.perm[p] / a.topk);
    }
    aptr[i] = a.act + row * Kdim + lchunk * 8;
  }
  // Weight rows are tiled (16-row groups, 2 KB blocks of 64 k in MFMA lane order): a pass
  // of the workgroup copies two whole blocks, 128 sixteen-byte units each, so global reads
  // are 2 KB runs; unit u = h*64 + q*16 + r is row r, k = q*16 + h*8 .. +7 of its block.
  const int bu = tid & 127, bgrp = tid >> 7;
  const int br = bu & 15, bq = (bu >> 4) & 3, bh = bu >> 6;
  const uint16_t* bptr[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int g = 2 * i + bgrp;  // 16-row group inside the 256-row weight tile
    const uint16_t* base;
    int n;
    if (kGateUp) {
      base = (g < 8) ? w0 : w1;
      n = n0 + (g & 7) * 16;
    } else {
      base = w0;
      n = n0 + g * 16;
    }
    n = min(n, Ndim - 16);
    bptr[i] = base + static_cast<size_t>(n >> 4) * 16 * Kdim + bu * 8;
  }
  const int lds_wr_b = (bgrp * 16 + br) * kPfRowBytes + (bq * 2 + bh) * 16;
  const int lds_wr = lrow * kPfRowBytes + lchunk * 16;

  f32x16 acc[4][2];
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.f;

  u32x4 ra[4], rb[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) ra[i] = *reinterpret_cast<const u32x4*>(aptr[i]);
#pragma unroll
  for (int i = 0; i < 8; ++i) rb[i] = *reinterpret_cast<const u32x4*>(bptr[i]);

  // fragment read offsets
  const int a_rd = fc * kPfRowBytes + fg * 16;
  int b_rd[2];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const int row = kGateUp ? (ni * (kPfBR / 2) + wave * 32 + fc) : (wave * 64 + ni * 32 + fc);
    b_rd[ni] = kPfLdsA + row * kPfRowBytes + fg * 16;
  }

  const int nk = Kdim / kPfBK;
  for (int kt = 0; kt < nk; ++kt) {
    __syncthreads();  // previous slab fully consumed
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<u32x4*>(lds + lds_wr + i * 32 * kPfRowBytes) = ra[i];
#pragma unroll
    for (int i = 0; i < 8; ++i)
      *reinterpret_cast<u32x4*>(lds + kPfLdsA + lds_wr_b + i * 32 * kPfRowBytes) = rb[i];
    __syncthreads();
    if (kt + 1 < nk) {
      const int ko = (kt + 1) * kPfBK;
#pragma unroll
      for (int i = 0; i < 4; ++i) ra[i] = *reinterpret_cast<const u32x4*>(aptr[i] + ko);
#pragma unroll
      for (int i = 0; i < 8; ++i) rb[i] = *reinterpret_cast<const u32x4*>(bptr[i] + (kt + 1) * 1024);
    }
#pragma unroll
    for (int ks = 0; ks < kPfBK / 16; ++ks) {
      bf16x8 fa[4], fb[2];
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
        fa[mi] = *reinterpret_cast<const bf16x8*>(lds + a_rd + mi * 32 * kPfRowBytes + ks * 32);
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) fb[ni] = *reinterpret_cast<const bf16x8*>(lds + b_rd[ni] + ks * 32);
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mi], fb[ni], acc[mi][ni], 0, 0, 0);
    }
  }

  // ---- epilogue ----------------------------------------------------------------
#pragma unroll
  for (int mi = 0; mi < 4; ++mi) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int m = mi * 32 + 8 * i + 4 * fg + j;
        if (m >= M) continue;
        const size_t p = static_cast<size_t>(r0 + m);
        if (kGateUp) {
          const int n = n0 + wave * 32 + fc;
          if (n < Ndim) {
            const float g = round_bf16(acc[mi][0][4 * i + j]);
            const float u = round_bf16(acc[mi][1][4 * i + j]);
            a.out[p * Ndim + n] = f32_to_bf16_bits(round_bf16(silu_f32(g)) * u);
          }
        } else {
          const float sc = s_scale[m];
#pragma unroll
          for (int ni = 0; ni < 2; ++ni) {
            const int n = n0 + wave * 64 + ni * 32 + fc;
            if (n < Ndim) a.out[p * Ndim + n] = f32_to_bf16_bits(round_bf16(acc[mi][ni][4 * i + j]) * sc);
          }
        }
      }
    }
  }
}

template <bool kGateUp>
static int launch_prefill(PrefillArgs& a, hipStream_t st) {
  const int cols_per_tile = kGateUp ? kPfBR / 2 : kPfBR;
  a.ntiles_n = (a.Ndim + cols_per_tile - 1) / cols_per_tile;
  int64_t grid = static_cast<int64_t>(a.ntiles_n) * a.max_mtiles;
  grid = (grid + kPfXcds - 1) / kPfXcds * kPfXcds;
  if (grid == 0) return SPARSE_HIP_OK;
  SP_REQUIRE(grid < (1ll << 31), "prefill_ffn: grid too large");
  ProfScope prof(kGateUp ? SPARSE_HIP_K_PREFILL_GATEUP : SPARSE_HIP_K_PREFILL_DOWN, st);
  hipLaunchKernelGGL((prefill_ffn_kernel<kGateUp>), dim3(static_cast<unsigned>(grid)), dim3(kPfThreads), 0, st,
                     a);
  SP_LAUNCH_CHECK("prefill_ffn_kernel");
  return SPARSE_HIP_OK;
}

int prefill_routed_bf16(const sparse_hip_experts* ex, const void* x, const void* topv, const int32_t* perm,
                        const int32_t* seg_offsets, const sparse_hip_seglist* segs, int Ttok, int K,
                        void* inter_ws, void* parts, hipStream_t st) {
  const uint64_t H = ex->hidden, I = ex->inter;
  PrefillArgs a = {};
  a.slab = static_cast<const uint16_t*>(ex->slab_dev);
  a.slot_stride = ex->slot_stride / 2;
  a.expert_slot = ex->expert_slot_dev;
  a.perm = perm;
  a.seg_offsets = seg_offsets;
  a.topk = K;
  a.T = Ttok;
  a.segs = *segs;
  a.max_mtiles = (Ttok * K + kPfBM - 1) / kPfBM + segs->n;
  a.mat_offset = 0;
  a.mat2_offset = I * H;
  a.act = static_cast<const uint16_t*>(x);
  a.out = static_cast<uint16_t*>(inter_ws);
  a.Kdim = static_cast<int32_t>(H);
  a.Ndim = static_cast<int32_t>(I);
  int rc = launch_prefill<true>(a, st);
  if (rc != SPARSE_HIP_OK) return rc;
  a.mat_offset = 2 * I * H;
  a.mat2_offset = 0;
  a.topv = static_cast<const uint16_t*>(topv);
  a.act = static_cast<const uint16_t*>(inter_ws);
  a.out = static_cast<uint16_t*>(parts);
  a.Kdim = static_cast<int32_t>(I);
  a.Ndim = static_cast<int32_t>(H);
  return launch_prefill<false>(a, st);
}

int prefill_shared_bf16(const void* x, const void* gate_w, const void* up_w, const void* down_w,
                        const void* shared_gate, int Ttok, int H, int Is, void* inter_ws, void* shared_out,
                        hipStream_t st) {
  PrefillArgs a = {};
  a.shared = 1;
  a.T = Ttok;
  a.topk = 1;
  a.max_mtiles = (Ttok + kPfBM - 1) / kPfBM;
  a.w_s = static_cast<const uint16_t*>(gate_w);
  a.w2_s = static_cast<const uint16_t*>(up_w);
  a.act = static_cast<const uint16_t*>(x);
  a.out = static_cast<uint16_t*>(inter_ws);
  a.Kdim = H;
  a.Ndim = Is;
  int rc = launch_prefill<true>(a, st);
  if (rc != SPARSE_HIP_OK) return rc;
  a.w_s = static_cast<const uint16_t*>(down_w);
  a.w2_s = nullptr;
  a.gate_s = static_cast<const uint16_t*>(shared_gate);
  a.act = static_cast<const uint16_t*>(inter_ws);
  a.out = static_cast<uint16_t*>(shared_out);
  a.Kdim = Is;
  a.Ndim = H;
  return launch_prefill<false>(a, st);
}

}  // namespace sparse
