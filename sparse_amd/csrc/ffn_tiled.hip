// Grouped SwiGLU FFN with plain FMA tiles: the fp32 path (correctness anchor, any T)
// and the element-type-generic fallback shape for segments of any length.
//
// C[m, n] = sum_k A[m, k] * W[n, k] per segment, 64x64 output tiles, BK = 16, staged
// through LDS; each thread owns a 4x4 micro-tile and walks k in order, so the fp32
// summation order is fixed.  Rows of A are gathered (gate-up: x[perm[p]/K]; down:
// inter[p]); the epilogue applies the same rounding points as the reference's
// F.linear -> act*up -> F.linear -> *w chain (utils/eval_core.py:11722-11731).
#include "common.h"

namespace sparse {

constexpr int kTlBM = 64, kTlBN = 64, kTlBK = 16, kTlThreads = 256;

struct TiledArgs {
  const void* slab;
  uint64_t slot_stride;  // elements
  uint64_t mat_offset;   // elements
  uint64_t mat2_offset;  // elements
  const int32_t* expert_slot;
  const int32_t* perm;
  const int32_t* seg_offsets;
  const void* topv;
  const void* act;
  void* out;
  int32_t topk;
  int32_t Kdim;
  int32_t Ndim;
  int32_t ntiles_n;
  // shared expert mode: one pseudo-segment of T identity rows
  int32_t shared;
  int32_t T;
  const void* w_s;
  const void* w2_s;
  const void* gate_s;
  sparse_hip_seglist segs;
};

template <typename T, bool kGateUp>
__global__ __launch_bounds__(kTlThreads) void ffn_tiled_kernel(const TiledArgs a) {
  constexpr int NM = kGateUp ? 2 : 1;
  __shared__ float As[kTlBK][kTlBM + 4];
  __shared__ float Bs[NM][kTlBK][kTlBN + 4];
  __shared__ int32_t s_seg[4];  // eid, first row, rows, slot

  const int tid = threadIdx.x;
  const int bn = blockIdx.x % a.ntiles_n;
  const int bm_global = blockIdx.x / a.ntiles_n;

  // ---- find (segment, m-tile) ------------------------------------------------
  if (tid == 0) {
    int eid = -1, r0 = 0, M = 0, slot_id = 0;
    if (a.shared) {
      if (bm_global * kTlBM < a.T) {
        eid = 0;
        r0 = bm_global * kTlBM;
        M = min(kTlBM, a.T - r0);
      }
    } else {
      int nseg = a.segs.n;
      if (a.segs.eids_dev != nullptr) nseg = min(nseg, a.segs.count_dev[0]);
      int left = bm_global;
      for (int s = 0; s < nseg; ++s) {
        const int e = (a.segs.eids_dev != nullptr) ? a.segs.eids_dev[s] : a.segs.eids[s];
        const int b = a.seg_offsets[e], m = a.seg_offsets[e + 1] - b;
        const int nt = (m + kTlBM - 1) / kTlBM;
        if (left < nt) {
          eid = e;
          slot_id = (a.segs.eids_dev != nullptr) ? a.expert_slot[e] : a.segs.slots[s];
          r0 = b + left * kTlBM;
          M = min(kTlBM, m - left * kTlBM);
          break;
        }
        left -= nt;
      }
    }
    s_seg[0] = eid;
    s_seg[1] = r0;
    s_seg[2] = M;
    s_seg[3] = slot_id;
  }
  __syncthreads();
  const int eid = s_seg[0], r0 = s_seg[1], M = s_seg[2];
  if (eid < 0) return;

  const T* w0;
  const T* w1 = nullptr;
  if (a.shared) {
    w0 = static_cast<const T*>(a.w_s);
    w1 = static_cast<const T*>(a.w2_s);
  } else {
    const T* slot = static_cast<const T*>(a.slab) + static_cast<uint64_t>(s_seg[3]) * a.slot_stride;
    w0 = slot + a.mat_offset;
    w1 = slot + a.mat2_offset;
  }
  const int Kdim = a.Kdim, Ndim = a.Ndim;
  const int n0 = bn * kTlBN;

  // loader mapping: 64 rows x 16 k, four consecutive k per thread
  const int lrow = tid >> 2, lk = (tid & 3) * 4;
  const T* arow = nullptr;
  if (lrow < M) {
    const int p = r0 + lrow;
    if (a.shared) {
      arow = static_cast<const T*>(a.act) + static_cast<size_t>(p) * Kdim;
    } else if (kGateUp) {
      arow = static_cast<const T*>(a.act) + static_cast<size_t>(a.perm[p] / a.topk) * Kdim;
    } else {
      arow = static_cast<const T*>(a.act) + static_cast<size_t>(p) * Kdim;
    }
  }
  const bool brow_ok = (n0 + lrow) < Ndim;
  // weights are tiled: 16-row groups, blocks of 64 k, (half, k-quarter, row, 8 k) inside
  const int wrow = brow_ok ? n0 + lrow : 0;
  const size_t wbase = static_cast<size_t>(wrow >> 4) * 16 * Kdim + (wrow & 15) * 8;

  const int ty = tid >> 4, tx = tid & 15;
  float acc[NM][4][4];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[m][i][j] = 0.f;

  for (int k0 = 0; k0 < Kdim; k0 += kTlBK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      As[lk + j][lrow] = (arow != nullptr) ? Elem<T>::load(arow + k0 + lk + j) : 0.f;
      const int kk = k0 + lk + j;
      const size_t wo = wbase + static_cast<size_t>(kk >> 6) * 1024 + ((kk >> 3) & 1) * 512 +
                        ((kk >> 4) & 3) * 128 + (kk & 7);
      Bs[0][lk + j][lrow] = brow_ok ? Elem<T>::load(w0 + wo) : 0.f;
      if (kGateUp) Bs[1][lk + j][lrow] = brow_ok ? Elem<T>::load(w1 + wo) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kTlBK; ++kk) {
      float av[4], bv[NM][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j) bv[m][j] = Bs[m][kk][tx * 4 + j];
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[m][i][j] = fmaf(av[i], bv[m][j], acc[m][i][j]);
    }
    __syncthreads();
  }

  // ---- epilogue --------------------------------------------------------------
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = ty * 4 + i;
    if (m >= M) continue;
    const int p = r0 + m;
    float scale = 1.f;
    bool has_scale = false;
    if (!kGateUp) {
      if (a.shared) {
        if (a.gate_s != nullptr) {
          scale = Elem<T>::round(sigmoid_f32(Elem<T>::load(static_cast<const T*>(a.gate_s) + p)));
          has_scale = true;
        }
      } else {
        scale = Elem<T>::load(static_cast<const T*>(a.topv) + a.perm[p]);
        has_scale = true;
      }
    }
    T* orow = static_cast<T*>(a.out) + static_cast<size_t>(p) * Ndim;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= Ndim) continue;
      float v;
      if (kGateUp) {
        const float g = Elem<T>::round(acc[0][i][j]);
        const float u = Elem<T>::round(acc[1][i][j]);
        v = Elem<T>::round(silu_f32(g)) * u;
      } else {
        v = Elem<T>::round(acc[0][i][j]);
        if (has_scale) v = v * scale;
      }
      Elem<T>::store(orow + n, v);
    }
  }
}

template <typename T, bool kGateUp>
static int launch_tiled(TiledArgs& a, int max_mtiles, hipStream_t st) {
  a.ntiles_n = (a.Ndim + kTlBN - 1) / kTlBN;
  const int64_t grid = static_cast<int64_t>(a.ntiles_n) * max_mtiles;
  if (grid == 0) return SPARSE_HIP_OK;
  SP_REQUIRE(grid < (1ll << 31), "ffn_tiled: grid too large");
  ProfScope prof(kGateUp ? SPARSE_HIP_K_TILED_GATEUP : SPARSE_HIP_K_TILED_DOWN, st);
  hipLaunchKernelGGL((ffn_tiled_kernel<T, kGateUp>), dim3(static_cast<unsigned>(grid)), dim3(kTlThreads), 0,
                     st, a);
  SP_LAUNCH_CHECK("ffn_tiled_kernel");
  return SPARSE_HIP_OK;
}

template <typename T>
int tiled_routed(const sparse_hip_experts* ex, const void* x, const void* topv, const int32_t* perm,
                 const int32_t* seg_offsets, const sparse_hip_seglist* segs, int Ttok, int K, void* inter_ws,
                 void* parts, hipStream_t st) {
  const uint64_t H = ex->hidden, I = ex->inter;
  const int max_mtiles = (Ttok * K + kTlBM - 1) / kTlBM + segs->n;
  TiledArgs a = {};
  a.slab = ex->slab_dev;
  a.slot_stride = ex->slot_stride / sizeof(T);
  a.expert_slot = ex->expert_slot_dev;
  a.perm = perm;
  a.seg_offsets = seg_offsets;
  a.topk = K;
  a.T = Ttok;
  a.segs = *segs;
  a.mat_offset = 0;
  a.mat2_offset = I * H;
  a.act = x;
  a.out = inter_ws;
  a.Kdim = static_cast<int32_t>(H);
  a.Ndim = static_cast<int32_t>(I);
  int rc = launch_tiled<T, true>(a, max_mtiles, st);
  if (rc != SPARSE_HIP_OK) return rc;
  a.mat_offset = 2 * I * H;
  a.mat2_offset = 0;
  a.topv = topv;
  a.act = inter_ws;
  a.out = parts;
  a.Kdim = static_cast<int32_t>(I);
  a.Ndim = static_cast<int32_t>(H);
  return launch_tiled<T, false>(a, max_mtiles, st);
}

template <typename T>
int tiled_shared(const void* x, const void* gate_w, const void* up_w, const void* down_w,
                 const void* shared_gate, int Ttok, int H, int Is, void* inter_ws, void* shared_out,
                 hipStream_t st) {
  const int mtiles = (Ttok + kTlBM - 1) / kTlBM;
  TiledArgs a = {};
  a.shared = 1;
  a.T = Ttok;
  a.topk = 1;
  a.w_s = gate_w;
  a.w2_s = up_w;
  a.act = x;
  a.out = inter_ws;
  a.Kdim = H;
  a.Ndim = Is;
  int rc = launch_tiled<T, true>(a, mtiles, st);
  if (rc != SPARSE_HIP_OK) return rc;
  a.w_s = down_w;
  a.w2_s = nullptr;
  a.gate_s = shared_gate;
  a.act = inter_ws;
  a.out = shared_out;
  a.Kdim = Is;
  a.Ndim = H;
  return launch_tiled<T, false>(a, mtiles, st);
}

template int tiled_routed<float>(const sparse_hip_experts*, const void*, const void*, const int32_t*,
                                 const int32_t*, const sparse_hip_seglist*, int, int, void*, void*, hipStream_t);
template int tiled_routed<uint16_t>(const sparse_hip_experts*, const void*, const void*, const int32_t*,
                                    const int32_t*, const sparse_hip_seglist*, int, int, void*, void*,
                                    hipStream_t);
template int tiled_shared<float>(const void*, const void*, const void*, const void*, const void*, int, int, int,
                                 void*, void*, hipStream_t);
template int tiled_shared<uint16_t>(const void*, const void*, const void*, const void*, const void*, int, int,
                                    int, void*, void*, hipStream_t);

}  // namespace sparse
