// Decode-time grouped SwiGLU expert FFN (bf16): the HBM-bandwidth path.
//
// With at most 32 tokens per call every expert sees a handful of rows, so the FFN is a
// stream of weight rows past a tiny activation block.  A workgroup owns 32 output
// rows of one expert (two 16-row MFMA tiles) and all of the expert's tokens (one or
// two 16-token MFMA column tiles).  Weights go HBM -> registers in the MFMA A-operand
// layout with no LDS hop: lane (r, q) of a wave loads 32 contiguous bytes of row r at
// k = d*64 + q*16, so four lanes cover one 128-byte line of a row, the four waves of
// the workgroup cover four adjacent lines, and every line is consumed by two
// back-to-back loads.  The reduction dimension is split across the four waves
// (64-wide slices dealt round-robin); partial 16x16 tiles meet in LDS once, in a
// fixed order, and the epilogue (rounding, SiLU*up or *route-weight) runs there.
//
// MFMA 16x16x32 bf16 operand layout (lane l, r = l & 15, q = l >> 4):
//   A: row r, k = q*8 .. q*8+7      B: column r, k = q*8 .. q*8+7
//   D: column r, rows q*4 .. q*4+3
// A and B use the same k mapping, so any permutation of k inside a 64-wide slice
// applied to both leaves the product unchanged; the 32-byte-per-lane load relies on it.
#include "common.h"
#include <hip/hip_ext.h>

namespace sparse {

constexpr int kDecThreads = 256;
constexpr int kDecWaves = 4;
constexpr int kDecTilesMax = 2;                 // 16-row tiles per workgroup (the kernel also exists with 1)
constexpr int kDecRowsMax = kDecTilesMax * 16;  // output rows per workgroup
constexpr int kDecSplit = 4;                    // parts of the shared down projection's reduction

struct DecodeArgs {
  // routed experts
  const uint16_t* slab;         // slot 0
  uint64_t slot_stride;         // elements between slots
  uint64_t mat_offset;          // element offset of the (first) matrix inside a slot
  uint64_t mat2_offset;         // element offset of the second matrix (gate-up only)
  const int32_t* expert_slot;   // [E]
  const int32_t* perm;          // [T*K]
  const int32_t* seg_offsets;   // [E+1]
  const uint16_t* topv;         // [T*K] route weights (down only)
  const uint16_t* act_r;        // gate-up: x [T,Kdim]; down: inter [T*K,Kdim]
  uint16_t* out_r;              // gate-up: inter [T*K,Ndim]; down: parts [T*K,Ndim]
  int32_t topk;
  int32_t Kdim;                 // reduction length of the routed matrices
  int32_t Ndim;                 // output rows of the routed matrices
  int32_t tiles_r;              // Ndim / kDecRows
  // shared expert (tiles_s == 0 when absent)
  const uint16_t* w_s;          // first matrix [Ndim_s, Kdim_s]
  const uint16_t* w2_s;         // second matrix (gate-up only)
  const uint16_t* act_s;        // [T, Kdim_s]
  const uint16_t* gate_s;       // [T] shared gate logits or NULL (down only)
  uint16_t* out_s;              // [T, Ndim_s]
  int32_t Kdim_s;
  int32_t Ndim_s;
  int32_t tiles_s;
  int32_t T;
  int32_t fp16;                 // 16-bit format of every tensor: 0 bfloat16, 1 IEEE half
  // shared down projection with its reduction cut into `split_s` parts, one workgroup each
  // (1 = not cut): fp32 partial sums [split_s][T][Ndim_s], finished by the combine step
  int32_t split_s;
  float* split_sums;
  // combine folded into the down projection (needs split_s > 1): the workgroup that finishes a
  // 32-column tile last, counted per tile in `tile_counters`, sums that tile's columns of
  // every token over its K routed rows and the shared expert and writes `final_out`
  int32_t* tile_counters;       // [Ndim / kDecRows], zero when the launch starts; NULL: no combine here
  // gate/up launch of a call whose down launch combines: the counters to put to zero, so that the call
  // does not depend on what an earlier call (another token count on the same workspace, a launch that
  // did not finish) left there
  int32_t* clear_counters;
  int32_t n_clear;
  const int32_t* inv_perm;      // [T*K]
  uint16_t* final_out;          // [T, Ndim]
  sparse_hip_seglist segs;
};

// Results that another workgroup of the same launch reads travel as device-scope relaxed
// atomics: such a store is written through to memory instead of staying in the writer's
// L2 (each XCD has its own), such a load is served from memory instead of a stale line of the
// reader's L2.  No cache-wide write-back or invalidate is involved, which is what a
// release / acquire fence at device scope costs.
__device__ __forceinline__ void st_device_u64(void* p, uint64_t v) {
  __hip_atomic_store(reinterpret_cast<uint64_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t ld_device_u64(const void* p) {
  return __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ bf16x8 ld_bf16x8(const uint16_t* p) {
  return *reinterpret_cast<const bf16x8*>(p);
}
// Weights are read once per launch: a non-temporal load keeps them from displacing the
// activations and partial results in the caches on their way through.
__device__ __forceinline__ bf16x8 ld_stream_bf16x8(const uint16_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p));
}

// TL: 16-row tiles per workgroup (2, or 1 for launches whose grid would otherwise end in a thin last
// round of long-lived workgroups); a.tiles_r / a.tiles_s count workgroup tiles of TL * 16 rows.
template <typename F, bool kGateUp, int NT, int TL>
__global__ __launch_bounds__(kDecThreads) void decode_ffn_kernel(const DecodeArgs a) {
  constexpr int NM = kGateUp ? 2 : 1;
  constexpr int kDecTiles = TL, kDecRows = TL * 16;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  if (kGateUp && a.clear_counters != nullptr && blockIdx.x == 0)   // before any workgroup of this launch can return
    for (int i = threadIdx.x; i < a.n_clear; i += kDecThreads) a.clear_counters[i] = 0;

  // ---- which tile of which matrix ------------------------------------------
  const int split = kGateUp ? 1 : a.split_s;
  const bool is_shared = static_cast<int>(blockIdx.x) < a.tiles_s * split;
  const uint16_t *w0, *w1 = nullptr;
  int Kdim, Ndim, row0, M, r0 = 0;
  int tile_s = 0, part = 0, kbeg = 0, klen = 0;  // which part of the shared reduction (whole: part 0 of 1)
  if (is_shared) {
    Kdim = a.Kdim_s;
    Ndim = a.Ndim_s;
    tile_s = blockIdx.x / split;
    part = blockIdx.x - tile_s * split;
    row0 = tile_s * kDecRows;
    M = a.T;
    w0 = a.w_s;
    w1 = a.w2_s;
    klen = Kdim / split;
    kbeg = part * klen;
  } else {
    const int b = blockIdx.x - a.tiles_s * split;
    const int si = b / a.tiles_r;
    int eid, slot_id;
    if (a.segs.eids_dev != nullptr) {
      const int cnt = min(a.segs.count_dev[0], a.segs.n);
      if (si >= cnt) return;
      eid = a.segs.eids_dev[si];
      slot_id = a.expert_slot[eid];
    } else {
      if (si >= a.segs.n) return;
      eid = a.segs.eids[si];
      slot_id = a.segs.slots[si];
    }
    Kdim = a.Kdim;
    Ndim = a.Ndim;
    klen = Kdim;
    row0 = (b - si * a.tiles_r) * kDecRows;
    r0 = a.seg_offsets[eid];
    M = a.seg_offsets[eid + 1] - r0;
    if (M <= 0 && (kGateUp || a.tile_counters == nullptr)) return;  // (an empty segment still counts as arrived)
    const uint16_t* slot = a.slab + static_cast<uint64_t>(slot_id) * a.slot_stride;
    w0 = slot + a.mat_offset;
    w1 = slot + a.mat2_offset;
  }

  // ---- B operand rows (activations) ----------------------------------------
  const uint16_t* brow[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = r + 16 * nt;
    brow[nt] = nullptr;
    if (n < M) {
      if (is_shared) {
        brow[nt] = a.act_s + static_cast<size_t>(n) * Kdim + kbeg;
      } else if (kGateUp) {
        brow[nt] = a.act_r + static_cast<size_t>(a.perm[r0 + n] / a.topk) * Kdim;
      } else {
        brow[nt] = a.act_r + static_cast<size_t>(r0 + n) * Kdim;
      }
    }
  }

  f32x4 acc[NM][kDecTiles][NT];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int tl = 0; tl < kDecTiles; ++tl)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[m][tl][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Weights are tiled: the K extent of a 16-row group is contiguous, cut into 2 KB blocks
  // of 64 k; the first KB of a block is the first MFMA's A operand in lane order, the
  // second KB the second MFMA's, so every load instruction of a wave reads 1 KB straight.
  const size_t group_stride = static_cast<size_t>(16) * Kdim;
  const size_t kskip = static_cast<size_t>(kbeg >> 6) << 10;  // 64-wide blocks before this part, 1 K elements each
  const uint16_t* wt0 = w0 + static_cast<size_t>(row0 >> 4) * group_stride + kskip + lane * 8;
  const uint16_t* wt1 = kGateUp ? w1 + static_cast<size_t>(row0 >> 4) * group_stride + lane * 8 : nullptr;
  const int ND = klen >> 6;

  // Two register stages per wavefront, used in turn: while one slice is multiplied the next
  // one is already in flight and the one after that is requested as soon as its stage is
  // free.  The steady-state loop below has no branches, so the wait before each batch of
  // MFMAs counts exactly the newer stage's loads as still outstanding; a conditional load
  // inside the loop would make every wait a full drain and leave one slice in flight.
  bf16x8 b0[NT][2], w0s[NM][kDecTiles][2];
  bf16x8 b1[NT][2], w1s[NM][kDecTiles][2];

  // token columns past the segment read the block's first activation row (always mapped):
  // their products land in output columns the epilogue never stores, so they need neither a
  // branch around the loads nor a mask
  const uint16_t* bsafe = is_shared ? a.act_s + kbeg : a.act_r;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    if (brow[nt] == nullptr) brow[nt] = bsafe;

// (weights first: their addresses need the segment's slot only, the token rows' addresses wait for the
// permutation entry as well, and the first weight loads should be in flight while that arrives)
#define SP_DEC_LOAD(B, W, d)                                                             \
  do {                                                                                   \
    const int koff_ = (d) << 6;                                                          \
    _Pragma("unroll") for (int tl = 0; tl < kDecTiles; ++tl) {                           \
      const size_t o_ = tl * group_stride + (static_cast<size_t>(d) << 10);              \
      W[0][tl][0] = ld_stream_bf16x8(wt0 + o_);                                                 \
      W[0][tl][1] = ld_stream_bf16x8(wt0 + o_ + 512);                                           \
      if (kGateUp) {                                                                     \
        W[NM - 1][tl][0] = ld_stream_bf16x8(wt1 + o_);                                          \
        W[NM - 1][tl][1] = ld_stream_bf16x8(wt1 + o_ + 512);                                    \
      }                                                                                  \
    }                                                                                    \
    _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) {                                  \
      B[nt][0] = ld_bf16x8(brow[nt] + koff_ + (q << 4));                                 \
      B[nt][1] = ld_bf16x8(brow[nt] + koff_ + (q << 4) + 8);                             \
    }                                                                                    \
  } while (0)

#define SP_DEC_MFMA(B, W)                                                                                   \
  do {                                                                                                      \
    _Pragma("unroll") for (int tl = 0; tl < kDecTiles; ++tl)                                                \
    _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                                       \
    _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                                        \
      acc[m][tl][nt] = F::mfma16(W[m][tl][0], B[nt][0], acc[m][tl][nt]);                                \
      acc[m][tl][nt] = F::mfma16(W[m][tl][1], B[nt][1], acc[m][tl][nt]);                                \
    }                                                                                                       \
  } while (0)

  // slice number i of this wavefront is 64-wide slice wave + i * kDecWaves of the reduction
  const int n = (ND - wave + kDecWaves - 1) / kDecWaves;
#define SP_DEC_SLICE(i) (wave + (i) * kDecWaves)
  int i = 0;
  // the first two loads are unconditional (a wavefront with fewer slices re-reads the last
  // valid one and never multiplies it): a branch around them would merge two different
  // outstanding-load states at the loop's entry and turn the loop's waits into full drains
  SP_DEC_LOAD(b0, w0s, min(SP_DEC_SLICE(0), ND - 1));
  SP_DEC_LOAD(b1, w1s, min(SP_DEC_SLICE(1), ND - 1));
  for (; i + 4 <= n; i += 2) {
    // fences keep the scheduler from sinking a stage's reload below the other stage's MFMAs
    SP_DEC_MFMA(b0, w0s);
    __builtin_amdgcn_sched_barrier(0);
    SP_DEC_LOAD(b0, w0s, SP_DEC_SLICE(i + 2));
    __builtin_amdgcn_sched_barrier(0);
    SP_DEC_MFMA(b1, w1s);
    __builtin_amdgcn_sched_barrier(0);
    SP_DEC_LOAD(b1, w1s, SP_DEC_SLICE(i + 3));
    __builtin_amdgcn_sched_barrier(0);
  }
  // up to three slices left; stage 0 holds slice i, stage 1 slice i + 1
  if (i < n) {
    SP_DEC_MFMA(b0, w0s);
    if (i + 2 < n) SP_DEC_LOAD(b0, w0s, SP_DEC_SLICE(i + 2));
  }
  if (i + 1 < n) SP_DEC_MFMA(b1, w1s);
  if (i + 2 < n) SP_DEC_MFMA(b0, w0s);
#undef SP_DEC_SLICE
#undef SP_DEC_MFMA
#undef SP_DEC_LOAD

  // A launch that also combines: where each token's K routed rows lie is asked for now, so that the answer
  // is there long before the hand-off needs it (thread -> (token, four columns) of the 32-column tile).
  constexpr int kPerTok = kDecRows / 4;   // threads per token in the combine: four columns each
  const int ct = threadIdx.x / kPerTok, cc4 = (threadIdx.x % kPerTok) * 4;
  int32_t pos[SPARSE_HIP_MAX_TOPK];
  if (!kGateUp && a.tile_counters != nullptr) {
#pragma unroll
    for (int k = 0; k < SPARSE_HIP_MAX_TOPK; ++k)
      pos[k] = (k < a.topk && ct < a.T) ? a.inv_perm[ct * a.topk + k] : 0x7fffffff;
  }

  // ---- split-K partials meet in LDS ----------------------------------------
  constexpr int NFRAG = kDecTiles * NT;
  __shared__ f32x4 red[kDecWaves][NFRAG * NM][64];
#pragma unroll
  for (int tl = 0; tl < kDecTiles; ++tl)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int m = 0; m < NM; ++m) red[wave][(tl * NT + nt) * NM + m][lane] = acc[m][tl][nt];
  __syncthreads();

  // one fragment of the tile: rows row0 + 16 tl + 4 q .. + 3 of token column n, as fp32 sums
  auto emit = [&](int tl, int n, const f32x4& s0, const f32x4& s1) {
    const int orow = row0 + tl * 16 + q * 4;
    float scale = 1.f;
    bool has_scale = false;
    if (!kGateUp) {
      if (is_shared) {
        if (a.gate_s != nullptr) {
          scale = F::round(sigmoid_f32(F::from_bits(a.gate_s[n])));
          has_scale = true;
        }
      } else {
        scale = F::from_bits(a.topv[a.perm[r0 + n]]);
        has_scale = true;
      }
    }
    uint16_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v;
      if (kGateUp) {
        const float g = F::round(s0[j]);
        const float u = F::round(s1[j]);
        v = F::round(silu_f32(g)) * u;
      } else {
        v = F::round(s0[j]);
        if (has_scale) v = v * scale;
      }
      o[j] = F::bits(v);
    }
    uint16_t* dst = is_shared ? a.out_s + static_cast<size_t>(n) * Ndim + orow
                              : a.out_r + static_cast<size_t>(r0 + n) * Ndim + orow;
    uint2 pk;
    pk.x = static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16);
    pk.y = static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16);
    if (!kGateUp && a.tile_counters != nullptr) {
      st_device_u64(dst, static_cast<uint64_t>(pk.x) | (static_cast<uint64_t>(pk.y) << 32));
    } else {
      *reinterpret_cast<uint2*>(dst) = pk;
    }
  };
  const bool fuse = !kGateUp && a.tile_counters != nullptr;

  if (!kGateUp && is_shared && split > 1) {
    // A part of a shared tile: its fp32 sums go to memory as they are; the combine step adds
    // the parts in their order, rounds, applies the shared gate and adds the result in.
    const size_t part_stride = static_cast<size_t>(a.T) * Ndim;
    for (int f = wave; f < NFRAG; f += kDecWaves) {
      const int tl = f / NT, nt = f - tl * NT;
      const int n = r + 16 * nt;
      if (n >= M) continue;
      f32x4 s0 = red[0][f][lane];
#pragma unroll
      for (int w = 1; w < kDecWaves; ++w) s0 += red[w][f][lane];
      float* dst = a.split_sums + part * part_stride + static_cast<size_t>(n) * Ndim + row0 + tl * 16 + q * 4;
      if (fuse) {
        st_device_u64(dst, static_cast<uint64_t>(__float_as_uint(s0[0])) | (static_cast<uint64_t>(__float_as_uint(s0[1])) << 32));
        st_device_u64(dst + 2, static_cast<uint64_t>(__float_as_uint(s0[2])) | (static_cast<uint64_t>(__float_as_uint(s0[3])) << 32));
      } else {
        *reinterpret_cast<f32x4*>(dst) = s0;
      }
    }
    if (!fuse) return;
  } else {
    for (int f = wave; f < NFRAG; f += kDecWaves) {
      const int tl = f / NT, nt = f - tl * NT;
      const int n = r + 16 * nt;
      if (n >= M) continue;
      f32x4 s0 = red[0][f * NM][lane];
      f32x4 s1 = kGateUp ? red[0][f * NM + 1][lane] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 1; w < kDecWaves; ++w) {
        s0 += red[w][f * NM][lane];
        if (kGateUp) s1 += red[w][f * NM + 1][lane];
      }
      emit(tl, n, s0, s1);
    }
  }

  if constexpr (!kGateUp) {
    if (!fuse) return;
    // ---- combine, by the workgroup that finishes this 32-column tile last ----------------
    // Every workgroup of the tile (one per active routed segment, `split` for the shared
    // expert) has written its rows through to memory; once its own writes are acknowledged it
    // counts itself in.  The last one finds everybody's rows in memory.
    __shared__ int s_last;
    // thread -> (token, four columns); the arithmetic is that of the stand-alone combine step:
    // K ordered adds rounded to bf16, then the shared expert finished from its parts.  Where the
    // token's rows lie was asked for before the reduction.
    const int Ttok = a.T, K = a.topk, H = a.Ndim_s;
    const int t = ct, c4 = cc4;
    // how many workgroups this tile has: read now, not between the barrier and the counter
    const int arrivals = ((a.segs.eids_dev != nullptr) ? min(a.segs.count_dev[0], a.segs.n) : a.segs.n) + split;
    // ascending row position = ascending expert id: the order of the stand-alone combine's adds.  Sorted
    // here, while this wavefront's stores are still on their way, by every workgroup: the one that turns out
    // to be last then has nothing left to do between the counter and its reads.
#pragma unroll
    for (int i = 1; i < SPARSE_HIP_MAX_TOPK; ++i) {
#pragma unroll
      for (int j = i; j > 0; --j) {
        const int32_t lo = min(pos[j - 1], pos[j]), hi = max(pos[j - 1], pos[j]);
        pos[j - 1] = lo;
        pos[j] = hi;
      }
    }
    __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);  // this wavefront's stores have been acknowledged
    __syncthreads();
    const int tile = row0 / kDecRows;
    if (threadIdx.x == 0) {
      const int prev = __hip_atomic_fetch_add(a.tile_counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = (prev == arrivals - 1);
      if (s_last) __hip_atomic_store(a.tile_counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    if (t >= Ttok) return;
    const int h = row0 + c4;
    // Every read is requested before the first one is consumed: the loads are ordered atomics, which the
    // compiler neither hoists nor overlaps with the additions that use them, so written row by row each
    // would cost its own trip to memory.  Rows past K and parts past `split` repeat the first address and
    // are not used.
    const size_t part_stride = static_cast<size_t>(Ttok) * H;
    const float* src = a.split_sums + static_cast<size_t>(t) * H + h;
    uint64_t part_lo[kDecSplit], part_hi[kDecSplit];
#pragma unroll
    for (int p = 0; p < kDecSplit; ++p) {
      const float* s = src + static_cast<size_t>(p < split ? p : 0) * part_stride;
      part_lo[p] = ld_device_u64(s);
      part_hi[p] = ld_device_u64(s + 2);
    }
    constexpr int kRowGroup = 8;
    static_assert(SPARSE_HIP_MAX_TOPK % kRowGroup == 0, "row groups must cover the top-k limit");
    float accv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < SPARSE_HIP_MAX_TOPK; g += kRowGroup) {
      if (g == 0 || g < K) {          // uniform: K is a launch argument
        uint64_t v[kRowGroup];
#pragma unroll
        for (int i = 0; i < kRowGroup; ++i) {
          const int32_t p = (g + i < K) ? pos[g + i] : pos[0];
          v[i] = ld_device_u64(a.out_r + static_cast<size_t>(p) * H + h);
        }
#pragma unroll
        for (int i = 0; i < kRowGroup; ++i) {
          if (g + i < K) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              accv[j] = F::round(accv[j] + F::from_bits(static_cast<uint16_t>(v[i] >> (16 * j))));
          }
        }
      }
    }
    float sh[4];
#pragma unroll
    for (int p = 0; p < kDecSplit; ++p) {
      if (p < split) {
        const float f0 = __uint_as_float(static_cast<uint32_t>(part_lo[p]));
        const float f1 = __uint_as_float(static_cast<uint32_t>(part_lo[p] >> 32));
        const float f2 = __uint_as_float(static_cast<uint32_t>(part_hi[p]));
        const float f3 = __uint_as_float(static_cast<uint32_t>(part_hi[p] >> 32));
        if (p == 0) {
          sh[0] = f0; sh[1] = f1; sh[2] = f2; sh[3] = f3;
        } else {
          sh[0] += f0; sh[1] += f1; sh[2] += f2; sh[3] += f3;
        }
      }
    }
    const bool gated = a.gate_s != nullptr;
    const float scale = gated ? F::round(sigmoid_f32(F::from_bits(a.gate_s[t]))) : 1.f;
    uint16_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v = F::round(sh[j]);
      if (gated) v = v * scale;
      o[j] = F::bits(accv[j] + F::round(v));
    }
    uint2 pk;
    pk.x = static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16);
    pk.y = static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16);
    *reinterpret_cast<uint2*>(a.final_out + static_cast<size_t>(t) * H + h) = pk;
  }
}

__global__ void decode_clear_kernel(int32_t* p, int n) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) p[i] = 0;
}

template <bool kGateUp>
static int launch_decode(const DecodeArgs& a0, int n_seg, hipStream_t st) {
  // A gate/up launch of up to 16 tokens whose 32-row workgroups would not all be resident at once (four
  // per compute unit, 256 units) runs with 16-row workgroups instead: twice as many, half as long-lived,
  // so the launch does not end on a thin last round of workgroups that started late (2.19 -> 2.17 ms per
  // batch-8 step).  A grid that fits keeps the wide form, which is the faster one there (batch 1).  Every
  // output row is computed by the same instructions either way.
  constexpr int kResidentWide = 4 * 256;
  // (the down projection's launch, tried the same way, gets slower, 2.21 against 2.18 ms per step; with
  // 64-row workgroups its own time drops by 1.5 us and the step time does not move)
  const bool narrow = kGateUp && a0.T <= 16 && a0.tiles_s + n_seg * a0.tiles_r > kResidentWide;
  DecodeArgs a = a0;
  if (narrow) {
    a.tiles_r *= kDecTilesMax;
    a.tiles_s *= kDecTilesMax;
  }
  const int grid = a.tiles_s * (kGateUp ? 1 : a.split_s) + n_seg * a.tiles_r;
  if (grid == 0) {
    if (kGateUp && a.clear_counters != nullptr) {   // nothing to project, but the counters are still this launch's job
      hipLaunchKernelGGL(decode_clear_kernel, dim3(1), dim3(256), 0, st, a.clear_counters, a.n_clear);
      SP_LAUNCH_CHECK("decode_clear_kernel");
    }
    return SPARSE_HIP_OK;
  }
  ProfScope prof(kGateUp ? SPARSE_HIP_K_DECODE_GATEUP : SPARSE_HIP_K_DECODE_DOWN, st, /*dispatch_events=*/true);
#define SP_DEC_LAUNCH(F, NT, TL)                                                                              \
  do {                                                                                                       \
    if (prof.active()) { /* profiling: the launch stamps the event pair with the dispatch's begin and end */ \
      hipExtLaunchKernelGGL((decode_ffn_kernel<F, kGateUp, NT, TL>), dim3(grid), dim3(kDecThreads), 0, st,   \
                            prof.start_, prof.stop_, 0, a);                                                  \
    } else {                                                                                                 \
      hipLaunchKernelGGL((decode_ffn_kernel<F, kGateUp, NT, TL>), dim3(grid), dim3(kDecThreads), 0, st, a);  \
    }                                                                                                        \
  } while (0)
  if (a.fp16) {
    if (narrow) SP_DEC_LAUNCH(Fp16, 1, 1); else if (a.T <= 16) SP_DEC_LAUNCH(Fp16, 1, 2); else SP_DEC_LAUNCH(Fp16, 2, 2);
  } else {
    if (narrow) SP_DEC_LAUNCH(Bf16, 1, 1); else if (a.T <= 16) SP_DEC_LAUNCH(Bf16, 1, 2); else SP_DEC_LAUNCH(Bf16, 2, 2);
  }
#undef SP_DEC_LAUNCH
  SP_LAUNCH_CHECK("decode_ffn_kernel");
  return SPARSE_HIP_OK;
}

// Routed experts, 16-bit formats (the slab's dtype picks bfloat16 or IEEE half).  Two launches: gate-up into inter_ws, down into parts.
int decode_routed_bf16(const sparse_hip_experts* ex, const void* x, const void* topv, const int32_t* perm,
                       const int32_t* seg_offsets, const sparse_hip_seglist* segs, int T, int K,
                       void* inter_ws, void* parts, hipStream_t st) {
  const uint64_t H = ex->hidden, I = ex->inter;
  DecodeArgs a = {};
  a.fp16 = ex->dtype == SPARSE_HIP_F16;
  a.split_s = 1;
  a.slab = static_cast<const uint16_t*>(ex->slab_dev);
  a.slot_stride = ex->slot_stride / 2;
  a.expert_slot = ex->expert_slot_dev;
  a.perm = perm;
  a.seg_offsets = seg_offsets;
  a.topk = K;
  a.T = T;
  a.segs = *segs;
  // gate-up
  a.mat_offset = 0;
  a.mat2_offset = I * H;
  a.act_r = static_cast<const uint16_t*>(x);
  a.out_r = static_cast<uint16_t*>(inter_ws);
  a.Kdim = static_cast<int32_t>(H);
  a.Ndim = static_cast<int32_t>(I);
  a.tiles_r = a.Ndim / kDecRowsMax;
  int rc = launch_decode<true>(a, segs->n, st);
  if (rc != SPARSE_HIP_OK) return rc;
  // down
  a.mat_offset = 2 * I * H;
  a.mat2_offset = 0;
  a.topv = static_cast<const uint16_t*>(topv);
  a.act_r = static_cast<const uint16_t*>(inter_ws);
  a.out_r = static_cast<uint16_t*>(parts);
  a.Kdim = static_cast<int32_t>(I);
  a.Ndim = static_cast<int32_t>(H);
  a.tiles_r = a.Ndim / kDecRowsMax;
  return launch_decode<false>(a, segs->n, st);
}

size_t decode_split_counter_offset(int T, int H);

// Routed experts and the shared expert in one launch pair, 16-bit formats, T <= 32.  The shared
// expert's tiles lead the grid (largest, known amount of work), routed segments follow.
int decode_fused_bf16(const sparse_hip_experts* ex, const void* x, const void* topv, const int32_t* perm,
                      const int32_t* seg_offsets, const sparse_hip_seglist* segs, int T, int K, void* inter_ws,
                      void* parts, const void* sh_gate_w, const void* sh_up_w, const void* sh_down_w,
                      const void* shared_gate, int Is, void* sh_inter_ws, void* shared_out, void* split_ws,
                      const int32_t* inv_perm, void* final_out, hipStream_t st) {
  const uint64_t H = ex->hidden, I = ex->inter;
  DecodeArgs a = {};
  a.fp16 = ex->dtype == SPARSE_HIP_F16;
  a.split_s = 1;
  a.slab = static_cast<const uint16_t*>(ex->slab_dev);
  a.slot_stride = ex->slot_stride / 2;
  a.expert_slot = ex->expert_slot_dev;
  a.perm = perm;
  a.seg_offsets = seg_offsets;
  a.topk = K;
  a.T = T;
  a.segs = *segs;
  // gate-up
  a.mat_offset = 0;
  a.mat2_offset = I * H;
  a.act_r = static_cast<const uint16_t*>(x);
  a.out_r = static_cast<uint16_t*>(inter_ws);
  a.Kdim = static_cast<int32_t>(H);
  a.Ndim = static_cast<int32_t>(I);
  a.tiles_r = a.Ndim / kDecRowsMax;
  a.w_s = static_cast<const uint16_t*>(sh_gate_w);
  a.w2_s = static_cast<const uint16_t*>(sh_up_w);
  a.act_s = static_cast<const uint16_t*>(x);
  a.out_s = static_cast<uint16_t*>(sh_inter_ws);
  a.Kdim_s = static_cast<int32_t>(H);
  a.Ndim_s = Is;
  // no gate / up matrices: sh_inter_ws already holds the shared expert's SiLU(gate x) * (up x)
  a.tiles_s = sh_gate_w != nullptr ? Is / kDecRowsMax : 0;
  const bool split = split_ws != nullptr && (Is / 64) % kDecSplit == 0;
  if (split && final_out != nullptr) {   // the down launch below combines: its arrival counters start at zero
    a.clear_counters = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(split_ws) + decode_split_counter_offset(T, static_cast<int>(H)));
    a.n_clear = (static_cast<int>(H) + 15) / 16;
  }
  int rc = launch_decode<true>(a, segs->n, st);
  if (rc != SPARSE_HIP_OK) return rc;
  a.clear_counters = nullptr;
  // down
  a.mat_offset = 2 * I * H;
  a.mat2_offset = 0;
  a.topv = static_cast<const uint16_t*>(topv);
  a.act_r = static_cast<const uint16_t*>(inter_ws);
  a.out_r = static_cast<uint16_t*>(parts);
  a.Kdim = static_cast<int32_t>(I);
  a.Ndim = static_cast<int32_t>(H);
  a.tiles_r = a.Ndim / kDecRowsMax;
  a.w_s = static_cast<const uint16_t*>(sh_down_w);
  a.w2_s = nullptr;
  a.act_s = static_cast<const uint16_t*>(sh_inter_ws);
  a.gate_s = static_cast<const uint16_t*>(shared_gate);
  a.out_s = static_cast<uint16_t*>(shared_out);
  a.Kdim_s = Is;
  a.Ndim_s = static_cast<int32_t>(H);
  a.tiles_s = a.Ndim_s / kDecRowsMax;
  // The shared down projection reduces over Is, several times the routed experts' I: as one
  // workgroup per tile it would still be streaming when everything else has finished.  With a
  // workspace it is cut into kDecSplit parts whose fp32 sums the combine step adds up.
  if (split) {
    a.split_s = kDecSplit;
    a.split_sums = static_cast<float*>(split_ws);
    if (final_out != nullptr) {  // the per-tile arrival counters follow the partial sums in the workspace
      a.tile_counters = reinterpret_cast<int32_t*>(static_cast<float*>(split_ws) + static_cast<size_t>(kDecSplit) * T * H);
      a.inv_perm = inv_perm;
      a.final_out = static_cast<uint16_t*>(final_out);
    }
  }
  return launch_decode<false>(a, segs->n, st);
}

// fp32 partial sums [kDecSplit][T][H], then one int32 arrival counter per 32-column tile
size_t decode_split_ws_bytes(int T, int H) {
  return static_cast<size_t>(kDecSplit) * T * H * sizeof(float) + static_cast<size_t>((H + 15) / 16) * sizeof(int32_t);   // one per 16-column tile, the narrowest form
}
size_t decode_split_counter_offset(int T, int H) { return static_cast<size_t>(kDecSplit) * T * H * sizeof(float); }
int decode_split_parts(int Is) { return (Is / 64) % kDecSplit == 0 ? kDecSplit : 1; }

// Shared expert, 16-bit formats, T <= 32.
int decode_shared_bf16(const void* x, const void* gate_w, const void* up_w, const void* down_w,
                       const void* shared_gate, int dtype, int T, int H, int Is, void* inter_ws, void* shared_out,
                       hipStream_t st) {
  DecodeArgs a = {};
  a.fp16 = dtype == SPARSE_HIP_F16;
  a.split_s = 1;
  a.T = T;
  a.topk = 1;
  a.tiles_r = 1;
  a.w_s = static_cast<const uint16_t*>(gate_w);
  a.w2_s = static_cast<const uint16_t*>(up_w);
  a.act_s = static_cast<const uint16_t*>(x);
  a.out_s = static_cast<uint16_t*>(inter_ws);
  a.Kdim_s = H;
  a.Ndim_s = Is;
  a.tiles_s = Is / kDecRowsMax;
  if (gate_w != nullptr) {  // else inter_ws already holds SiLU(gate x) * (up x)
    int rc = launch_decode<true>(a, 0, st);
    if (rc != SPARSE_HIP_OK) return rc;
  }
  a.w_s = static_cast<const uint16_t*>(down_w);
  a.w2_s = nullptr;
  a.act_s = static_cast<const uint16_t*>(inter_ws);
  a.gate_s = static_cast<const uint16_t*>(shared_gate);
  a.out_s = static_cast<uint16_t*>(shared_out);
  a.Kdim_s = Is;
  a.Ndim_s = H;
  a.tiles_s = H / kDecRowsMax;
  return launch_decode<false>(a, 0, st);
}

}  // namespace sparse
