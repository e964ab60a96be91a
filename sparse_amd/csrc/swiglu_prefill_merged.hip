// Prefill-time SwiGLU FFN of a whole layer call, routed experts and shared expert together, as two
// launches (all gate/up projections, then all down projections).
//
// The tile arithmetic is that of swiglu_prefill.hip: a workgroup (4 wavefronts) computes a 128-row x
// 256-weight-row tile with 16x16x32 MFMAs, activation rows through a three-buffer LDS ring (direct
// global -> LDS copies, chunks swizzled by row), weight fragments straight from the tiled layout into
// two alternating register sets, every operand requested two 64-wide k slabs ahead, vector-memory
// completion awaited by count.  Results are bit-identical to that kernel's.
//
// What differs is the tile list.  The tiles of the routed segments and of the shared expert sit in
// eight queues, one per XCD (workgroup b runs on XCD b % 8 and takes entry b / 8 of that queue): each
// queue holds a contiguous share of the shared expert's tiles (column tile, row tile) and a contiguous
// share of the routed tiles in the order (expert, column tile, row tile), so the row tiles of one weight
// tile run on one XCD close in time and the weight tile is read from HBM once.  One launch per
// projection instead of two means one tail of half-empty compute units instead of two, and the shared
// expert's dense tiles fill what the ragged routed segments leave.
//
// Operand addresses: everything that does not depend on the lane sits in scalar registers, a lane adds
// a 32-bit byte offset of its own.
#include <atomic>
#include <type_traits>

#include "common.h"
#include "prefill_tiles.h"

namespace sparse {

struct PfxArgs {
  // routed operand set
  const uint16_t* slab;
  uint64_t slot_stride;   // elements
  uint64_t mat_offset;    // elements: gate (gate/up launch) or down matrix inside a slot
  uint64_t mat2_offset;   // elements: up matrix inside a slot
  const int32_t* perm;
  const uint16_t* topv;
  const uint16_t* act_r;
  uint16_t* out_r;
  int32_t topk;
  uint32_t topk_magic;    // ceil(2^32 / topk); 0 for topk == 1
  int32_t Kdim_r, Ndim_r;
  // shared operand set
  int32_t Kdim_s, Ndim_s;
  const uint16_t* w_s;
  const uint16_t* w2_s;
  const uint16_t* gate_s;
  const uint16_t* act_s;
  uint16_t* out_s;
  // queues of this launch
  const PfTile* map;     // entry 0 is an idle entry
  const int32_t* qhdr;   // [0..7] first map entry of queue x, [8..15] entries in it
  unsigned long long* clk;
};

// A pointer every lane holds the same value of, moved to scalar registers.
template <typename T>
__device__ __forceinline__ T* pfx_uniform(T* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
  return reinterpret_cast<T*>((static_cast<uint64_t>(hi) << 32) | lo);
}

// kDrainWaits replaces the counted vector-memory waits of the k loop by full drains: slower, and
// correct whatever else the compiler has in flight.  Both variants must give the same bits.
template <typename F, bool kGateUp, bool kDrainWaits>
__global__ __launch_bounds__(kPfThreads, 2) void prefill_merged_kernel(const PfxArgs a) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kPfStages][kPfLdsA];
  __shared__ float s_scale[kPfBM];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int fr = lane & 15, fq = lane >> 4;
  const long long clk_c0 = clock64();
  const unsigned long long clk_t0 = wall_clock64();
  const int xcd = blockIdx.x % kPfXcds;

  // s_waitcnt vmcnt(n), other counters untouched
  constexpr int kWaitVm0 = kWaitVmcnt0, kWaitVm20 = kDrainWaits ? kWaitVmcnt0 : kWaitVmcnt20;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) uint8_t*)(&lds[0][0])));

  // ---- which tile (wavefront-uniform) ------------------------------------------------
  const int rank = blockIdx.x / kPfXcds;
  if (rank >= a.qhdr[kPfXcds + xcd]) return;   // the grid is sized for the longest possible queue
  const PfTile tile = a.map[a.qhdr[xcd] + rank];
  const int slot = __builtin_amdgcn_readfirstlane(tile.slot), r0 = __builtin_amdgcn_readfirstlane(tile.r0);
  const int M = __builtin_amdgcn_readfirstlane(tile.rows), bn = __builtin_amdgcn_readfirstlane(tile.bn);
  if (M <= 0) return;
  const bool shared = slot < 0;
  const int Kdim = shared ? a.Kdim_s : a.Kdim_r, Ndim = shared ? a.Ndim_s : a.Ndim_r;
  const int nk = Kdim / kPfBK;
  uint16_t* out = shared ? a.out_s : a.out_r;
  const int n0 = bn * (kGateUp ? kPfBR / 2 : kPfBR);   // first output column of this tile

  // ---- operand addresses ------------------------------------------------------------
  // Which 16-byte piece of its row a lane copies: row r keeps chunk 2q + h at position (q + 4h) ^ f(r),
  // f(r) = ((r >> 1) & 7) ^ ((r & 1) << 2), and the lane that lands at position `pos` fetches the chunk
  // that belongs there.  With r = 32 wave + 8 it + (lane >> 3), f depends on `it` only through its low
  // bit, which flips bit 2 of the position, i.e. bit 0 of the chunk.
  const int l3 = lane >> 3;
  const int pos0 = (lane & 7) ^ ((l3 >> 1) ^ ((l3 & 1) << 2));
  const uint32_t chunk0 = ((pos0 & 3) << 1) | (pos0 >> 2);
  const uint16_t* abase = pfx_uniform(shared ? a.act_s : a.act_r);
  uint32_t doff[4];   // byte offset of lane's piece of copy `it` inside k slab 0
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int p = r0 + min(wave * 32 + it * 8 + l3, M - 1);
    // gate/up of a routed tile gathers token rows through the permutation (flat index / K: a multiply
    // by ceil(2^32 / K), exact below 2^32 / K); everything else reads its own permuted row
    uint32_t grow = static_cast<uint32_t>(p);
    if (kGateUp && !shared) {
      grow = static_cast<uint32_t>(a.perm[p]);
      if (a.topk_magic != 0) grow = __umulhi(grow, a.topk_magic);
    }
    doff[it] = (grow * static_cast<uint32_t>(Kdim) + ((chunk0 ^ (it & 1)) << 3)) * 2u;
  }
  // Issued as inline assembly: the compiler would otherwise make every barrier wait for all
  // outstanding vector memory operations because one of them writes LDS.
  auto stage_slab = [&](int slab, int buf) {
    const uint16_t* sb = abase + slab * kPfBK;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + buf * kPfLdsA + (wave * 4 + it) * 1024);
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(doff[it]), "s"(sb), "s"(dst)
                   : "memory", "m0");
    }
  };
  // The wavefront's 64 weight rows are four 16-row groups; in the tiled layout a group's 64-wide slab is
  // 2 KB: the first KB is the A operand of the MFMA over its k half 0 in lane order, the second KB that of
  // half 1.  Gate/up: groups 0, 1 are gate rows of 32 neurons, groups 2, 3 the up rows of the same neurons.
  const uint16_t* wbase[4];          // first fragment of 16-row group g (lane 0)
  const uint32_t woff = lane * 16;   // a wavefront load of a fragment is 1 KB in lane order
  {
    const uint16_t *w0, *w1;
    if (shared) {
      w0 = a.w_s;
      w1 = a.w2_s;
    } else {
      const uint16_t* base = a.slab + static_cast<uint64_t>(slot) * a.slot_stride;
      w0 = base + a.mat_offset;
      w1 = base + a.mat2_offset;
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint16_t* base = (kGateUp && g >= 2) ? w1 : w0;
      int n = kGateUp ? (n0 + wave * 32 + (g & 1) * 16) : (n0 + wave * 64 + g * 16);
      n = min(n, Ndim - 16);
      wbase[g] = pfx_uniform(base + static_cast<size_t>(n >> 4) * 16 * Kdim);
    }
  }
  // (the pointer comes out of scalar registers as an integer: say that it is global memory, or the load
  // becomes a flat one, which also counts as an LDS operation)
  typedef const __attribute__((address_space(1))) char* gptr_t;
  auto wload = [&](int g, int slab, int h) __attribute__((always_inline)) {
    gptr_t p = (gptr_t)(reinterpret_cast<uintptr_t>(wbase[g]) + static_cast<size_t>(slab) * 2048 + h * 1024);
    return *reinterpret_cast<const __attribute__((address_space(1))) bf16x8*>(p + woff);
  };

  // per-row epilogue scale (down projection only): the route weight, or the shared expert's gate
  if (!kGateUp && tid < kPfBM) {
    float sc = 1.f;
    if (tid < M) {
      const int p = r0 + tid;
      if (!shared) sc = F::from_bits(a.topv[a.perm[p]]);
      else if (a.gate_s != nullptr) sc = F::round(sigmoid_f32(F::from_bits(a.gate_s[p])));
    }
    s_scale[tid] = sc;
  }

  // The tile's rows are processed in sub-tiles of 32 (one MFMA row block); a segment's last tile is
  // specialised on how many of them hold rows, so that a ragged tail costs the MFMAs, LDS reads and
  // stores of its own sub-tiles only.
  auto body = [&](auto nmi_c) {
    constexpr int NMI = decltype(nmi_c)::value;   // 32-row sub-tiles that hold rows
    constexpr int NMT = 2 * NMI;                  // 16-row MFMA column tiles
    f32x4 acc[NMT][4];
#pragma unroll
    for (int mt = 0; mt < NMT; ++mt)
#pragma unroll
      for (int g = 0; g < 4; ++g) acc[mt][g] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Pipeline: while slab kt is multiplied, the activation rows of slab kt+2 travel to the third LDS
    // buffer and the weight fragments of slab kt+2 to the registers half h has just finished with.
    // Vector memory operations retire in order, so "the copies of slab kt+1 have landed" is a count of
    // the younger operations: the 8 fragment loads of slab kt-1's halves, the 4 copies of slab kt+2 and
    // the 8 fragment loads of slab kt's halves -- vmcnt(20).  Slabs past the end refetch the last one
    // instead of branching.
    bf16x8 wfrag[2][2][4];   // [stage][k half][16-row group]
    stage_slab(0, 0);
    stage_slab(min(1, nk - 1), 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int g = 0; g < 4; ++g) wfrag[st][h][g] = wload(g, min(st, nk - 1), h);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(kWaitVm20);
    __syncthreads();

    // activation fragment of lane (r, q), tile mt, half h: row 16*mt + r, position (q + 4h) ^ f(r)
    const int fsw = ((fr >> 1) & 7) ^ ((fr & 1) << 2);
    const int a_row = fr * kPfRowBytes, a_x = (fq ^ fsw) << 4;
    int cur = 0, nxt2 = 2;  // buffer of slab kt, buffer of slab kt+2
    auto slab = [&](auto stage_c, int kt) {
      constexpr int st = decltype(stage_c)::value;
      const int kt2 = min(kt + 2, nk - 1);
      const uint8_t* la = lds[cur] + a_row;
      // Activation fragments come from LDS two at a time (two 16-row tiles: eight MFMAs), and the next
      // pair is requested before the current pair multiplies.  The full fences keep that order.
      constexpr int NP = NMT / 2, NB = 2 * NP;   // pairs per k half, pairs per slab
      bf16x8 fa[2][2];
      if (NP == 1) {   // one pair per half: the copies go first, so that every tile height issues its
        stage_slab(kt2, nxt2);   // vector memory operations in the order the counted wait assumes
        __builtin_amdgcn_sched_barrier(0);
      }
      auto rd = [&](int idx, bf16x8 (&f)[2]) __attribute__((always_inline)) {
        const int h = idx / NP, mb = 2 * (idx % NP);
#pragma unroll
        for (int i = 0; i < 2; ++i)
          f[i] = *reinterpret_cast<const bf16x8*>(la + (mb + i) * 16 * kPfRowBytes + (a_x ^ (h << 6)));
      };
      rd(0, fa[0]);
#pragma unroll
      for (int idx = 0; idx < NB; ++idx) {
        const int h = idx / NP, mb = 2 * (idx % NP);
        if (idx + 1 < NB) rd(idx + 1, fa[(idx + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);    // the next pair's reads stay ahead of this pair's MFMAs
        if (idx % NP != NP - 1) {
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g)
              acc[mb + i][g] = F::mfma16(wfrag[st][h][g], fa[idx & 1][i], acc[mb + i][g]);
          __builtin_amdgcn_sched_barrier(0);
        } else {
          // last pair of the half: group by group, each group's fragment of slab kt+2 requested right
          // behind its last MFMA, so that the four loads are spread over the pair
#pragma unroll
          for (int g = 0; g < 4; ++g) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
              acc[mb + i][g] = F::mfma16(wfrag[st][h][g], fa[idx & 1][i], acc[mb + i][g]);
            __builtin_amdgcn_sched_barrier(0);
            wfrag[st][h][g] = wload(g, kt2, h);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if (NP > 1 && idx == 0) {   // the copies of slab kt+2 go out once the matrix pipe has work
          stage_slab(kt2, nxt2);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      __builtin_amdgcn_s_waitcnt(kWaitVm20);
      __syncthreads();
      cur = (cur == kPfStages - 1) ? 0 : cur + 1;
      nxt2 = (nxt2 == kPfStages - 1) ? 0 : nxt2 + 1;
    };
    // Slabs go in pairs with no branch inside the loop (a conditional second slab would give the loop
    // head two different pictures of the outstanding fragment loads).
    int kt = 0;
    for (; kt + 2 <= nk; kt += 2) {
      slab(std::integral_constant<int, 0>{}, kt);
      slab(std::integral_constant<int, 1>{}, kt + 1);
    }
    if (kt < nk) slab(std::integral_constant<int, 0>{}, kt);
    __builtin_amdgcn_s_waitcnt(kWaitVm0);  // no copy may land in LDS after the epilogue starts to reuse it
    __syncthreads();

    // ---- epilogue ----------------------------------------------------------------
    // The product was formed as W * X^T, so a lane holds one row m (= 16*mt + fr) and, per 16-row
    // weight group, four consecutive output columns 4*fq + j: eight bytes of 16-bit values that go to the
    // wave's private staging area in LDS as one write.  The area holds a 128-row x 32-column tile, rows
    // of 64 bytes with the 16-byte chunks swizzled by row; it is read back a row quarter per lane and
    // stored with 16-byte writes, 64 contiguous bytes per row.
    uint8_t* st = &lds[0][0] + wave * (kPfBM * 64);
#pragma unroll
    for (int pass = 0; pass < (kGateUp ? 1 : 2); ++pass) {
      if (pass) __syncthreads();  // staging rows are reused
#pragma unroll
      for (int mt = 0; mt < NMT; ++mt) {
        const int m = mt * 16 + fr;
        const float sc = kGateUp ? 1.f : s_scale[m];
#pragma unroll
        for (int p = 0; p < 2; ++p) {   // the pass's two 16-column groups
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (kGateUp) {
              const float g = F::round(acc[mt][p][j]);
              const float u = F::round(acc[mt][2 + p][j]);
              v[j] = F::round(silu_f32(g)) * u;
            } else {
              v[j] = F::round(acc[mt][2 * pass + p][j]) * sc;
            }
          }
          uint2 pk;
          pk.x = F::pack2(v[0], v[1]);
          pk.y = F::pack2(v[2], v[3]);
          const int chunk = (2 * p + (fq >> 1)) ^ ((m >> 1) & 3);
          *reinterpret_cast<uint2*>(st + m * 64 + chunk * 16 + (fq & 1) * 8) = pk;
        }
      }
      __syncthreads();
      const int ncol0 = kGateUp ? (n0 + wave * 32) : (n0 + wave * 64 + pass * 32);
#pragma unroll
      for (int it = 0; it < 2 * NMI; ++it) {
        const int m = it * 16 + (lane >> 2), q = lane & 3;
        const uint4 val = *reinterpret_cast<const uint4*>(st + m * 64 + (q ^ ((m >> 1) & 3)) * 16);
        const int n = ncol0 + q * 8;
        if (m < M && n + 8 <= Ndim)
          *reinterpret_cast<uint4*>(out + static_cast<size_t>(r0 + m) * Ndim + n) = val;
      }
    }
  };
  switch ((M + 31) >> 5) {
    case 1: body(std::integral_constant<int, 1>{}); break;
    case 2: body(std::integral_constant<int, 2>{}); break;
    case 3: body(std::integral_constant<int, 3>{}); break;
    default: body(std::integral_constant<int, 4>{}); break;
  }
  if (a.clk != nullptr && tid == 0) {
    atomicAdd(&a.clk[0], static_cast<unsigned long long>(clock64() - clk_c0));
    atomicAdd(&a.clk[1], wall_clock64() - clk_t0);
  }
}

// ---- queues -------------------------------------------------------------------------------------
struct PfxMapArgs {
  const int32_t* expert_slot;
  const int32_t* seg_offsets;
  sparse_hip_seglist segs;
  int32_t* hdr;            // per launch (gate/up, down) 16 ints: first entry [8], entries [8]
  PfTile* map_gu;          // entry 0 of each map is the idle entry
  PfTile* map_dn;
  int32_t nt_gu, nt_dn;    // column tiles of a routed expert
  int32_t nts_gu, nts_dn;  // column tiles of the shared expert (0: none)
  int32_t mt_shared;       // row tiles of the shared expert
  int32_t T;               // tokens (rows of the shared expert)
  int32_t cap_gu, cap_dn;  // entries in each map
};

// Share x of n items cut into kPfXcds contiguous shares starts here.
__device__ __forceinline__ int pfx_start(int n, int x) { return static_cast<int>(static_cast<int64_t>(n) * x / kPfXcds); }
__device__ __forceinline__ int pfx_share_of(int n, int i) {
  int x = min(kPfXcds - 1, static_cast<int>(static_cast<int64_t>(i) * kPfXcds / max(n, 1)));
  while (x + 1 < kPfXcds && pfx_start(n, x + 1) <= i) ++x;
  while (x > 0 && pfx_start(n, x) > i) --x;
  return x;
}
// Queue x of a launch with R routed and S shared tiles: its share of the shared tiles, then its share
// of the routed ones (the shared expert's down tiles are the long ones, so they go first).
__device__ __forceinline__ int pfx_queue_base(int R, int S, int x) { return 1 + pfx_start(S, x) + pfx_start(R, x); }

// Workgroups [0, nt_gu) and [nt_gu, nt_gu + nt_dn): one per routed column tile of the two launches --
// segment s -> its row-tile count, scan, then thread s writes the entries of (segment s, this column
// tile, row tile 0 ..), routed order (segment, column tile, row tile).  The two last workgroups write
// the shared expert's entries (column tile, row tile) and the queue headers of their launch.
__global__ __launch_bounds__(256) void prefill_queue_kernel(const PfxMapArgs a) {
  __shared__ int32_t s_scan[SPARSE_HIP_MAX_EXPERTS];
  const int tid = threadIdx.x;
  int nseg = a.segs.n;
  if (a.segs.eids_dev != nullptr) nseg = min(nseg, a.segs.count_dev[0]);
  int mt = 0, slot = 0, r0 = 0, rows = 0;
  if (tid < nseg) {
    const int e = (a.segs.eids_dev != nullptr) ? a.segs.eids_dev[tid] : a.segs.eids[tid];
    r0 = a.seg_offsets[e];
    rows = a.seg_offsets[e + 1] - r0;
    mt = (rows + kPfBM - 1) / kPfBM;
    slot = (a.segs.eids_dev != nullptr) ? a.expert_slot[e] : a.segs.slots[tid];
  }
  s_scan[tid] = mt;
  __syncthreads();
  for (int off = 1; off < 256; off <<= 1) {
    const int v = (tid >= off) ? s_scan[tid - off] : 0;
    __syncthreads();
    s_scan[tid] += v;
    __syncthreads();
  }
  const int total_mt = s_scan[255];
  const int b = blockIdx.x;
  if (b < a.nt_gu + a.nt_dn) {
    const int which = b < a.nt_gu ? 0 : 1;
    const int bn = which == 0 ? b : b - a.nt_gu;
    PfTile* map = which == 0 ? a.map_gu : a.map_dn;
    const int nt = which == 0 ? a.nt_gu : a.nt_dn;
    const int cap = which == 0 ? a.cap_gu : a.cap_dn;
    const int R = total_mt * nt, S = a.mt_shared * (which == 0 ? a.nts_gu : a.nts_dn);
    if (mt > 0) {
      const int g0 = (s_scan[tid] - mt) * nt + bn * mt;
      for (int bm = 0; bm < mt; ++bm) {
        const int g = g0 + bm;
        const int x = pfx_share_of(R, g);
        const int pos = pfx_queue_base(R, S, x) + (pfx_start(S, x + 1) - pfx_start(S, x)) + (g - pfx_start(R, x));
        if (pos < cap) map[pos] = PfTile{slot, r0 + bm * kPfBM, min(kPfBM, rows - bm * kPfBM), bn};
      }
    }
    return;
  }
  const int which = b - (a.nt_gu + a.nt_dn);
  PfTile* map = which == 0 ? a.map_gu : a.map_dn;
  const int nt = which == 0 ? a.nt_gu : a.nt_dn;
  const int cap = which == 0 ? a.cap_gu : a.cap_dn;
  const int R = total_mt * nt, S = a.mt_shared * (which == 0 ? a.nts_gu : a.nts_dn);
  // The shared expert's tiles.  Where the tile grid divides evenly, XCD x takes a block of it -- a quarter
  // of the row tiles by half of the column tiles -- and walks the block down its rows first, so that the
  // 64 workgroups an XCD runs at a time cover about 8 x 8 tiles: each activation row tile and each weight
  // tile is then fetched into that L2 once per 8 users.  (Column by column over all row tiles, an XCD reads
  // the whole activation matrix, four times its L2, once per column tile.)  Otherwise: contiguous shares
  // of the (column tile, row tile) order.
  const int nts = which == 0 ? a.nts_gu : a.nts_dn;
  const bool blocked = a.mt_shared % 4 == 0 && nts % 2 == 0 && nts > 0;
  const int RG = a.mt_shared / 4, per_xcd = S / kPfXcds;
  for (int h = tid; h < S; h += 256) {
    int bn, bm, x, local;
    if (blocked) {
      x = h / per_xcd;
      local = h - x * per_xcd;
      bm = (x & 3) * RG + local % RG;
      bn = (x >> 2) * (nts / 2) + local / RG;
    } else {
      bn = h / a.mt_shared;
      bm = h - bn * a.mt_shared;
      x = pfx_share_of(S, h);
      local = h - pfx_start(S, x);
    }
    const int pos = pfx_queue_base(R, S, x) + local;
    if (pos < cap) map[pos] = PfTile{-1, bm * kPfBM, min(kPfBM, a.T - bm * kPfBM), bn};
  }
  if (tid == 0) map[0] = PfTile{0, 0, 0, 0};
  if (tid < kPfXcds) {
    int32_t* hdr = a.hdr + which * 16;
    hdr[tid] = pfx_queue_base(R, S, tid);
    hdr[kPfXcds + tid] = (pfx_start(S, tid + 1) - pfx_start(S, tid)) + (pfx_start(R, tid + 1) - pfx_start(R, tid));
  }
}

static inline int pfx_max_mtiles(int Ttok, int K, int nseg) { return (Ttok * K + kPfBM - 1) / kPfBM + nseg; }

struct PfxLayout {
  int nt_gu, nt_dn, nts_gu, nts_dn, mt_shared, cap_gu, cap_dn;
};
static PfxLayout pfx_layout(int Ttok, int K, int nseg, int H, int I, int Is) {
  PfxLayout l;
  l.nt_gu = (I + kPfBR / 2 - 1) / (kPfBR / 2);
  l.nt_dn = (H + kPfBR - 1) / kPfBR;
  l.nts_gu = Is > 0 ? (Is + kPfBR / 2 - 1) / (kPfBR / 2) : 0;
  l.nts_dn = Is > 0 ? l.nt_dn : 0;
  l.mt_shared = Is > 0 ? (Ttok + kPfBM - 1) / kPfBM : 0;
  const int mt = nseg > 0 ? pfx_max_mtiles(Ttok, K, nseg) : 0;
  l.cap_gu = 1 + mt * l.nt_gu + l.mt_shared * l.nts_gu;
  l.cap_dn = 1 + mt * l.nt_dn + l.mt_shared * l.nts_dn;
  return l;
}

constexpr size_t kPfWsHeader = 256;   // two launches x 16 ints, padded

size_t prefill_merged_ws_bytes(int Ttok, int K, int nseg, int H, int I, int Is) {
  const PfxLayout l = pfx_layout(Ttok, K, nseg, H, I, Is);
  return kPfWsHeader + (static_cast<size_t>(l.cap_gu) + l.cap_dn) * sizeof(PfTile);
}

extern std::atomic<int> g_prefill_drain_waits;
extern std::atomic<unsigned long long*> g_prefill_clock;

// `cap` entries at most (idle entry included): a queue holds a share of the shared and a share of the
// routed tiles, each rounded up, i.e. at most (cap - 1) / 8 + 2 entries.
template <bool kGateUp>
static int launch_merged(PfxArgs& a, int cap, bool fp16, hipStream_t st) {
  const int64_t grid = (static_cast<int64_t>(cap - 1) / kPfXcds + 2) * kPfXcds;
  SP_REQUIRE(grid < (1ll << 31), "prefill_ffn: grid too large");
  ProfScope prof(kGateUp ? SPARSE_HIP_K_PREFILL_GATEUP : SPARSE_HIP_K_PREFILL_DOWN, st);
  a.clk = g_prefill_clock.load(std::memory_order_relaxed);
  const bool drain = g_prefill_drain_waits.load(std::memory_order_relaxed) != 0;
#define SP_PFX_LAUNCH(F, D) \
  hipLaunchKernelGGL((prefill_merged_kernel<F, kGateUp, D>), dim3(static_cast<unsigned>(grid)), dim3(kPfThreads), 0, st, a)
  if (fp16) {
    if (drain) SP_PFX_LAUNCH(Fp16, true); else SP_PFX_LAUNCH(Fp16, false);
  } else {
    if (drain) SP_PFX_LAUNCH(Bf16, true); else SP_PFX_LAUNCH(Bf16, false);
  }
#undef SP_PFX_LAUNCH
  SP_LAUNCH_CHECK("prefill_merged_kernel");
  return SPARSE_HIP_OK;
}

// Routed experts (segs->n > 0) and / or the shared expert (sh_down_w != nullptr) of one call.
int prefill_merged(const sparse_hip_experts* ex, const void* x, const void* topv, const int32_t* perm,
                   const int32_t* seg_offsets, const sparse_hip_seglist* segs, int Ttok, int K, void* inter_ws,
                   void* parts, const void* sh_gate_w, const void* sh_up_w, const void* sh_down_w,
                   const void* shared_gate, int Is, void* sh_inter_ws, void* shared_out, void* tile_ws,
                   hipStream_t st) {
  const int H = ex->hidden, I = ex->inter;
  const bool shared = sh_down_w != nullptr;
  const PfxLayout l = pfx_layout(Ttok, K, segs->n, H, I, shared ? Is : 0);
  int32_t* hdr = static_cast<int32_t*>(tile_ws);
  PfTile* map_gu = reinterpret_cast<PfTile*>(static_cast<uint8_t*>(tile_ws) + kPfWsHeader);
  PfTile* map_dn = map_gu + l.cap_gu;
  {
    PfxMapArgs m = {};
    m.expert_slot = ex->expert_slot_dev;
    m.seg_offsets = seg_offsets;
    m.segs = *segs;
    m.hdr = hdr;
    m.map_gu = map_gu;
    m.map_dn = map_dn;
    m.nt_gu = l.nt_gu;
    m.nt_dn = l.nt_dn;
    m.nts_gu = l.nts_gu;
    m.nts_dn = l.nts_dn;
    m.mt_shared = l.mt_shared;
    m.T = Ttok;
    m.cap_gu = l.cap_gu;
    m.cap_dn = l.cap_dn;
    hipLaunchKernelGGL(prefill_queue_kernel, dim3(l.nt_gu + l.nt_dn + 2), dim3(256), 0, st, m);
    SP_LAUNCH_CHECK("prefill_queue_kernel");
  }
  const bool fp16 = ex->dtype == SPARSE_HIP_F16;
  PfxArgs a = {};
  a.slab = static_cast<const uint16_t*>(ex->slab_dev);
  a.slot_stride = ex->slot_stride / 2;
  a.perm = perm;
  a.topv = static_cast<const uint16_t*>(topv);
  a.topk = K;
  a.topk_magic = K == 1 ? 0u : static_cast<uint32_t>(((1ull << 32) + K - 1) / K);
  // gate/up: x -> inter
  a.mat_offset = 0;
  a.mat2_offset = static_cast<uint64_t>(I) * H;
  a.act_r = static_cast<const uint16_t*>(x);
  a.out_r = static_cast<uint16_t*>(inter_ws);
  a.Kdim_r = H;
  a.Ndim_r = I;
  a.w_s = static_cast<const uint16_t*>(sh_gate_w);
  a.w2_s = static_cast<const uint16_t*>(sh_up_w);
  a.gate_s = nullptr;
  a.act_s = static_cast<const uint16_t*>(x);
  a.out_s = static_cast<uint16_t*>(sh_inter_ws);
  a.Kdim_s = H;
  a.Ndim_s = shared ? Is : 64;
  a.map = map_gu;
  a.qhdr = hdr;
  int rc = launch_merged<true>(a, l.cap_gu, fp16, st);
  if (rc != SPARSE_HIP_OK) return rc;
  // down: inter -> parts * route weight (shared: * sigmoid(gate) where there is one)
  a.mat_offset = 2ull * I * H;
  a.mat2_offset = 0;
  a.act_r = static_cast<const uint16_t*>(inter_ws);
  a.out_r = static_cast<uint16_t*>(parts);
  a.Kdim_r = I;
  a.Ndim_r = H;
  a.w_s = static_cast<const uint16_t*>(sh_down_w);
  a.w2_s = nullptr;
  a.gate_s = static_cast<const uint16_t*>(shared_gate);
  a.act_s = static_cast<const uint16_t*>(sh_inter_ws);
  a.out_s = static_cast<uint16_t*>(shared_out);
  a.Kdim_s = shared ? Is : 64;
  a.Ndim_s = H;
  a.map = map_dn;
  a.qhdr = hdr + 16;
  return launch_merged<false>(a, l.cap_dn, fp16, st);
}

}  // namespace sparse
