// Prefill-time grouped SwiGLU expert FFN (bf16 / fp16): the MFMA grouped-GEMM path.
//
// C[p, n] = sum_k A[p, k] * W[n, k] per expert segment.  A workgroup (4 waves) owns a
// 128-row x 256-weight-row tile; wave w owns all 128 rows and 64 of the weight rows
// (eight by four 16x16x32 MFMA tiles, 128 accumulator registers).  For the gate/up
// projection the 256 weight rows are 128 gate rows and the 128 matching up rows, and a
// wave's four 16-row groups are the gate groups and the up groups of the same 32 neurons, so
// SiLU(gate)*up is a lane-local epilogue.
//
// The two operands take different roads.  Activation rows are shared by the four waves:
// they go HBM/L2 -> LDS directly (no register hop) in 64-wide k slabs, three LDS buffers,
// two slabs ahead of the multiply, one barrier per slab, chunks swizzled by row so that
// 16-byte fragment reads are bank-conflict free.
// Weight rows are private to a wave: they go HBM/L2 -> registers directly in MFMA
// A-operand order, which is exactly the order the tiled layout stores them in (a wave
// load is one 1 KB run), two slabs ahead of the multiply.  LDS thus carries a third
// of the bytes of a both-operands-through-LDS design, which is what bounds this shape.
//
// Which tile a workgroup owns is read from a map built by a one-workgroup kernel before
// the launch (segment lengths are only known on the device).  Block ids are dealt to the
// eight XCDs round-robin by the hardware; the map index is re-derived so that an XCD
// works through whole experts, m-tiles of one weight tile adjacent in time, which keeps a
// weight tile in that XCD's L2 while it is reused.
//
// MFMA 16x16x32 operand layout (lane l, r = l & 15, q = l >> 4):
//   A: row r, eight k    B: column r, the same eight k    D: column r, rows 4*q + j for register j
// The weights are passed as A and the activations as B, so D is the transposed output tile: a lane
// owns one activation row and four consecutive output columns.  Which eight k a lane holds is free as
// long as A and B agree; the tiled weight layout fixes it: half h of a 64-wide slab is the A operand
// of one MFMA in lane order, lane (r, q) holding k = 16*q + 8*h + 0..7, i.e. the 16-byte chunk 2*q + h
// of a 128-byte slab row, and the activation fragments are read from LDS in the same order.
// (The 16x16x32 shape moves half the accumulator data per flop of the 32x32x16 one; with real operands
// the part is power-capped in either, and a loop of this wavefront tile fed from LDS sustained 8 % more
// with it.)
#include <atomic>
#include <type_traits>

#include "common.h"
#include "prefill_tiles.h"

namespace sparse {


struct PrefillArgs {
  const uint16_t* slab;
  uint64_t slot_stride;  // elements
  uint64_t mat_offset;   // elements
  uint64_t mat2_offset;  // elements
  const int32_t* perm;
  const uint16_t* topv;
  const uint16_t* act;
  uint16_t* out;
  const PfTile* map;      // routed: one entry per tile
  const int32_t* total;   // routed: number of tiles in the map
  int32_t topk;
  int32_t Kdim;
  int32_t Ndim;       // output columns (neurons for gate-up, hidden for down)
  int32_t ntiles_n;
  int32_t shared;
  int32_t T;
  const uint16_t* w_s;
  const uint16_t* w2_s;
  const uint16_t* gate_s;
  int32_t fp16;             // 16-bit format of every tensor: 0 bfloat16, 1 IEEE half
  unsigned long long* clk;  // clock probe: [0] += shader-clock cycles, [1] += 100 MHz ticks per workgroup; may be null
};

struct PfMapArgs {
  const int32_t* expert_slot;
  const int32_t* seg_offsets;
  PfTile* map_gu;
  PfTile* map_dn;
  int32_t* totals;  // [0] gate/up tiles, [1] down tiles
  int32_t ntiles_gu, ntiles_dn;
  int32_t cap_gu, cap_dn;  // entries in each map
  sparse_hip_seglist segs;
};

// One workgroup per column tile of each of the two maps (gate/up first): segment s -> its m-tile
// count, scan (every workgroup does its own: 256 entries), then thread s writes the entries of
// (segment s, this column tile, m-tile 0 ..) -- tiles in the order segment, column tile, m-tile.
// The workgroups of column tile 0 also mark the rest of their map idle and write its tile count.
__global__ __launch_bounds__(256) void prefill_tile_map_kernel(const PfMapArgs a) {
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
  const int which = static_cast<int>(blockIdx.x) < a.ntiles_gu ? 0 : 1;
  const int bn = which == 0 ? blockIdx.x : blockIdx.x - a.ntiles_gu;
  PfTile* map = which == 0 ? a.map_gu : a.map_dn;
  const int nt = which == 0 ? a.ntiles_gu : a.ntiles_dn;
  const int cap = which == 0 ? a.cap_gu : a.cap_dn;
  if (mt > 0) {
    const int base = (s_scan[tid] - mt) * nt + bn * mt;
    for (int bm = 0; bm < mt; ++bm)
      if (base + bm < cap) map[base + bm] = PfTile{slot, r0 + bm * kPfBM, min(kPfBM, rows - bm * kPfBM), bn};
  }
  if (bn == 0) {
    for (int idx = total_mt * nt + tid; idx < cap; idx += 256) map[idx] = PfTile{0, 0, 0, 0};
    if (tid == 0) a.totals[which] = total_mt * nt;
  }
}

// kDrainWaits replaces the counted vector-memory waits of the k loop by full drains: slower,
// and correct whatever else the compiler has in flight.  It exists to check the counted
// waits: both variants must give the same bits.
template <typename F, bool kGateUp, bool kDrainWaits>
__global__ __launch_bounds__(kPfThreads, 2) void prefill_ffn_kernel(const PrefillArgs a) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kPfStages][kPfLdsA];
  __shared__ float s_scale[kPfBM];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int fr = lane & 15, fq = lane >> 4;
  const long long clk_c0 = clock64();
  const unsigned long long clk_t0 = wall_clock64();

  // ---- which tile (XCD-aware order) ----------------------------------------------
  // The real tile count is split evenly over the XCDs (the grid is sized for the worst
  // case, and the idle remainder must not fall on one XCD).
  int slot_id = 0, r0, M, bn;
  const int mt_s = (a.T + kPfBM - 1) / kPfBM;
  const int total = a.shared ? mt_s * a.ntiles_n : a.total[0];
  const int per_xcd = (total + kPfXcds - 1) / kPfXcds;
  const int in_xcd = blockIdx.x / kPfXcds;
  const int logical = (blockIdx.x % kPfXcds) * per_xcd + in_xcd;
  if (in_xcd >= per_xcd || logical >= total) return;
  if (a.shared) {
    const int mt = mt_s;
    bn = logical / mt;
    r0 = (logical - bn * mt) * kPfBM;
    M = min(kPfBM, a.T - r0);
  } else {
    const PfTile tile = a.map[logical];
    if (tile.rows <= 0) return;
    slot_id = tile.slot;
    r0 = tile.r0;
    M = tile.rows;
    bn = tile.bn;
  }

  const int Kdim = a.Kdim, Ndim = a.Ndim;
  const uint16_t *w0, *w1 = nullptr;
  if (a.shared) {
    w0 = a.w_s;
    w1 = a.w2_s;
  } else {
    const uint16_t* slot = a.slab + static_cast<uint64_t>(slot_id) * a.slot_stride;
    w0 = slot + a.mat_offset;
    w1 = slot + a.mat2_offset;
  }
  const int n0 = bn * (kGateUp ? kPfBR / 2 : kPfBR);  // first output column of this tile

  // per-row epilogue scale (down projection only)
  if (!kGateUp && tid < kPfBM) {
    float sc = 1.f;
    if (tid < M) {
      const int p = r0 + tid;
      if (a.shared) {
        if (a.gate_s != nullptr) sc = F::round(sigmoid_f32(F::from_bits(a.gate_s[p])));
      } else {
        sc = F::from_bits(a.topv[a.perm[p]]);
      }
    }
    s_scale[tid] = sc;
  }

  // ---- activation loader: global -> LDS without passing through registers ----------
  // One wave instruction moves 64 sixteen-byte pieces to 1 KB of consecutive LDS (lane l
  // lands at byte 16*l), i.e. eight 128-byte rows of the slab; the lane chooses which
  // piece of which row it fetches.  Row r keeps its chunk j = 2q + h (the eight k values of
  // MFMA lane group q in k half h) at position (q + 4h) ^ f(r) with
  // f(r) = ((r >> 1) & 7) ^ ((r & 1) << 2): a fragment read (16 rows, the four q of one half)
  // then takes the four clocks of a conflict-free one -- with the chunks in their natural order
  // the same read measured 6.4.  Wave w owns rows 32w .. 32w+31.
  const uint16_t* dptr[4];
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int row = wave * 32 + it * 8 + (lane >> 3);
    const int p = r0 + min(row, M - 1);
    const size_t grow = (a.shared || !kGateUp) ? static_cast<size_t>(p) : static_cast<size_t>(a.perm[p] / a.topk);
    const int f = ((row >> 1) & 7) ^ ((row & 1) << 2);
    const int pos = (lane & 7) ^ f;                    // position q + 4h holds chunk 2q + h
    dptr[it] = a.act + grow * Kdim + ((((pos & 3) << 1) | (pos >> 2)) << 3);
  }
  // Issued as inline assembly: the compiler would otherwise make every barrier wait for all
  // outstanding vector memory operations because one of them writes LDS, which is exactly
  // the prefetch distance this loop exists for.  Completion is awaited by count below.
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) uint8_t*)(&lds[0][0])));
  auto stage_slab = [&](int slab, int buf) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const uint16_t* g = dptr[it] + slab * kPfBK;
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + buf * kPfLdsA + (wave * 4 + it) * 1024);
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(dst) : "memory", "m0");
    }
  };

  // ---- weight fragments straight from the tiled layout ------------------------------
  // The wavefront's 64 weight rows are four 16-row groups; in the tiled layout a group's 64-wide slab
  // is 2 KB: the first KB is the A operand of the MFMA over its k half 0 in lane order, the second KB
  // that of half 1.  Gate/up: groups 0, 1 are gate rows of 32 neurons, groups 2, 3 the up rows of the
  // same neurons.
  const uint16_t* wptr[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const uint16_t* base = (kGateUp && g >= 2) ? w1 : w0;
    int n = kGateUp ? (n0 + wave * 32 + (g & 1) * 16) : (n0 + wave * 64 + g * 16);
    n = min(n, Ndim - 16);
    wptr[g] = base + static_cast<size_t>(n >> 4) * 16 * Kdim + lane * 8;
  }

  // The tile's rows are processed in sub-tiles of 32 (one MFMA row block); a segment's last
  // tile is specialised on how many of them hold rows, so that a ragged tail costs the MFMAs,
  // LDS reads and stores of its own sub-tiles only.
  auto body = [&](auto nmi_c) {
    constexpr int NMI = decltype(nmi_c)::value;   // 32-row sub-tiles that hold rows
    constexpr int NMT = 2 * NMI;                  // 16-row MFMA column tiles
    f32x4 acc[NMT][4];
  #pragma unroll
    for (int mt = 0; mt < NMT; ++mt)
  #pragma unroll
      for (int g = 0; g < 4; ++g) acc[mt][g] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Pipeline: while slab kt is multiplied, the activation rows of slab kt+2 travel to the
    // third LDS buffer and the weight fragments of slab kt+2 to the registers half h has just
    // finished with (two fragment sets, used alternately), so every operand is requested two
    // slabs of MFMA work before its use -- enough bytes in flight to cover an HBM miss.
    // Vector memory operations retire in order, so "the copies of slab kt+1 have landed" is a
    // count of the younger operations: the 8 fragment loads of slab kt-1's halves, the 4 copies
    // of slab kt+2 and the 8 fragment loads of slab kt's halves -- vmcnt(20) -- and the
    // scheduling fences keep exactly that order (copies, half 0, half 1 in every slab).  Slabs past the end refetch the last one
    // instead of branching.
    // s_waitcnt vmcnt(n), other counters untouched
    constexpr int kWaitVm0 = kWaitVmcnt0, kWaitVm20 = kDrainWaits ? kWaitVmcnt0 : kWaitVmcnt20;
    const int nk = Kdim / kPfBK;
    bf16x8 wfrag[2][2][4];   // [stage][k half][16-row group]
    stage_slab(0, 0);
    stage_slab(min(1, nk - 1), 1);
    __builtin_amdgcn_sched_barrier(0);
  #pragma unroll
    for (int st = 0; st < 2; ++st)
  #pragma unroll
      for (int h = 0; h < 2; ++h)
  #pragma unroll
        for (int g = 0; g < 4; ++g)
          wfrag[st][h][g] =
              *reinterpret_cast<const bf16x8*>(wptr[g] + static_cast<size_t>(min(st, nk - 1)) * 1024 + h * 512);
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
      // Activation fragments come from LDS two at a time (two 16-row tiles: eight MFMAs), and the next pair
      // is requested before the current pair multiplies: a wavefront on its own then waits for an LDS read
      // once per slab instead of once per pair.  The full fences keep that order (the compiler otherwise
      // sinks every read to just in front of its first use).
      constexpr int NP = NMT / 2, NB = 2 * NP;   // pairs per k half, pairs per slab
      bf16x8 fa[2][2];
      if (NP == 1) {   // one pair per half: the copies go first, so that every tile height issues its
        stage_slab(kt2, nxt2);   // vector memory operations in the order the counted wait below assumes
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
          // last pair of the half: group by group, each group's fragment of slab kt+2 requested right behind
          // its last MFMA, so that the four loads are spread over the pair instead of queueing behind it
  #pragma unroll
          for (int g = 0; g < 4; ++g) {
  #pragma unroll
            for (int i = 0; i < 2; ++i)
              acc[mb + i][g] = F::mfma16(wfrag[st][h][g], fa[idx & 1][i], acc[mb + i][g]);
            __builtin_amdgcn_sched_barrier(0);
            wfrag[st][h][g] = *reinterpret_cast<const bf16x8*>(wptr[g] + static_cast<size_t>(kt2) * 1024 + h * 512);
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
    // Slabs go in pairs with no branch inside the loop: a conditional second slab would give the
    // loop head two different pictures of the outstanding fragment loads, and the waits the
    // compiler puts before each MFMA would then assume the shorter one (eight loads behind
    // instead of sixteen), i.e. drain the loads issued for the slab after next.
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
    // weight group, four consecutive output columns 4*fq + j: eight bytes of 16-bit values that go
    // to the wave's private staging area in LDS (free now: every wave is past the last barrier of
    // the k loop) as one write.  The area holds a 128-row x 32-column tile, rows of 64 bytes with
    // the 16-byte chunks swizzled by row; it is read back a row quarter per lane and stored with
    // 16-byte writes, 64 contiguous bytes per row.
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
          *reinterpret_cast<uint4*>(a.out + static_cast<size_t>(r0 + m) * Ndim + n) = val;
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

// also read by the persistent-workgroup form of this kernel
std::atomic<int> g_prefill_drain_waits{0};
std::atomic<unsigned long long*> g_prefill_clock{nullptr};

void prefill_set_clock_probe(void* counters_dev) {
  g_prefill_clock.store(static_cast<unsigned long long*>(counters_dev));
}

int prefill_set_drain_waits(int on) { return g_prefill_drain_waits.exchange(on ? 1 : 0); }

template <bool kGateUp>
static int launch_prefill(PrefillArgs& a, int max_mtiles, hipStream_t st) {
  int64_t grid = static_cast<int64_t>(a.ntiles_n) * max_mtiles;
  grid = (grid + kPfXcds - 1) / kPfXcds * kPfXcds;
  if (grid == 0) return SPARSE_HIP_OK;
  SP_REQUIRE(grid < (1ll << 31), "prefill_ffn: grid too large");
  ProfScope prof(kGateUp ? SPARSE_HIP_K_PREFILL_GATEUP : SPARSE_HIP_K_PREFILL_DOWN, st);
  a.clk = g_prefill_clock.load(std::memory_order_relaxed);
  const bool drain = g_prefill_drain_waits.load(std::memory_order_relaxed) != 0;
#define SP_PF_LAUNCH(F, D) \
  hipLaunchKernelGGL((prefill_ffn_kernel<F, kGateUp, D>), dim3(static_cast<unsigned>(grid)), dim3(kPfThreads), 0, st, a)
  if (a.fp16) {
    if (drain) SP_PF_LAUNCH(Fp16, true); else SP_PF_LAUNCH(Fp16, false);
  } else {
    if (drain) SP_PF_LAUNCH(Bf16, true); else SP_PF_LAUNCH(Bf16, false);
  }
#undef SP_PF_LAUNCH
  SP_LAUNCH_CHECK("prefill_ffn_kernel");
  return SPARSE_HIP_OK;
}

static inline int pf_max_mtiles(int Ttok, int K, int nseg) { return (Ttok * K + kPfBM - 1) / kPfBM + nseg; }
static inline int64_t pf_round8(int64_t v) { return (v + kPfXcds - 1) / kPfXcds * kPfXcds; }

size_t prefill_ws_bytes(int Ttok, int K, int nseg, int H, int I) {
  const int64_t mt = pf_max_mtiles(Ttok, K, nseg);
  const int64_t gu = pf_round8(mt * ((I + kPfBR / 2 - 1) / (kPfBR / 2)));
  const int64_t dn = pf_round8(mt * ((H + kPfBR - 1) / kPfBR));
  return static_cast<size_t>(gu + dn + 1) * sizeof(PfTile);  // one leading entry holds the two totals
}

int prefill_routed_bf16(const sparse_hip_experts* ex, const void* x, const void* topv, const int32_t* perm,
                        const int32_t* seg_offsets, const sparse_hip_seglist* segs, int Ttok, int K,
                        void* inter_ws, void* parts, void* tile_ws, hipStream_t st) {
  const uint64_t H = ex->hidden, I = ex->inter;
  const int mt = pf_max_mtiles(Ttok, K, segs->n);
  const int nt_gu = static_cast<int>((I + kPfBR / 2 - 1) / (kPfBR / 2));
  const int nt_dn = static_cast<int>((H + kPfBR - 1) / kPfBR);
  const int cap_gu = static_cast<int>(pf_round8(static_cast<int64_t>(mt) * nt_gu));
  const int cap_dn = static_cast<int>(pf_round8(static_cast<int64_t>(mt) * nt_dn));
  int32_t* totals = static_cast<int32_t*>(tile_ws);
  PfTile* map_gu = static_cast<PfTile*>(tile_ws) + 1;
  PfTile* map_dn = map_gu + cap_gu;
  {
    PfMapArgs m = {};
    m.expert_slot = ex->expert_slot_dev;
    m.seg_offsets = seg_offsets;
    m.map_gu = map_gu;
    m.map_dn = map_dn;
    m.totals = totals;
    m.ntiles_gu = nt_gu;
    m.ntiles_dn = nt_dn;
    m.cap_gu = cap_gu;
    m.cap_dn = cap_dn;
    m.segs = *segs;
    hipLaunchKernelGGL(prefill_tile_map_kernel, dim3(nt_gu + nt_dn), dim3(256), 0, st, m);
    SP_LAUNCH_CHECK("prefill_tile_map_kernel");
  }
  PrefillArgs a = {};
  a.fp16 = ex->dtype == SPARSE_HIP_F16;
  a.slab = static_cast<const uint16_t*>(ex->slab_dev);
  a.slot_stride = ex->slot_stride / 2;
  a.perm = perm;
  a.topk = K;
  a.T = Ttok;
  a.mat_offset = 0;
  a.mat2_offset = I * H;
  a.act = static_cast<const uint16_t*>(x);
  a.out = static_cast<uint16_t*>(inter_ws);
  a.map = map_gu;
  a.total = totals;
  a.Kdim = static_cast<int32_t>(H);
  a.Ndim = static_cast<int32_t>(I);
  a.ntiles_n = nt_gu;
  int rc = launch_prefill<true>(a, mt, st);
  if (rc != SPARSE_HIP_OK) return rc;
  a.mat_offset = 2 * I * H;
  a.mat2_offset = 0;
  a.topv = static_cast<const uint16_t*>(topv);
  a.act = static_cast<const uint16_t*>(inter_ws);
  a.out = static_cast<uint16_t*>(parts);
  a.map = map_dn;
  a.total = totals + 1;
  a.Kdim = static_cast<int32_t>(I);
  a.Ndim = static_cast<int32_t>(H);
  a.ntiles_n = nt_dn;
  return launch_prefill<false>(a, mt, st);
}

int prefill_shared_bf16(const void* x, const void* gate_w, const void* up_w, const void* down_w,
                        const void* shared_gate, int dtype, int Ttok, int H, int Is, void* inter_ws,
                        void* shared_out, hipStream_t st) {
  PrefillArgs a = {};
  a.fp16 = dtype == SPARSE_HIP_F16;
  a.shared = 1;
  a.T = Ttok;
  a.topk = 1;
  const int mt = (Ttok + kPfBM - 1) / kPfBM;
  a.w_s = static_cast<const uint16_t*>(gate_w);
  a.w2_s = static_cast<const uint16_t*>(up_w);
  a.act = static_cast<const uint16_t*>(x);
  a.out = static_cast<uint16_t*>(inter_ws);
  a.Kdim = H;
  a.Ndim = Is;
  a.ntiles_n = (Is + kPfBR / 2 - 1) / (kPfBR / 2);
  int rc = launch_prefill<true>(a, mt, st);
  if (rc != SPARSE_HIP_OK) return rc;
  a.w_s = static_cast<const uint16_t*>(down_w);
  a.w2_s = nullptr;
  a.gate_s = static_cast<const uint16_t*>(shared_gate);
  a.act = static_cast<const uint16_t*>(inter_ws);
  a.out = static_cast<uint16_t*>(shared_out);
  a.Kdim = Is;
  a.Ndim = H;
  a.ntiles_n = (H + kPfBR - 1) / kPfBR;
  return launch_prefill<false>(a, mt, st);
}

}  // namespace sparse
