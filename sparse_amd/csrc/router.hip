// Router: gate projection (logits), fused softmax + top-k with wavefront shuffles, and
// the single-launch decode router (logits -> top-k -> permutation).
#include "permute_device.h"

namespace sparse {

// ---------------------------------------------------------------------------
// logits[t, e] = <x[t, :], wg[e, :]>, one workgroup per (expert row, 32-token tile).
// Row `E` of the grid (when present) is the shared-expert gate vector.
// Every thread owns 8 consecutive h per 2048-wide sweep so that one sweep of the
// workgroup reads a weight row with 16-byte (bf16) / 32-byte (fp32) loads per lane.
// ---------------------------------------------------------------------------
constexpr int kRouterThreads = 256;
constexpr int kRouterTokTile = 32;

// Eight consecutive elements as they sit in memory, and their widening to fp32.
template <typename T>
struct Raw8;
template <>
struct Raw8<float> {
  float4 a, b;
  __device__ __forceinline__ void load(const float* p) {
    a = *reinterpret_cast<const float4*>(p);
    b = *reinterpret_cast<const float4*>(p + 4);
  }
  __device__ __forceinline__ void widen(float (&v)[8]) const {
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
};
template <>
struct Raw8<uint16_t> {
  u32x4 a;
  __device__ __forceinline__ void load(const uint16_t* p) { a = *reinterpret_cast<const u32x4*>(p); }
  __device__ __forceinline__ void widen(float (&v)[8]) const {
    v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
    v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
    v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xffff0000u);
    v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xffff0000u);
  }
};
template <>
struct Raw8<f16_t> {
  f16x8 a;
  __device__ __forceinline__ void load(const f16_t* p) { a = *reinterpret_cast<const f16x8*>(p); }
  __device__ __forceinline__ void widen(float (&v)[8]) const {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = static_cast<float>(a[j]);
  }
};
template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&v)[8]) {
  Raw8<T> r;
  r.load(p);
  r.widen(v);
}

// Dot products of one weight row with up to 32 token rows; the workgroup's result for
// token i lands in thread i (i < nt) and is stored by `store(token, value)`.
template <typename T, typename Store>
__device__ __forceinline__ void router_row_dots(const T* __restrict__ x, const T* __restrict__ w, int t0, int nt,
                                                int H, Store store) {
  float acc[kRouterTokTile];
#pragma unroll
  for (int i = 0; i < kRouterTokTile; ++i) acc[i] = 0.f;
  for (int h = threadIdx.x * 8; h < H; h += kRouterThreads * 8) {
    float wv[8];
    load8<T>(w + h, wv);
#pragma unroll
    for (int i = 0; i < kRouterTokTile; ++i) {
      if (i < nt) {
        float xv[8];
        load8<T>(x + static_cast<size_t>(t0 + i) * H + h, xv);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i] = fmaf(xv[j], wv[j], acc[i]);
      }
    }
  }
  __shared__ float red[kRouterThreads / 64][kRouterTokTile];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < kRouterTokTile; ++i) {
    if (i < nt) {
      const float s = wave_sum(acc[i]);
      if (lane == 0) red[wave][i] = s;
    }
  }
  __syncthreads();
  if (static_cast<int>(threadIdx.x) < nt) {
    float s = 0.f;
#pragma unroll
    for (int wv = 0; wv < kRouterThreads / 64; ++wv) s += red[wv][threadIdx.x];
    store(t0 + static_cast<int>(threadIdx.x), s);
  }
}

template <typename T, typename TL>
__global__ __launch_bounds__(kRouterThreads) void router_logits_kernel(
    const T* __restrict__ x, const T* __restrict__ wg, const T* __restrict__ wsg, int Ttok, int H,
    int E, TL* __restrict__ logits, T* __restrict__ shared_gate) {
  const int row = blockIdx.x;  // expert id, or E for the shared gate
  const int t0 = blockIdx.y * kRouterTokTile;
  const int nt = min(kRouterTokTile, Ttok - t0);
  const T* w = (row < E) ? wg + static_cast<size_t>(row) * H : wsg;
  router_row_dots<T>(x, w, t0, nt, H, [&](int t, float s) {
    if (row < E) {
      Elem<TL>::store(logits + static_cast<size_t>(t) * E + row, s);
    } else {
      Elem<T>::store(shared_gate + t, s);
    }
  });
}

// ---------------------------------------------------------------------------
// Prefill-size router logits (bf16): one workgroup per 16 tokens, the four wavefronts
// split H.  A wavefront multiplies its 16 x (H/4) slice of x with 64 gate rows at a time
// (four 16x16x32 MFMA tiles; x rows are the A operand, gate rows the B operand, both read
// from global memory in operand order: lane (r = l & 15, q = l >> 4) holds row r,
// k = q*8 .. q*8+7), the four partial tiles meet in LDS and are summed in wavefront order.
// Row E (when present) is the shared-expert gate vector.  Needs H % 512 == 0.
// ---------------------------------------------------------------------------
constexpr int kRlTok = 16;
constexpr int kRlRows = 64;   // gate rows per pass
constexpr int kRlPad = 65;    // LDS row stride in floats

template <typename F, typename TL>
__global__ __launch_bounds__(256) void router_logits_mfma_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ wg, const uint16_t* __restrict__ wsg, int Ttok,
    int H, int E, TL* __restrict__ logits, uint16_t* __restrict__ shared_gate) {
  __shared__ float part[4][kRlTok][kRlPad];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, q = lane >> 4;
  const int t0 = blockIdx.x * kRlTok;
  const int R = E + (wsg != nullptr ? 1 : 0);
  const int kspan = H / 4, kbeg = wave * kspan;
  const uint16_t* xrow = x + static_cast<size_t>(min(t0 + r, Ttok - 1)) * H + kbeg + q * 8;

  for (int row0 = 0; row0 < R; row0 += kRlRows) {
    const uint16_t* wrow[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int row = row0 + nt * 16 + r;
      wrow[nt] = (row < E ? wg + static_cast<size_t>(row) * H : (row == E && wsg != nullptr ? wsg : wg)) + kbeg + q * 8;
    }
    f32x4 acc[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < kspan; k0 += 128) {
      bf16x8 av[4], bv[4][4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        av[u] = *reinterpret_cast<const bf16x8*>(xrow + k0 + u * 32);
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) bv[u][nt] = *reinterpret_cast<const bf16x8*>(wrow[nt] + k0 + u * 32);
      }
      __builtin_amdgcn_sched_barrier(0);  // all 20 loads of the span in flight before the first MFMA
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
          acc[nt] = F::mfma16(av[u], bv[u][nt], acc[nt]);
    }
    // D: lane holds gate row (column) nt*16 + r for tokens q*4 .. q*4+3
    if (row0 > 0) __syncthreads();
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int v = 0; v < 4; ++v) part[wave][q * 4 + v][nt * 16 + r] = acc[nt][v];
    __syncthreads();
    for (int i = tid; i < kRlTok * kRlRows; i += 256) {
      const int tok = i >> 6, col = i & 63;
      const int row = row0 + col, t = t0 + tok;
      if (t < Ttok && row < R) {
        const float sum = ((part[0][tok][col] + part[1][tok][col]) + part[2][tok][col]) + part[3][tok][col];
        if (row < E) {
          Elem<TL>::store(logits + static_cast<size_t>(t) * E + row, sum);
        } else {
          shared_gate[t] = F::bits(sum);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Fused softmax(fp32) + top-k of one token by one wavefront; lane l holds experts
// l, l+64, l+128, l+192.  Selection runs K rounds of a wave-wide arg-max on the LOGITS
// themselves, in the order (logit descending, expert id ascending): softmax is monotone, so
// this is the order of the probabilities wherever those differ, and it does not depend on
// how exp and the division round when two logits one ulp apart collapse to one probability.
// A probability is computed only for the K winners (and nothing else of the row needs one:
// a group's best probability belongs to its best logit).  With `softmax` off the row is
// ranked and returned as it is (top-k of given probabilities).  All cross-lane steps are
// DPP reductions.  Lane r < K also returns the r-th selected expert.
// ---------------------------------------------------------------------------
constexpr int kTopkWaves = 4;
constexpr int kTopkNV = SPARSE_HIP_MAX_EXPERTS / 64;

template <typename TL, typename TO>
__device__ __forceinline__ int topk_token(const TL* __restrict__ row, int E, int K, int renorm,
                                          TO* __restrict__ topv_row, int64_t* __restrict__ topi_row, int lane,
                                          int n_group = 0, int topk_group = 0, bool softmax = true,
                                          float scale = 1.f, float* __restrict__ pseudo_row = nullptr) {
  float key[kTopkNV];  // what is ranked: the logit (-inf once masked by the group limit)
  unsigned alive = 0u;  // bit j: expert lane + 64*j exists and has not been selected yet
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < kTopkNV; ++j) {
    const int e = lane + 64 * j;
    key[j] = -INFINITY;
    if (64 * j < E) {  // uniform: whole groups of 64 experts that do not exist cost nothing
      if (e < E) {
        key[j] = Elem<TL>::load(row + e);
        alive |= 1u << j;
      }
      m = fmaxf(m, key[j]);
    }
  }
  float s = 1.f;
  if (softmax) {
    m = wave_max(m);
    s = 0.f;
#pragma unroll
    for (int j = 0; j < kTopkNV; ++j) s += ((alive >> j) & 1u) ? expf(key[j] - m) : 0.f;
    s = wave_sum(s);
  }

  if (n_group > 1) {
    // group-limited selection: the experts form n_group equal runs of ids; a group's score is
    // its largest probability, i.e. that of its largest logit; the topk_group best groups
    // (score descending, then lower group id) stay; every other expert's probability becomes
    // 0 and still takes part in the top-k -- here: its key becomes -inf, whose probability is 0
    const int gsz = E / n_group;
    float gscore = -INFINITY;  // lane g < n_group: score of group g
    for (int g = 0; g < n_group; ++g) {
      float gm = -INFINITY;
#pragma unroll
      for (int j = 0; j < kTopkNV; ++j) {
        const int e = lane + 64 * j;
        if (e < E && e / gsz == g) gm = fmaxf(gm, key[j]);
      }
      gm = wave_max(gm);
      if (lane == g) gscore = gm;
    }
    unsigned long long keep = 0ull, taken = 0ull;
    for (int r = 0; r < topk_group; ++r) {
      const bool cand = lane < n_group && !((taken >> lane) & 1ull);
      const float wv = wave_max(cand ? gscore : -INFINITY);
      const int wi = wave_min_int((cand && gscore == wv) ? lane : 0x7fffffff);
      keep |= 1ull << wi;
      taken |= 1ull << wi;
    }
#pragma unroll
    for (int j = 0; j < kTopkNV; ++j) {
      const int e = lane + 64 * j;
      if (e < E && !((keep >> (e / gsz)) & 1ull)) key[j] = -INFINITY;
    }
  }

  float sel_v = 0.f;  // lane r keeps the r-th selection
  int sel_i = 0;
  float sum_sel = 0.f;
  for (int r = 0; r < K; ++r) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;  // a lane without a candidate never wins the id comparison
#pragma unroll
    for (int j = 0; j < kTopkNV; ++j) {
      // ascending j == ascending id, so strict > keeps the lower id among equal keys
      if (((alive >> j) & 1u) && (bi == 0x7fffffff || key[j] > bv)) {
        bv = key[j];
        bi = lane + 64 * j;
      }
    }
    const float wv = wave_max(bv);
    const int wi = wave_min_int(bv == wv ? bi : 0x7fffffff);
    // every lane now holds the winner; its owner retires it
    if ((wi & 63) == lane) alive &= ~(1u << (wi >> 6));
    const float pv = softmax ? expf(wv - m) / s : wv;
    if (lane == r) {
      sel_v = pv;
      sel_i = wi;
    }
    sum_sel += pv;
  }
  if (pseudo_row != nullptr) {
    // pseudo logits (utils/eval_core.py:9490-9499): -inf everywhere but at the selected experts
#pragma unroll
    for (int j = 0; j < kTopkNV; ++j)
      if (lane + 64 * j < E) pseudo_row[lane + 64 * j] = -INFINITY;
  }
  if (lane < K) {
    float v = sel_v;
    if (renorm) v = v / fmaxf(sum_sel, 1e-12f);
    v *= scale;   // the routed scaling factor, applied in fp32 before the one rounding to the output type
    Elem<TO>::store(topv_row + lane, v);
    topi_row[lane] = static_cast<int64_t>(sel_i);
    // ... where they hold the log of the weight as the layer will use it (rounded), clamped at 1e-12;
    // a lane's stores to one address keep their order
    if (pseudo_row != nullptr) pseudo_row[sel_i] = logf(fmaxf(Elem<TO>::round(v), 1e-12f));
  }
  return sel_i;  // lane r < K: the r-th selected expert
}

template <typename TL, typename TO>
__global__ __launch_bounds__(kTopkWaves * 64) void gate_topk_kernel(
    const TL* __restrict__ logits, int Ttok, int E, int K, int renorm, TO* __restrict__ topv,
    int64_t* __restrict__ topi, int n_group, int topk_group, int softmax, float scale, float* __restrict__ pseudo) {
  const int t = blockIdx.x * kTopkWaves + (threadIdx.x >> 6);
  if (t >= Ttok) return;
  topk_token<TL, TO>(logits + static_cast<size_t>(t) * E, E, K, renorm, topv + static_cast<size_t>(t) * K,
                     topi + static_cast<size_t>(t) * K, threadIdx.x & 63, n_group, topk_group, softmax != 0, scale,
                     pseudo != nullptr ? pseudo + static_cast<size_t>(t) * E : nullptr);
}

// Pseudo logits of a routing that was not computed here (utils/eval_core.py:11137-11155, the replayed
// prediction of the previous layer): `fill` everywhere but at the K given experts of a token, which hold
// log(max(weight, eps)).  One wavefront per token.
template <typename TV>
__global__ __launch_bounds__(kTopkWaves * 64) void pseudo_logits_kernel(const TV* __restrict__ topv,
                                                                        const int64_t* __restrict__ topi, int Ttok,
                                                                        int K, int E, float eps, float fill,
                                                                        float* __restrict__ out) {
  const int t = blockIdx.x * kTopkWaves + (threadIdx.x >> 6);
  if (t >= Ttok) return;
  const int lane = threadIdx.x & 63;
  float* row = out + static_cast<size_t>(t) * E;
  for (int e = lane; e < E; e += 64) {
    float v = fill;
    for (int k = 0; k < K; ++k)   // (the last slot that names an expert wins, as a scatter in slot order would have it)
      if (topi[static_cast<size_t>(t) * K + k] == e) v = logf(fmaxf(Elem<TV>::load(topv + static_cast<size_t>(t) * K + k), eps));
    row[e] = v;
  }
}

// ---------------------------------------------------------------------------
// Decode router in one launch (T <= 32).  Workgroup t owns token t: its 16 wavefronts
// compute the token's E logits (and the shared gate), four weight rows per wavefront at
// a time with the activation chunk shared between them, the values meet in LDS and
// wavefront 0 runs softmax/top-k on them -- so no workgroup waits for another up to
// here.  The workgroup that finishes last (a device atomic behind a fence) builds the
// permutation of all T*K items from one 32-bit token mask per expert and puts the
// counter back to zero for the next launch.
// ---------------------------------------------------------------------------
struct RouteArgs {
  const void* x;
  const void* wg;
  const void* wsg;
  void* logits;
  void* shared_gate;
  void* topv;
  int64_t* topi;
  int32_t* perm;
  int32_t* inv_perm;
  int32_t* seg_offsets;
  int32_t* active_eids;
  int32_t* n_active;
  int32_t* counter;
  int32_t T, H, E, K, renorm;
  int32_t packed_shared_gate;  // packed gate matrix only: row E is the shared-expert gate vector
};

constexpr int kRouteThreads = 1024;
constexpr int kRouteWaves = kRouteThreads / 64;
constexpr int kRouteRowsPerWave = 4;

// Stable bucketing of T*K items (T <= 32) by expert id, run by one 1024-thread block.
// A token picks an expert at most once, so bit t of mask[e] says "token t chose e" and
// the rank of item (t, k) inside its segment is the popcount of the bits below t.
__device__ __forceinline__ void permute_small_block(const int64_t* __restrict__ topi, int T, int K, int E,
                                                    int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm,
                                                    int32_t* __restrict__ seg_offsets,
                                                    int32_t* __restrict__ active_eids,
                                                    int32_t* __restrict__ n_active) {
  __shared__ __attribute__((aligned(16))) uint32_t mask[SPARSE_HIP_MAX_EXPERTS];
  __shared__ int32_t base[SPARSE_HIP_MAX_EXPERTS];
  const int tid = threadIdx.x;
  if (tid < SPARSE_HIP_MAX_EXPERTS) mask[tid] = 0u;
  __syncthreads();
  const int n = T * K;
  int e = -1, t = 0;
  if (tid < n) {
    const int64_t ev = topi[tid];
    t = tid / K;
    if (ev >= 0 && ev < E) {
      e = static_cast<int>(ev);
      atomicOr(&mask[e], 1u << t);
    }
  }
  __syncthreads();
  // thread e < E owns expert e: segment start = items of lower ids (an exclusive prefix sum
  // of the popcounts, scanned inside each wavefront and carried across the at most four
  // wavefronts through LDS), rank among the active experts likewise
  constexpr int kScanWaves = SPARSE_HIP_MAX_EXPERTS / 64;
  __shared__ int32_t wave_items[kScanWaves], wave_active[kScanWaves];
  const int lane = tid & 63, wave = tid >> 6;
  int32_t mine = 0, upto = 0, act = 0;
  if (tid < SPARSE_HIP_MAX_EXPERTS) {
    mine = (tid < E) ? __popc(mask[tid]) : 0;
    upto = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int32_t below = __shfl_up(upto, d);
      if (lane >= d) upto += below;
    }
    const unsigned long long has = __ballot(mine > 0);
    act = __popcll(has & ((1ull << lane) - 1ull));
    if (lane == 63) {
      wave_items[wave] = upto;
      wave_active[wave] = __popcll(has);
    }
  }
  if (E > 64) {  // the same for every thread of the block
    __syncthreads();
    if (tid < SPARSE_HIP_MAX_EXPERTS) {
      for (int w = 0; w < wave; ++w) {
        upto += wave_items[w];
        act += wave_active[w];
      }
    }
  }
  if (tid < E) {
    const int32_t off = upto - mine;
    base[tid] = off;
    seg_offsets[tid] = off;
    if (mine > 0) active_eids[act] = tid;
    if (tid == E - 1) {
      seg_offsets[E] = upto;
      n_active[0] = act + (mine > 0);
    }
  }
  __syncthreads();
  if (e >= 0) {
    const int32_t pos = base[e] + __popc(mask[e] & ((1u << t) - 1u));
    perm[pos] = tid;
    inv_perm[tid] = pos;
  }
}

template <typename T, typename TL>
__global__ __launch_bounds__(kRouteThreads) void route_decode_kernel(const RouteArgs a) {
  __shared__ float s_logit[SPARSE_HIP_MAX_EXPERTS];
  __shared__ int s_last;
  constexpr int kSweeps = sizeof(T) == 2 ? 4 : 1;  // 16-byte loads in flight per row: 4 (bf16), 2 (fp32)
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int E = a.E, H = a.H;
  const int R = E + (a.wsg != nullptr ? 1 : 0);  // row E is the shared-expert gate vector
  const T* x = static_cast<const T*>(a.x) + static_cast<size_t>(t) * H;
  const T* wg = static_cast<const T*>(a.wg);
  TL* logits = static_cast<TL*>(a.logits) + static_cast<size_t>(t) * E;

  for (int r0 = 0; r0 < R; r0 += kRouteWaves * kRouteRowsPerWave) {
    const T* wrow[kRouteRowsPerWave];
    float acc[kRouteRowsPerWave];
#pragma unroll
    for (int j = 0; j < kRouteRowsPerWave; ++j) {
      const int r = r0 + wave + kRouteWaves * j;
      wrow[j] = (r < E) ? wg + static_cast<size_t>(r) * H
                        : (r == E && a.wsg != nullptr ? static_cast<const T*>(a.wsg) : wg);
      acc[j] = 0.f;
    }
    for (int hh = 0; hh < H; hh += kSweeps * 512) {
      Raw8<T> rx[kSweeps], rw[kSweeps][kRouteRowsPerWave];
      bool ok[kSweeps];
#pragma unroll
      for (int sw = 0; sw < kSweeps; ++sw) {
        const int h = hh + sw * 512 + lane * 8;
        ok[sw] = h < H;
        const int hc = ok[sw] ? h : 0;
        rx[sw].load(x + hc);
#pragma unroll
        for (int j = 0; j < kRouteRowsPerWave; ++j) rw[sw][j].load(wrow[j] + hc);
      }
      __builtin_amdgcn_sched_barrier(0);  // every load of the span is in flight before the first use
#pragma unroll
      for (int sw = 0; sw < kSweeps; ++sw) {
        float xv[8];
        rx[sw].widen(xv);
#pragma unroll
        for (int i = 0; i < 8; ++i) xv[i] = ok[sw] ? xv[i] : 0.f;
#pragma unroll
        for (int j = 0; j < kRouteRowsPerWave; ++j) {
          float wv[8];
          rw[sw][j].widen(wv);
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[j] = fmaf(xv[i], wv[i], acc[j]);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < kRouteRowsPerWave; ++j) {
      const int r = r0 + wave + kRouteWaves * j;
      const float s = wave_sum(acc[j]);
      if (lane == 0) {
        if (r < E) {
          Elem<TL>::store(logits + r, s);
          s_logit[r] = Elem<TL>::round(s);
        } else if (r == E && a.wsg != nullptr) {
          Elem<T>::store(static_cast<T*>(a.shared_gate) + t, s);
        }
      }
    }
  }
  __syncthreads();
  if (wave == 0)
    topk_token<float, T>(s_logit, E, a.K, a.renorm, static_cast<T*>(a.topv) + static_cast<size_t>(t) * a.K,
                         a.topi + static_cast<size_t>(t) * a.K, lane);
  if (gridDim.x > 1) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");  // this token's top-k is visible before it is counted
    __syncthreads();
    if (threadIdx.x == 0) {
      const int prev = atomicAdd(a.counter, 1);
      s_last = (prev == static_cast<int>(gridDim.x) - 1);
    }
    __syncthreads();
    if (!s_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (threadIdx.x == 0) a.counter[0] = 0;
  } else {
    __syncthreads();
  }
  permute_small_block(a.topi, a.T, a.K, E, a.perm, a.inv_perm, a.seg_offsets, a.active_eids, a.n_active);
}

// ---------------------------------------------------------------------------
// Decode router for up to 16 bf16 tokens in ONE workgroup, on a gate matrix packed ahead of
// time: 64 rows (the E <= 64 gate rows, then the shared-expert gate vector when there is
// one, then zero rows) in the tiled weight layout, so that every load instruction of a
// wavefront reads 1 KB straight, as the expert kernels do.  No step waits for another
// workgroup or reads its own results back from memory: the 16 wavefronts take the 64-wide
// k blocks in turn and multiply the token rows (A operand) with the four 16-row groups (B
// operand) as 16x16x32 MFMAs, two blocks = 20 loads in flight before the first MFMA; the 16
// partial tiles are folded to 8 and summed in wavefront order in LDS; wavefront t runs
// softmax/top-k of token t on the LDS copy of its logits, and the permutation is built from
// the selections kept in LDS.
// ---------------------------------------------------------------------------
constexpr int kRpTok = SPARSE_HIP_ROUTE_PACKED_MAX_TOKENS;
static_assert(kRpTok == kRouteWaves && SPARSE_HIP_ROUTE_PACKED_ROWS == kRlRows, "one wavefront per token, four 16-row groups");

template <typename T16, typename TL>
__device__ __forceinline__ void route_packed_block(const RouteArgs& a) {
  using F = typename FormatOf<T16>::type;
  __shared__ float part[kRouteWaves / 2][kRpTok][kRlPad];
  __shared__ float s_logit[kRpTok][kRlRows];
  __shared__ int64_t s_topi[kRpTok * SPARSE_HIP_MAX_TOPK];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, q = lane >> 4;
  const int T = a.T, H = a.H, E = a.E;
  const int R = E + (a.packed_shared_gate ? 1 : 0);
  const uint16_t* xrow = static_cast<const uint16_t*>(a.x) + static_cast<size_t>(min(r, T - 1)) * H + q * 16;
  const uint16_t* wt = static_cast<const uint16_t*>(a.wg) + lane * 8;
  const size_t group_stride = static_cast<size_t>(16) * H;
  const int nblk = H >> 6;
  f32x4 acc[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  int b = wave;
  for (; b + kRouteWaves < nblk; b += 2 * kRouteWaves) {
    bf16x8 av[2][2], bv[2][4][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int blk = b + j * kRouteWaves;
      av[j][0] = *reinterpret_cast<const bf16x8*>(xrow + blk * 64);
      av[j][1] = *reinterpret_cast<const bf16x8*>(xrow + blk * 64 + 8);
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const uint16_t* p = wt + nt * group_stride + static_cast<size_t>(blk) * 1024;
        bv[j][nt][0] = *reinterpret_cast<const bf16x8*>(p);
        bv[j][nt][1] = *reinterpret_cast<const bf16x8*>(p + 512);
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // all 20 loads in flight before the first MFMA
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
          acc[nt] = F::mfma16(av[j][h], bv[j][nt][h], acc[nt]);
  }
  if (b < nblk) {
    const bf16x8 av0 = *reinterpret_cast<const bf16x8*>(xrow + b * 64);
    const bf16x8 av1 = *reinterpret_cast<const bf16x8*>(xrow + b * 64 + 8);
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const uint16_t* p = wt + nt * group_stride + static_cast<size_t>(b) * 1024;
      acc[nt] = F::mfma16(av0, *reinterpret_cast<const bf16x8*>(p), acc[nt]);
      acc[nt] = F::mfma16(av1, *reinterpret_cast<const bf16x8*>(p + 512), acc[nt]);
    }
  }
  // D: lane holds gate row nt*16 + r for tokens q*4 .. q*4+3.  Wavefronts 8..15 hand their
  // tiles to wavefronts 0..7, whose sums are then added in wavefront order.
  if (wave >= kRouteWaves / 2) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int v = 0; v < 4; ++v) part[wave - kRouteWaves / 2][q * 4 + v][nt * 16 + r] = acc[nt][v];
  }
  __syncthreads();
  if (wave < kRouteWaves / 2) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int v = 0; v < 4; ++v) part[wave][q * 4 + v][nt * 16 + r] += acc[nt][v];
  }
  __syncthreads();
  {
    const int tok = tid >> 6, col = tid & 63;
    float sum = part[0][tok][col];
#pragma unroll
    for (int w = 1; w < kRouteWaves / 2; ++w) sum += part[w][tok][col];
    if (tok < T && col < R) {
      if (col < E) {
        Elem<TL>::store(static_cast<TL*>(a.logits) + static_cast<size_t>(tok) * E + col, sum);
        s_logit[tok][col] = Elem<TL>::round(sum);
      } else {
        static_cast<uint16_t*>(a.shared_gate)[tok] = F::bits(sum);
      }
    }
  }
  __syncthreads();
  if (wave < T) {
    const int sel = topk_token<float, T16>(s_logit[wave], E, a.K, a.renorm,
                                           static_cast<T16*>(a.topv) + static_cast<size_t>(wave) * a.K,
                                           a.topi + static_cast<size_t>(wave) * a.K, lane);
    if (lane < a.K) s_topi[wave * a.K + lane] = static_cast<int64_t>(sel);
  }
  __syncthreads();
  permute_small_block(s_topi, T, a.K, E, a.perm, a.inv_perm, a.seg_offsets, a.active_eids, a.n_active);
}

template <typename T16, typename TL>
__global__ __launch_bounds__(kRouteThreads) void route_decode_packed_kernel(const RouteArgs a) {
  route_packed_block<T16, TL>(a);
}

// ---------------------------------------------------------------------------
// The same routing workgroup, and beside it -- routing is one workgroup's work and leaves the
// memory system idle -- the shared expert's gate and up projections with SiLU*up, which need
// the token rows only: workgroup 1 + j computes rows 32 j .. 32 j + 31 of both matrices for
// all (at most 16) tokens.  Its 16 wavefronts cut the reduction into 64-wide slices dealt
// round-robin and request every slice they own before the first MFMA, so the whole of the two
// matrices is in flight at once; the 16 partial tiles meet in LDS and are added in wavefront
// order.  Operand layouts, the tiled weight format and the epilogue's roundings are those of
// the decode expert kernel (swiglu_decode.hip).
// ---------------------------------------------------------------------------
struct SharedUpArgs {
  const uint16_t* gate_w;   // [Is, H] tiled
  const uint16_t* up_w;     // [Is, H] tiled
  const uint16_t* x;        // [T, H]
  uint16_t* inter;          // [T, Is]: silu(gate x) * (up x)
  int32_t T, H, Is;
};

constexpr int kSuRows = 32;   // output rows per workgroup: two 16-row MFMA tiles

template <typename F>
__device__ __forceinline__ void shared_gateup_block(const SharedUpArgs& s, int tile) {
  __shared__ f32x4 red[kRouteWaves][4][64];   // [wavefront][2 * row tile + matrix][lane]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int H = s.H, ND = H >> 6;
  const size_t group_stride = static_cast<size_t>(16) * H;
  const uint16_t* wt[2] = {s.gate_w + static_cast<size_t>(tile * 2) * group_stride + lane * 8,
                           s.up_w + static_cast<size_t>(tile * 2) * group_stride + lane * 8};
  // token column r (columns past T read token 0: their products are never stored)
  const uint16_t* brow = s.x + static_cast<size_t>(r < s.T ? r : 0) * H + (q << 4);
  f32x4 acc[2][2];   // [row tile][matrix]
#pragma unroll
  for (int tl = 0; tl < 2; ++tl)
#pragma unroll
    for (int m = 0; m < 2; ++m) acc[tl][m] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int d0 = wave; d0 < ND; d0 += 2 * kRouteWaves) {
    const int d1 = d0 + kRouteWaves;           // this wavefront's next slice, if there is one
    const int dd[2] = {d0, d1 < ND ? d1 : d0};
    bf16x8 b[2][2], w[2][2][2][2];             // [slice][k half], [slice][row tile][matrix][k half]
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      b[j][0] = *reinterpret_cast<const bf16x8*>(brow + (dd[j] << 6));
      b[j][1] = *reinterpret_cast<const bf16x8*>(brow + (dd[j] << 6) + 8);
#pragma unroll
      for (int tl = 0; tl < 2; ++tl)
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          const uint16_t* p = wt[m] + tl * group_stride + (static_cast<size_t>(dd[j]) << 10);
          w[j][tl][m][0] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p));
          w[j][tl][m][1] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p + 512));
        }
    }
    __builtin_amdgcn_sched_barrier(0);          // all 20 loads in flight before the first MFMA
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if (j == 1 && d1 >= ND) break;
#pragma unroll
      for (int tl = 0; tl < 2; ++tl)
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          acc[tl][m] = F::mfma16(w[j][tl][m][0], b[j][0], acc[tl][m]);
          acc[tl][m] = F::mfma16(w[j][tl][m][1], b[j][1], acc[tl][m]);
        }
    }
  }
#pragma unroll
  for (int tl = 0; tl < 2; ++tl)
#pragma unroll
    for (int m = 0; m < 2; ++m) red[wave][tl * 2 + m][lane] = acc[tl][m];
  __syncthreads();
  // wavefront tl finishes row tile tl: lane (r, q) holds rows 4 q .. 4 q + 3 of token r
  if (wave < 2 && r < s.T) {
    const int tl = wave;
    f32x4 g = red[0][tl * 2][lane], u = red[0][tl * 2 + 1][lane];
#pragma unroll
    for (int w2 = 1; w2 < kRouteWaves; ++w2) {
      g += red[w2][tl * 2][lane];
      u += red[w2][tl * 2 + 1][lane];
    }
    uint16_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float gv = F::round(g[j]), uv = F::round(u[j]);
      o[j] = F::bits(F::round(silu_f32(gv)) * uv);
    }
    uint2 pk;
    pk.x = static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16);
    pk.y = static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16);
    *reinterpret_cast<uint2*>(s.inter + static_cast<size_t>(r) * s.Is + tile * kSuRows + tl * 16 + q * 4) = pk;
  }
}

// the shared expert's half alone, for callers that route some other way
template <typename F>
__global__ __launch_bounds__(kRouteThreads) void shared_gateup_kernel(const SharedUpArgs s) {
  shared_gateup_block<F>(s, static_cast<int>(blockIdx.x));
}

template <typename T16, typename TL>
__global__ __launch_bounds__(kRouteThreads) void route_packed_shared_kernel(const RouteArgs a, const SharedUpArgs s) {
  if (blockIdx.x == 0) {
    route_packed_block<T16, TL>(a);
  } else {
    shared_gateup_block<typename FormatOf<T16>::type>(s, static_cast<int>(blockIdx.x) - 1);
  }
}

template <typename T, typename TL>
static int launch_router_logits(const void* x, const void* wg, const void* wsg, int Ttok, int H, int E,
                                void* logits, void* shared_gate, hipStream_t st) {
  if constexpr (sizeof(T) == 2) {
    if (Ttok >= 64 && H % 512 == 0) {
      ProfScope prof(SPARSE_HIP_K_ROUTER_LOGITS, st);
      hipLaunchKernelGGL((router_logits_mfma_kernel<typename FormatOf<T>::type, TL>),
                         dim3((Ttok + kRlTok - 1) / kRlTok), dim3(256), 0, st,
                         static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(wg),
                         static_cast<const uint16_t*>(wsg), Ttok, H, E, static_cast<TL*>(logits),
                         static_cast<uint16_t*>(shared_gate));
      SP_LAUNCH_CHECK("router_logits_mfma_kernel");
      return SPARSE_HIP_OK;
    }
  }
  dim3 grid(E + (wsg != nullptr ? 1 : 0), (Ttok + kRouterTokTile - 1) / kRouterTokTile);
  ProfScope prof(SPARSE_HIP_K_ROUTER_LOGITS, st);
  hipLaunchKernelGGL((router_logits_kernel<T, TL>), grid, dim3(kRouterThreads), 0, st,
                     static_cast<const T*>(x), static_cast<const T*>(wg), static_cast<const T*>(wsg), Ttok,
                     H, E, static_cast<TL*>(logits), static_cast<T*>(shared_gate));
  SP_LAUNCH_CHECK("router_logits_kernel");
  return SPARSE_HIP_OK;
}

template <typename TL, typename TO>
static int launch_gate_topk(const void* logits, int Ttok, int E, int K, int renorm, void* topv,
                            int64_t* topi, hipStream_t st, int n_group = 0, int topk_group = 0, int softmax = 1,
                            float scale = 1.f, float* pseudo = nullptr) {
  dim3 grid((Ttok + kTopkWaves - 1) / kTopkWaves);
  ProfScope prof(SPARSE_HIP_K_GATE_TOPK, st);
  hipLaunchKernelGGL((gate_topk_kernel<TL, TO>), grid, dim3(kTopkWaves * 64), 0, st,
                     static_cast<const TL*>(logits), Ttok, E, K, renorm, static_cast<TO*>(topv), topi, n_group,
                     topk_group, softmax, scale, pseudo);
  SP_LAUNCH_CHECK("gate_topk_kernel");
  return SPARSE_HIP_OK;
}

template <typename T, typename TL>
static int launch_route_decode(const RouteArgs& a, hipStream_t st) {
  ProfScope prof(SPARSE_HIP_K_ROUTE_DECODE, st);
  hipLaunchKernelGGL((route_decode_kernel<T, TL>), dim3(a.T), dim3(kRouteThreads), 0, st, a);
  SP_LAUNCH_CHECK("route_decode_kernel");
  return SPARSE_HIP_OK;
}

}  // namespace sparse

using namespace sparse;

template <typename T16, typename TL>
static void launch_route_packed(const RouteArgs& a, const SharedUpArgs* shared, hipStream_t st) {
  if (shared != nullptr) {
    const dim3 grid(1 + shared->Is / kSuRows);
    hipLaunchKernelGGL((route_packed_shared_kernel<T16, TL>), grid, dim3(kRouteThreads), 0, st, a, *shared);
  } else {
    hipLaunchKernelGGL((route_decode_packed_kernel<T16, TL>), dim3(1), dim3(kRouteThreads), 0, st, a);
  }
}

extern "C" {

int sparse_hip_router_logits(const void* x_dev, const void* wg_dev, const void* wsg_dev, int dtype,
                             int logits_dtype, int T, int H, int E, void* logits_dev,
                             void* shared_gate_dev, void* stream) {
  SP_REQUIRE(valid_dtype(dtype) && valid_dtype(logits_dtype), "router_logits: unknown dtype");
  SP_REQUIRE(logits_dtype == dtype || logits_dtype == SPARSE_HIP_F32,
             "router_logits: logits_dtype must equal dtype or be fp32");
  SP_REQUIRE(T >= 0 && H > 0 && E > 0, "router_logits: bad shape T=%d H=%d E=%d", T, H, E);
  SP_REQUIRE(H % 8 == 0, "router_logits: H=%d must be a multiple of 8", H);
  SP_REQUIRE(x_dev && wg_dev && logits_dev, "router_logits: NULL pointer");
  SP_REQUIRE(wsg_dev == nullptr || shared_gate_dev != nullptr, "router_logits: shared gate output is NULL");
  if (T == 0) return SPARSE_HIP_OK;
  hipStream_t st = as_stream(stream);
  if (dtype == SPARSE_HIP_F32)
    return launch_router_logits<float, float>(x_dev, wg_dev, wsg_dev, T, H, E, logits_dev, shared_gate_dev, st);
  if (dtype == SPARSE_HIP_F16) {
    if (logits_dtype == SPARSE_HIP_F32)
      return launch_router_logits<f16_t, float>(x_dev, wg_dev, wsg_dev, T, H, E, logits_dev, shared_gate_dev, st);
    return launch_router_logits<f16_t, f16_t>(x_dev, wg_dev, wsg_dev, T, H, E, logits_dev, shared_gate_dev, st);
  }
  if (logits_dtype == SPARSE_HIP_F32)
    return launch_router_logits<uint16_t, float>(x_dev, wg_dev, wsg_dev, T, H, E, logits_dev, shared_gate_dev, st);
  return launch_router_logits<uint16_t, uint16_t>(x_dev, wg_dev, wsg_dev, T, H, E, logits_dev, shared_gate_dev, st);
}

int sparse_hip_gate_topk(const void* logits_dev, int logits_dtype, int T, int E, int K, int renorm,
                         int out_dtype, void* topv_dev, int64_t* topi_dev, void* stream) {
  return sparse_hip_gate_topk_grouped(logits_dev, logits_dtype, T, E, K, renorm, 1, 1, out_dtype, topv_dev, topi_dev,
                                      stream);
}

int sparse_hip_gate_topk_grouped(const void* logits_dev, int logits_dtype, int T, int E, int K, int renorm,
                                 int n_group, int topk_group, int out_dtype, void* topv_dev, int64_t* topi_dev,
                                 void* stream) {
  return sparse_hip_gate_topk_scaled(logits_dev, logits_dtype, T, E, K, renorm, n_group, topk_group, 1.0f, out_dtype,
                                     topv_dev, topi_dev, nullptr, stream);
}

int sparse_hip_gate_topk_scaled(const void* logits_dev, int logits_dtype, int T, int E, int K, int renorm,
                                int n_group, int topk_group, float scale, int out_dtype, void* topv_dev,
                                int64_t* topi_dev, float* pseudo_logits_dev, void* stream) {
  SP_REQUIRE(scale == scale && scale > 0.f, "gate_topk: scale must be positive");
  SP_REQUIRE(valid_dtype(logits_dtype) && valid_dtype(out_dtype), "gate_topk: unknown dtype");
  SP_REQUIRE(n_group >= 1 && n_group <= 64 && E % n_group == 0, "gate_topk: n_group=%d must divide E=%d and be <= 64",
             n_group, E);
  SP_REQUIRE(topk_group >= 1 && topk_group <= n_group, "gate_topk: topk_group=%d outside [1,n_group=%d]", topk_group,
             n_group);
  SP_REQUIRE(T >= 0, "gate_topk: T=%d", T);
  SP_REQUIRE(E >= 1 && E <= SPARSE_HIP_MAX_EXPERTS, "gate_topk: E=%d outside [1,%d]", E, SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(K >= 1 && K <= SPARSE_HIP_MAX_TOPK && K <= E, "gate_topk: K=%d outside [1,min(%d,E)]", K,
             SPARSE_HIP_MAX_TOPK);
  SP_REQUIRE(logits_dev && topv_dev && topi_dev, "gate_topk: NULL pointer");
  if (T == 0) return SPARSE_HIP_OK;
  hipStream_t st = as_stream(stream);
  SP_REQUIRE(!(is_16bit(logits_dtype) && is_16bit(out_dtype)) || logits_dtype == out_dtype,
             "gate_topk: 16-bit logits and 16-bit weights must be of the same format");
  const int ng = (n_group > 1 && topk_group < n_group) ? n_group : 0;  // every group kept = plain top-k
#define SP_TOPK_CASE(LD, OD, TL, TO)                                                                          \
  if (logits_dtype == (LD) && out_dtype == (OD))                                                              \
    return launch_gate_topk<TL, TO>(logits_dev, T, E, K, renorm, topv_dev, topi_dev, st, ng, topk_group, 1, scale, \
                                    pseudo_logits_dev);
  SP_TOPK_CASE(SPARSE_HIP_BF16, SPARSE_HIP_BF16, uint16_t, uint16_t)
  SP_TOPK_CASE(SPARSE_HIP_BF16, SPARSE_HIP_F32, uint16_t, float)
  SP_TOPK_CASE(SPARSE_HIP_F32, SPARSE_HIP_BF16, float, uint16_t)
  SP_TOPK_CASE(SPARSE_HIP_F16, SPARSE_HIP_F16, f16_t, f16_t)
  SP_TOPK_CASE(SPARSE_HIP_F16, SPARSE_HIP_F32, f16_t, float)
  SP_TOPK_CASE(SPARSE_HIP_F32, SPARSE_HIP_F16, float, f16_t)
#undef SP_TOPK_CASE
  return launch_gate_topk<float, float>(logits_dev, T, E, K, renorm, topv_dev, topi_dev, st, ng, topk_group, 1, scale,
                                        pseudo_logits_dev);
}

int sparse_hip_pseudo_logits(const void* topv_dev, int dtype, const int64_t* topi_dev, int T, int K, int E, float eps,
                             float fill, float* out_dev, void* stream) {
  SP_REQUIRE(valid_dtype(dtype), "pseudo_logits: unknown dtype %d", dtype);
  SP_REQUIRE(T >= 0, "pseudo_logits: T=%d", T);
  SP_REQUIRE(E >= 1 && K >= 1 && K <= SPARSE_HIP_MAX_TOPK, "pseudo_logits: E=%d, K=%d (K at most %d)", E, K,
             SPARSE_HIP_MAX_TOPK);
  SP_REQUIRE(eps > 0.f, "pseudo_logits: eps must be positive");
  SP_REQUIRE(topv_dev && topi_dev && out_dev, "pseudo_logits: NULL pointer");
  if (T == 0) return SPARSE_HIP_OK;
  hipStream_t st = as_stream(stream);
  dim3 grid((T + kTopkWaves - 1) / kTopkWaves);
  if (dtype == SPARSE_HIP_F32) {
    hipLaunchKernelGGL((pseudo_logits_kernel<float>), grid, dim3(kTopkWaves * 64), 0, st,
                       static_cast<const float*>(topv_dev), topi_dev, T, K, E, eps, fill, out_dev);
  } else if (dtype == SPARSE_HIP_F16) {
    hipLaunchKernelGGL((pseudo_logits_kernel<f16_t>), grid, dim3(kTopkWaves * 64), 0, st,
                       static_cast<const f16_t*>(topv_dev), topi_dev, T, K, E, eps, fill, out_dev);
  } else {
    hipLaunchKernelGGL((pseudo_logits_kernel<uint16_t>), grid, dim3(kTopkWaves * 64), 0, st,
                       static_cast<const uint16_t*>(topv_dev), topi_dev, T, K, E, eps, fill, out_dev);
  }
  SP_LAUNCH_CHECK("pseudo_logits_kernel");
  return SPARSE_HIP_OK;
}

int sparse_hip_topk(const void* values_dev, int T, int E, int K, int renorm, int out_dtype, void* topv_dev,
                    int64_t* topi_dev, void* stream) {
  SP_REQUIRE(valid_dtype(out_dtype), "topk: unknown dtype");
  SP_REQUIRE(T >= 0, "topk: T=%d", T);
  SP_REQUIRE(E >= 1 && E <= SPARSE_HIP_MAX_EXPERTS, "topk: E=%d outside [1,%d]", E, SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(K >= 1 && K <= SPARSE_HIP_MAX_TOPK && K <= E, "topk: K=%d outside [1,min(%d,E)]", K, SPARSE_HIP_MAX_TOPK);
  SP_REQUIRE(values_dev && topv_dev && topi_dev, "topk: NULL pointer");
  if (T == 0) return SPARSE_HIP_OK;
  hipStream_t st = as_stream(stream);
  if (out_dtype == SPARSE_HIP_BF16)
    return launch_gate_topk<float, uint16_t>(values_dev, T, E, K, renorm, topv_dev, topi_dev, st, 0, 0, 0);
  if (out_dtype == SPARSE_HIP_F16)
    return launch_gate_topk<float, f16_t>(values_dev, T, E, K, renorm, topv_dev, topi_dev, st, 0, 0, 0);
  return launch_gate_topk<float, float>(values_dev, T, E, K, renorm, topv_dev, topi_dev, st, 0, 0, 0);
}

int sparse_hip_route_decode(const void* x_dev, const void* wg_dev, const void* wsg_dev, int dtype,
                            int logits_dtype, int T, int H, int E, int K, int renorm, void* logits_dev,
                            void* shared_gate_dev, void* topv_dev, int64_t* topi_dev, int32_t* perm_dev,
                            int32_t* inv_perm_dev, int32_t* seg_offsets_dev, int32_t* active_eids_dev,
                            int32_t* n_active_dev, int32_t* counter_dev, void* stream) {
  SP_REQUIRE(valid_dtype(dtype) && valid_dtype(logits_dtype), "route_decode: unknown dtype");
  SP_REQUIRE(logits_dtype == dtype || logits_dtype == SPARSE_HIP_F32,
             "route_decode: logits_dtype must equal dtype or be fp32");
  SP_REQUIRE(T >= 1 && T <= SPARSE_HIP_DECODE_MAX_TOKENS, "route_decode: T=%d outside [1,%d]", T,
             SPARSE_HIP_DECODE_MAX_TOKENS);
  SP_REQUIRE(H > 0 && H % 8 == 0, "route_decode: H=%d must be a positive multiple of 8", H);
  SP_REQUIRE(E >= 1 && E <= SPARSE_HIP_MAX_EXPERTS, "route_decode: E=%d outside [1,%d]", E, SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(K >= 1 && K <= SPARSE_HIP_MAX_TOPK && K <= E, "route_decode: K=%d outside [1,min(%d,E)]", K,
             SPARSE_HIP_MAX_TOPK);
  SP_REQUIRE(x_dev && wg_dev && logits_dev && topv_dev && topi_dev && perm_dev && inv_perm_dev && seg_offsets_dev &&
                 active_eids_dev && n_active_dev && counter_dev,
             "route_decode: NULL pointer");
  SP_REQUIRE(wsg_dev == nullptr || shared_gate_dev != nullptr, "route_decode: shared gate output is NULL");
  RouteArgs a = {x_dev,     wg_dev,       wsg_dev,         logits_dev,      shared_gate_dev, topv_dev,   topi_dev,
                 perm_dev,  inv_perm_dev, seg_offsets_dev, active_eids_dev, n_active_dev,    counter_dev,
                 T,         H,            E,               K,               renorm,          0};
  hipStream_t st = as_stream(stream);
  if (dtype == SPARSE_HIP_F32) return launch_route_decode<float, float>(a, st);
  if (dtype == SPARSE_HIP_F16) {
    if (logits_dtype == SPARSE_HIP_F32) return launch_route_decode<f16_t, float>(a, st);
    return launch_route_decode<f16_t, f16_t>(a, st);
  }
  if (logits_dtype == SPARSE_HIP_F32) return launch_route_decode<uint16_t, float>(a, st);
  return launch_route_decode<uint16_t, uint16_t>(a, st);
}

static int route_packed_impl(const void* x_dev, const void* gate_packed_dev, int has_shared_gate, int dtype,
                             int logits_dtype, int T, int H, int E, int K, int renorm, void* logits_dev,
                             void* shared_gate_dev, void* topv_dev, int64_t* topi_dev, int32_t* perm_dev,
                             int32_t* inv_perm_dev, int32_t* seg_offsets_dev, int32_t* active_eids_dev,
                             int32_t* n_active_dev, const SharedUpArgs* shared, void* stream) {
  SP_REQUIRE(is_16bit(dtype), "route_decode_packed: dtype must be bf16 or fp16");
  SP_REQUIRE(logits_dtype == dtype || logits_dtype == SPARSE_HIP_F32,
             "route_decode_packed: logits_dtype must be the activations' dtype or fp32");
  SP_REQUIRE(T >= 1 && T <= SPARSE_HIP_ROUTE_PACKED_MAX_TOKENS, "route_decode_packed: T=%d outside [1,%d]", T,
             SPARSE_HIP_ROUTE_PACKED_MAX_TOKENS);
  SP_REQUIRE(H > 0 && H % 64 == 0, "route_decode_packed: H=%d must be a positive multiple of 64", H);
  SP_REQUIRE(E >= 1 && E + (has_shared_gate ? 1 : 0) <= SPARSE_HIP_ROUTE_PACKED_ROWS,
             "route_decode_packed: E=%d (+ shared gate row) exceeds the %d packed rows", E,
             SPARSE_HIP_ROUTE_PACKED_ROWS);
  SP_REQUIRE(K >= 1 && K <= SPARSE_HIP_MAX_TOPK && K <= E, "route_decode_packed: K=%d outside [1,min(%d,E)]", K,
             SPARSE_HIP_MAX_TOPK);
  SP_REQUIRE(x_dev && gate_packed_dev && logits_dev && topv_dev && topi_dev && perm_dev && inv_perm_dev &&
                 seg_offsets_dev && active_eids_dev && n_active_dev,
             "route_decode_packed: NULL pointer");
  SP_REQUIRE(!has_shared_gate || shared_gate_dev != nullptr, "route_decode_packed: shared gate output is NULL");
  RouteArgs a = {x_dev,    gate_packed_dev, nullptr,         logits_dev,      shared_gate_dev, topv_dev, topi_dev,
                 perm_dev, inv_perm_dev,    seg_offsets_dev, active_eids_dev, n_active_dev,    nullptr,
                 T,        H,               E,               K,               renorm,          has_shared_gate ? 1 : 0};
  hipStream_t st = as_stream(stream);
  ProfScope prof(SPARSE_HIP_K_ROUTE_DECODE, st);
  const bool wide_logits = logits_dtype == SPARSE_HIP_F32;
  if (dtype == SPARSE_HIP_F16) {
    if (wide_logits) launch_route_packed<f16_t, float>(a, shared, st); else launch_route_packed<f16_t, f16_t>(a, shared, st);
  } else {
    if (wide_logits) launch_route_packed<uint16_t, float>(a, shared, st); else launch_route_packed<uint16_t, uint16_t>(a, shared, st);
  }
  SP_LAUNCH_CHECK(shared != nullptr ? "route_packed_shared_kernel" : "route_decode_packed_kernel");
  return SPARSE_HIP_OK;
}

int sparse_hip_route_decode_packed(const void* x_dev, const void* gate_packed_dev, int has_shared_gate, int dtype,
                                   int logits_dtype, int T, int H, int E, int K, int renorm, void* logits_dev,
                                   void* shared_gate_dev, void* topv_dev, int64_t* topi_dev, int32_t* perm_dev,
                                   int32_t* inv_perm_dev, int32_t* seg_offsets_dev, int32_t* active_eids_dev,
                                   int32_t* n_active_dev, void* stream) {
  return route_packed_impl(x_dev, gate_packed_dev, has_shared_gate, dtype, logits_dtype, T, H, E, K, renorm,
                           logits_dev, shared_gate_dev, topv_dev, topi_dev, perm_dev, inv_perm_dev, seg_offsets_dev,
                           active_eids_dev, n_active_dev, nullptr, stream);
}

int sparse_hip_shared_gate_up(const void* x_dev, const void* shared_gate_w_dev, const void* shared_up_w_dev, int dtype,
                              int T, int H, int Is, void* shared_inter_dev, void* stream) {
  SP_REQUIRE(is_16bit(dtype), "shared_gate_up: dtype must be bf16 or fp16");
  SP_REQUIRE(x_dev && shared_gate_w_dev && shared_up_w_dev && shared_inter_dev, "shared_gate_up: NULL pointer");
  SP_REQUIRE(T >= 1 && T <= SPARSE_HIP_ROUTE_PACKED_MAX_TOKENS, "shared_gate_up: T=%d outside [1,%d]", T,
             SPARSE_HIP_ROUTE_PACKED_MAX_TOKENS);
  SP_REQUIRE(H > 0 && H % 64 == 0, "shared_gate_up: H=%d must be a positive multiple of 64", H);
  SP_REQUIRE(Is > 0 && Is % kSuRows == 0, "shared_gate_up: Is=%d must be a positive multiple of %d", Is, kSuRows);
  SharedUpArgs s = {static_cast<const uint16_t*>(shared_gate_w_dev), static_cast<const uint16_t*>(shared_up_w_dev),
                    static_cast<const uint16_t*>(x_dev), static_cast<uint16_t*>(shared_inter_dev), T, H, Is};
  hipStream_t st = as_stream(stream);
  if (dtype == SPARSE_HIP_F16) {
    hipLaunchKernelGGL((shared_gateup_kernel<Fp16>), dim3(Is / kSuRows), dim3(kRouteThreads), 0, st, s);
  } else {
    hipLaunchKernelGGL((shared_gateup_kernel<Bf16>), dim3(Is / kSuRows), dim3(kRouteThreads), 0, st, s);
  }
  SP_LAUNCH_CHECK("shared_gateup_kernel");
  return SPARSE_HIP_OK;
}

int sparse_hip_route_decode_packed_shared(const void* x_dev, const void* gate_packed_dev, int has_shared_gate,
                                          int dtype, int logits_dtype, int T, int H, int E, int K, int renorm,
                                          void* logits_dev, void* shared_gate_dev, void* topv_dev,
                                          int64_t* topi_dev, int32_t* perm_dev, int32_t* inv_perm_dev,
                                          int32_t* seg_offsets_dev, int32_t* active_eids_dev, int32_t* n_active_dev,
                                          const void* shared_gate_w_dev, const void* shared_up_w_dev, int Is,
                                          void* shared_inter_dev, void* stream) {
  SP_REQUIRE(shared_gate_w_dev && shared_up_w_dev && shared_inter_dev, "route_decode_packed_shared: NULL pointer");
  SP_REQUIRE(Is > 0 && Is % kSuRows == 0, "route_decode_packed_shared: Is=%d must be a positive multiple of %d", Is,
             kSuRows);
  SharedUpArgs s = {static_cast<const uint16_t*>(shared_gate_w_dev), static_cast<const uint16_t*>(shared_up_w_dev),
                    static_cast<const uint16_t*>(x_dev), static_cast<uint16_t*>(shared_inter_dev), T, H, Is};
  return route_packed_impl(x_dev, gate_packed_dev, has_shared_gate, dtype, logits_dtype, T, H, E, K, renorm,
                           logits_dev, shared_gate_dev, topv_dev, topi_dev, perm_dev, inv_perm_dev, seg_offsets_dev,
                           active_eids_dev, n_active_dev, &s, stream);
}

}  // extern "C"
