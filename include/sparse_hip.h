/*
 * sparse_hip.h -- C ABI of the MI355X (gfx950) MoE-layer execution path.
 *
 * The reference (louislichen/SPARSE) has no FFI: its MoE layer is a Python class
 * (`DistributedSparseMoeBlock`, utils/eval_core.py:4407-17215) that issues ATen calls.
 * Each entry point below replaces one run of those ATen calls; the comment on each
 * names the reference lines it stands in for.  The Python host in `sparse_amd/`
 * binds them with ctypes; any other host can bind them the same way.
 *
 * Conventions
 *   - Every function returns 0 on success, a negative SPARSE_HIP_E* code otherwise;
 *     `sparse_hip_last_error()` returns a thread-local message for the last failure.
 *   - All pointers named *_dev are device (HBM) pointers; *_host are host pointers.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *   - Nothing here allocates device memory or synchronises the host unless its
 *     comment says so: callers pass workspaces and outputs.  Launches are
 *     asynchronous with respect to the host and may be captured into a HIP graph.
 *   - Activations, logits and outputs are row-major.  Weight matrices are
 *     [out_features, in_features] = [R, K] as in torch.nn.Linear, but stored TILED
 *     (R % 16 == 0, K % 64 == 0): element (row, k) lives at element offset
 *         (row/16)*16*K + (k/64)*1024 + ((k/8)%2)*512 + ((k/16)%4)*128 + (row%16)*8 + k%8
 *     i.e. the K extent of a 16-row group is one contiguous run, cut into 2 KB (bf16)
 *     blocks of 64 k whose two halves are the A operands of two 16x16x32 MFMAs in lane
 *     order.  Streaming a weight matrix is then a sequence of contiguous 1 KB wave
 *     loads; row-major rows 4 KB apart would pile onto the same HBM channels.
 *     `sparse_hip_tile_weight` converts.  The router gate matrix `wg` and the shared
 *     gate vector stay row-major.
 *   - dtype codes: SPARSE_HIP_F32 = 0, SPARSE_HIP_BF16 = 1, SPARSE_HIP_F16 = 2 (IEEE half, the
 *     dtype of the reference's formal runs, scripts/run/run_case.sh:199).  Wherever this file says
 *     bf16 for a kernel's 16-bit path, fp16 takes the same kernel with its own conversions and MFMA.
 */
#ifndef SPARSE_HIP_H
#define SPARSE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPARSE_HIP_ABI_VERSION 3

#define SPARSE_HIP_F32 0
#define SPARSE_HIP_BF16 1
#define SPARSE_HIP_F16 2

#define SPARSE_HIP_OK 0
#define SPARSE_HIP_EINVAL (-1)   /* bad argument (shape, dtype, alignment, NULL) */
#define SPARSE_HIP_ELAUNCH (-2)  /* HIP runtime reported an error */
#define SPARSE_HIP_ENOTREADY 1   /* event_query: work still in flight (not an error) */

/* Largest expert count / top-k / decode batch the kernels are built for. */
#define SPARSE_HIP_MAX_EXPERTS 256
#define SPARSE_HIP_MAX_TOPK 16
#define SPARSE_HIP_DECODE_MAX_TOKENS 32
#define SPARSE_HIP_ROUTE_PACKED_MAX_TOKENS 16
#define SPARSE_HIP_ROUTE_PACKED_ROWS 64
#define SPARSE_HIP_PERMUTE_STATIC_MAX_TOKENS 65536

/* ---- library identity ------------------------------------------------------ */

/* ABI version of the loaded library (SPARSE_HIP_ABI_VERSION at build time). */
int sparse_hip_version(void);
/* Code-object architecture the kernels were built for ("gfx950"). */
const char* sparse_hip_arch(void);
/* Message of the last failure on the calling thread ("" if none). */
const char* sparse_hip_last_error(void);

/* ---- expert weight slab ---------------------------------------------------- */

/*
 * Where the routed experts of one layer live in HBM.  One slot holds one expert:
 * gate [I,H], up [I,H], down [H,I], contiguous in that order, `slot_stride` bytes
 * apart.  `expert_slot_dev[e]` is the slot that currently holds expert e (any value
 * for experts that are not touched by the call).  An all-resident layer uses the
 * identity table.  Replaces the per-expert tensors the reference keeps in
 * `local_gate_cpu/local_up_cpu/local_down_cpu2` and in cache payload tuples
 * (utils/eval_core.py:5097-5123, :11427-11435).
 */
typedef struct sparse_hip_experts {
  const void* slab_dev;            /* base of slot 0 */
  uint64_t slot_stride;            /* bytes between slots (>= 3*I*H*elem) */
  const int32_t* expert_slot_dev;  /* [E] expert id -> slot (device segment lists only) */
  int32_t num_experts;             /* E */
  int32_t hidden;                  /* H */
  int32_t inter;                   /* I */
  int32_t dtype;                   /* SPARSE_HIP_F32 | SPARSE_HIP_BF16 | SPARSE_HIP_F16 */
} sparse_hip_experts;

/*
 * Which expert segments one launch executes, in launch order.  If `eids_dev` is
 * non-NULL the list is read on the device: `eids_dev[0 .. *count_dev)` with at most
 * `n` entries (the grid is sized for n), and the weights of expert e are in slot
 * `expert_slot_dev[e]`.  Otherwise the first `n` entries of `eids` are used and the
 * weights of `eids[i]` are in slot `slots[i]`: the host decides order and residency
 * per launch and nothing on the device has to be rewritten between launches.  A
 * segment is the run of permuted rows of one expert (utils/eval_core.py:13240-13262).
 */
typedef struct sparse_hip_seglist {
  const int32_t* eids_dev;
  const int32_t* count_dev;
  int32_t n;
  int16_t eids[SPARSE_HIP_MAX_EXPERTS];
  int16_t slots[SPARSE_HIP_MAX_EXPERTS];
} sparse_hip_seglist;

/* ---- A1: router ------------------------------------------------------------ */

/*
 * logits[t,e] = sum_h x[t,h] * wg[e,h], accumulated in fp32 and rounded once to
 * `logits_dtype` -- `router_logits = self.gate(x)` (utils/eval_core.py:9519) when
 * logits_dtype == dtype; the DeepSeek gate's fp32 logits when logits_dtype is F32.
 * If `wsg_dev` is non-NULL also writes shared_gate_dev[t] = sum_h x[t,h]*wsg[h] in
 * `dtype` -- `self.shared_expert_gate(x)` (utils/eval_core.py:9461).
 * x [T,H], wg [E,H], wsg [H] in `dtype`.  H % 8 == 0.
 */
int sparse_hip_router_logits(const void* x_dev, const void* wg_dev, const void* wsg_dev,
                             int dtype, int logits_dtype, int T, int H, int E,
                             void* logits_dev, void* shared_gate_dev, void* stream);

/*
 * probs = softmax(logits, fp32); (topv, topi) = top-K of probs, descending, ties to
 * the lower expert id; optional renormalisation topv /= max(sum topv, 1e-12); topv is
 * rounded to `out_dtype`, topi is int64 -- utils/eval_core.py:9520, :9590-9595.
 * The ranking is done on the logits (descending, then lower id), which is the order of the
 * probabilities wherever two of them differ and does not depend on the rounding of exp: the
 * indices are a function of the logits alone.
 * logits [T,E] in `logits_dtype`; topv [T,K]; topi [T,K].  E <= 256, K <= 16, K <= E.
 */
int sparse_hip_gate_topk(const void* logits_dev, int logits_dtype, int T, int E, int K,
                         int renorm, int out_dtype, void* topv_dev, int64_t* topi_dev,
                         void* stream);

/*
 * The same with DeepSeek-V2's group-limited selection in front of the top-k: the experts form
 * `n_group` equal runs of ids, a group scores its largest probability, the `topk_group` best
 * groups stay (ties to the lower group id) and every other expert's probability is replaced
 * by 0 before the top-k.  This is the `group_limited_greedy` method of the gate the reference
 * delegates to (`self.gate(...)`, utils/eval_core.py:9503-9517; the gate module itself is the
 * model's, e.g. transformers' DeepseekV2TopkRouter).  n_group <= 64, E % n_group == 0;
 * n_group == 1 or topk_group == n_group is plain top-k.
 */
int sparse_hip_gate_topk_grouped(const void* logits_dev, int logits_dtype, int T, int E, int K,
                                 int renorm, int n_group, int topk_group, int out_dtype,
                                 void* topv_dev, int64_t* topi_dev, void* stream);

/*
 * The same with the two things the DeepSeek branch of `_routing_router` does after the gate
 * (utils/eval_core.py:9503-9517, :9490-9499) in the same launch: the weights are multiplied by the
 * gate's routed scaling factor `scale` in fp32 before their one rounding to `out_dtype` (as the gate
 * module multiplies before the reference casts), and, where `pseudo_logits_dev` [T,E] fp32 is not
 * NULL, it receives -inf everywhere but at the selected experts, which hold
 * log(max(weight as rounded, 1e-12)).  scale == 1 and NULL give sparse_hip_gate_topk_grouped.
 */
int sparse_hip_gate_topk_scaled(const void* logits_dev, int logits_dtype, int T, int E, int K,
                                int renorm, int n_group, int topk_group, float scale, int out_dtype,
                                void* topv_dev, int64_t* topi_dev, float* pseudo_logits_dev, void* stream);

/*
 * Pseudo logits of a routing that is given rather than computed: out [T,E] fp32 = `fill` everywhere
 * but at topi[t, k], which holds log(max(topv[t, k], eps)) -- what `_routing_for_execute` returns when
 * a layer executes its predecessor's prediction (utils/eval_core.py:11137-11155, fill -1e9, eps from the
 * block's rs_prob_to_logit_eps) and what :9490-9499 builds (fill -inf, eps 1e-12).  topv in `dtype`.
 */
int sparse_hip_pseudo_logits(const void* topv_dev, int dtype, const int64_t* topi_dev, int T, int K, int E,
                             float eps, float fill, float* out_dev, void* stream);

/*
 * Top-K of each row of given probabilities, no softmax: values descending, ties to the lower
 * index; optional renormalisation as above; topv rounded to `out_dtype`.  This is the
 * `torch.topk` the reference applies to the next-layer predictor's output before planning
 * prefetches and before replaying a predicted routing (utils/eval_core.py:10985-10996,
 * :10971-10983), with the tie order torch leaves open fixed.  values [T,E] fp32; E <= 256,
 * K <= 16, K <= E.
 */
int sparse_hip_topk(const void* values_dev, int T, int E, int K, int renorm, int out_dtype,
                    void* topv_dev, int64_t* topi_dev, void* stream);

/* ---- A5: token x K expansion + permutation --------------------------------- */

/*
 * Stable bucketing of the flat routed items f = t*K + k by expert id:
 *   perm[p] = f of the p-th item in (expert id, f) order,  inv_perm[f] = p,
 *   seg_offsets[e] .. seg_offsets[e+1] = rows of expert e (exclusive prefix sum of
 *   the per-expert counts), active_eids[0 .. *n_active) = ids with >= 1 item,
 *   ascending.
 * Stands in for `argsort(flat_i)` + segment scan + `out[order] = out_sorted`
 * (utils/eval_core.py:14728-14730, :13240-13262, :13359-13360) without host syncs.
 * topi [T,K] int64 with 0 <= id < E.  Outputs int32: perm [T*K], inv_perm [T*K],
 * seg_offsets [E+1], active_eids [E], n_active [1].  `ws_dev` is a workspace of
 * sparse_hip_permute_ws_bytes(T, K, E) bytes.
 */
size_t sparse_hip_permute_ws_bytes(int T, int K, int E);
int sparse_hip_permute_build(const int64_t* topi_dev, int T, int K, int E, int32_t* perm_dev,
                             int32_t* inv_perm_dev, int32_t* seg_offsets_dev,
                             int32_t* active_eids_dev, int32_t* n_active_dev, void* ws_dev,
                             void* stream);

/*
 * sparse_hip_permute_build for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): same inputs, same
 * outputs, no workspace argument.  It has no counterpart in the reference.  The per-block
 * histograms live in a 256 KB array built into the library (one copy per GPU, held until
 * the process ends), which bounds T at SPARSE_HIP_PERMUTE_STATIC_MAX_TOKENS; a larger T is
 * rejected with SPARSE_HIP_EINVAL.  The call allocates nothing; the first call on a device
 * looks up the array's address (make that call outside a graph capture).  All calls on one
 * GPU share the array: calls that overlap there, on different streams or from different
 * threads, race.  Nothing has to be cleared between calls -- every entry that is read was
 * written by the same call.
 */
int sparse_hip_permute_build_static(const int64_t* topi_dev, int T, int K, int E, int32_t* perm_dev,
                                    int32_t* inv_perm_dev, int32_t* seg_offsets_dev,
                                    int32_t* active_eids_dev, int32_t* n_active_dev, void* stream);

/*
 * Decode fast path: sparse_hip_router_logits + sparse_hip_gate_topk +
 * sparse_hip_permute_build in ONE launch for T <= SPARSE_HIP_DECODE_MAX_TOKENS (topv is
 * written in `dtype`).  Each workgroup computes one token's logits and its top-k; the
 * workgroup that finishes last (counted in `counter_dev` behind a device-scope fence)
 * builds the permutation.  `counter_dev` is one int32 that must be zero before the
 * first call; every call leaves it zero.  The logits may differ from
 * sparse_hip_router_logits' in the last fp32 bit before rounding (another summation
 * order); top-k and permutation are, bit for bit, what sparse_hip_gate_topk and
 * sparse_hip_permute_build return for the logits written here
 * (utils/eval_core.py:9519-9595, :14728-14730, :13240-13262).
 */
int sparse_hip_route_decode(const void* x_dev, const void* wg_dev, const void* wsg_dev, int dtype,
                            int logits_dtype, int T, int H, int E, int K, int renorm, void* logits_dev,
                            void* shared_gate_dev, void* topv_dev, int64_t* topi_dev, int32_t* perm_dev,
                            int32_t* inv_perm_dev, int32_t* seg_offsets_dev, int32_t* active_eids_dev,
                            int32_t* n_active_dev, int32_t* counter_dev, void* stream);

/*
 * The same routing step (utils/eval_core.py:9519-9520, :9590-9595, and the stable bucketing
 * of :13224-13243) for 16-bit activations (`dtype`: bf16 or fp16; `logits_dtype`: the same, or
 * fp32) and at most SPARSE_HIP_ROUTE_PACKED_MAX_TOKENS tokens,
 * on a gate matrix packed ahead of time so that one workgroup streams it with contiguous
 * wave loads and finishes logits, top-k and permutation without waiting for another
 * workgroup: `gate_packed_dev` is a [SPARSE_HIP_ROUTE_PACKED_ROWS, H] matrix of that dtype in the tiled
 * layout (`sparse_hip_tile_weight` of the row-major matrix whose rows are the E gate rows,
 * then the shared-expert gate vector if `has_shared_gate`, then zero rows); H % 64 == 0 and
 * E + has_shared_gate <= SPARSE_HIP_ROUTE_PACKED_ROWS.  Outputs are those of
 * `sparse_hip_route_decode`; the logits differ from it only in the order of the fp32 sum.
 */
int sparse_hip_route_decode_packed(const void* x_dev, const void* gate_packed_dev, int has_shared_gate, int dtype,
                                   int logits_dtype, int T, int H, int E, int K, int renorm, void* logits_dev,
                                   void* shared_gate_dev, void* topv_dev, int64_t* topi_dev, int32_t* perm_dev,
                                   int32_t* inv_perm_dev, int32_t* seg_offsets_dev, int32_t* active_eids_dev,
                                   int32_t* n_active_dev, void* stream);
/* The same routing, and in the same launch the shared expert's gate and up projections with
 * SiLU*up (which need the token rows only): shared_inter_dev [T, Is] = SiLU(x Wg^T) * (x Wu^T),
 * rounded like the expert kernels round it.  Routing is one workgroup's work; the rest of the
 * device reads the two matrices meanwhile instead of idling.  shared_gate_w_dev / shared_up_w_dev
 * are [Is, H] in the tiled layout (sparse_hip_tile_weight), Is a multiple of 32.  The expert
 * kernels are then called without these two matrices (NULL) and take shared_inter_dev as it is.
 * Routing results are those of sparse_hip_route_decode_packed bit for bit.  No counterpart in
 * the reference, whose block computes router and shared expert one after the other
 * (utils/eval_core.py:16488, :16522-16525).
 * sparse_hip_shared_gate_up is the shared expert's half alone (same kernel code, same bits),
 * for a call that routes some other way; T <= SPARSE_HIP_ROUTE_PACKED_MAX_TOKENS, H % 64 == 0. */
int sparse_hip_shared_gate_up(const void* x_dev, const void* shared_gate_w_dev, const void* shared_up_w_dev, int dtype,
                              int T, int H, int Is, void* shared_inter_dev, void* stream);
int sparse_hip_route_decode_packed_shared(const void* x_dev, const void* gate_packed_dev, int has_shared_gate,
                                          int dtype, int logits_dtype, int T, int H, int E, int K, int renorm,
                                          void* logits_dev, void* shared_gate_dev, void* topv_dev,
                                          int64_t* topi_dev, int32_t* perm_dev, int32_t* inv_perm_dev,
                                          int32_t* seg_offsets_dev, int32_t* active_eids_dev, int32_t* n_active_dev,
                                          const void* shared_gate_w_dev, const void* shared_up_w_dev, int Is,
                                          void* shared_inter_dev, void* stream);

/* ---- A4/A6: grouped SwiGLU expert FFN -------------------------------------- */

/*
 * For every segment in `segs` (expert e, rows p in [seg_offsets[e], seg_offsets[e+1])):
 *   cur   = x[perm[p] / K]
 *   inter = act(gate_e(cur)) * up_e(cur)         (each Linear rounded to dtype, the
 *                                                 activation and the product too)
 *   parts[p] = down_e(inter) * topv_flat[perm[p]]  (rounded to dtype twice)
 * i.e. `_plain_ep_compute_segment` / `_module_expert_forward`
 * (utils/eval_core.py:11700-11793) over segments, writing rows in permuted order.
 * Rows of segments that are not in `segs` are left untouched.
 *
 * `_decode` is the HBM-bandwidth path: T <= SPARSE_HIP_DECODE_MAX_TOKENS, weights are
 * streamed once.  `_prefill` is the MFMA grouped-GEMM path for any T (bf16), and the
 * tiled FMA path for fp32.  Both produce the same rows up to fp32 summation order.
 * x [T,H]; topv [T,K] in dtype; inter_ws [T*K, I] and parts [T*K, H] in dtype.
 * H % 64 == 0 and I % 64 == 0.  `_prefill` also takes `tile_ws_dev`, a workspace of
 * sparse_hip_prefill_ws_bytes(T, K, segs->n, H, I) bytes in which a one-workgroup kernel
 * lays out which tile every workgroup owns (segment lengths are only known on the device).
 */
size_t sparse_hip_prefill_ws_bytes(int T, int K, int num_segments, int H, int I);
int sparse_hip_grouped_swiglu_decode(const sparse_hip_experts* experts, const void* x_dev,
                                     const void* topv_dev, const int32_t* perm_dev,
                                     const int32_t* seg_offsets_dev,
                                     const sparse_hip_seglist* segs, int T, int K,
                                     void* inter_ws_dev, void* parts_dev, void* stream);
int sparse_hip_grouped_swiglu_prefill(const sparse_hip_experts* experts, const void* x_dev,
                                      const void* topv_dev, const int32_t* perm_dev,
                                      const int32_t* seg_offsets_dev,
                                      const sparse_hip_seglist* segs, int T, int K,
                                      void* inter_ws_dev, void* parts_dev, void* tile_ws_dev,
                                      void* stream);

/* ---- A8: shared expert ----------------------------------------------------- */

/*
 * shared[t] = down_s(act(gate_s(x[t])) * up_s(x[t])), times
 * sigmoid(shared_gate[t]) when `shared_gate_dev` is non-NULL (each step rounded to
 * dtype) -- `_shared_expert_forward` (utils/eval_core.py:9455-9463).
 * gate_s, up_s [Is,H], down_s [H,Is] (tiled); inter_ws [T,Is]; shared [T,H].
 * Uses the decode kernels when T <= SPARSE_HIP_DECODE_MAX_TOKENS, the prefill
 * kernels otherwise.  For a bf16 call of at most SPARSE_HIP_DECODE_MAX_TOKENS tokens gate_w_dev
 * and up_w_dev may both be NULL: inter_ws then already holds act(gate_s x) * up_s x
 * (sparse_hip_shared_gate_up) and only the down projection runs.
 */
int sparse_hip_shared_expert(const void* x_dev, const void* gate_w_dev, const void* up_w_dev,
                             const void* down_w_dev, const void* shared_gate_dev, int dtype,
                             int T, int H, int Is, void* inter_ws_dev, void* shared_dev,
                             void* stream);

/*
 * Prefill fast path: sparse_hip_grouped_swiglu_prefill and sparse_hip_shared_expert of one call
 * as two launches of persistent workgroups (every gate/up projection, then every down projection),
 * bf16 or fp16, any T.  Tiles of the routed segments and of the shared expert sit in one set of
 * queues (one per XCD, built on the device in `tile_ws_dev`); a workgroup takes tile after tile and
 * requests the first operands of its next tile while it finishes the current one, so routed and
 * shared work share one tail per launch and no tile but a workgroup's first pays a prologue.
 * Results are bit-identical to the two separate calls.  Arguments as in those two functions
 * (utils/eval_core.py:11700-11793 for the routed experts, :9455-9463 and :16520-16526 for the shared
 * expert).  `sh_down_w_dev` NULL: no shared expert (the other sh_* arguments are ignored);
 * segs->n == 0: the shared expert alone.  `tile_ws_dev`: 256-byte aligned workspace of
 * sparse_hip_moe_ffn_prefill_ws_bytes(T, K, segs->n, H, I, Is) bytes (Is = 0 without a shared
 * expert).  Calls that share a workspace must be ordered on one stream.
 */
size_t sparse_hip_moe_ffn_prefill_ws_bytes(int T, int K, int num_segments, int H, int I, int Is);
int sparse_hip_moe_ffn_prefill(const sparse_hip_experts* experts, const void* x_dev, const void* topv_dev,
                               const int32_t* perm_dev, const int32_t* seg_offsets_dev,
                               const sparse_hip_seglist* segs, int T, int K, void* inter_ws_dev,
                               void* parts_dev, const void* sh_gate_w_dev, const void* sh_up_w_dev,
                               const void* sh_down_w_dev, const void* shared_gate_dev, int Is,
                               void* sh_inter_ws_dev, void* shared_dev, void* tile_ws_dev, void* stream);

/*
 * Decode fast path: sparse_hip_grouped_swiglu_decode and sparse_hip_shared_expert of one
 * call in a single launch pair (gate/up of every routed segment and of the shared
 * expert, then all down projections), so the chip sees one fat stream of weights
 * instead of four thinner launches.  bf16 or fp16 (the slab's dtype), T <= SPARSE_HIP_DECODE_MAX_TOKENS.
 * Arguments as in those two functions; `sh_*` are the shared expert's
 * (utils/eval_core.py:16520-16526).
 * `split_ws_dev` is NULL or a workspace of sparse_hip_decode_split_ws_bytes(T, H) bytes.  With
 * NULL the results are identical to the two separate calls.  With a workspace, and when
 * sparse_hip_decode_split_parts(Is) > 1, the shared expert's down projection, whose reduction
 * is Is long against the routed experts' I, is cut into that many workgroups per tile so that
 * it no longer trails the launch: `shared_dev` is then NOT written, the workspace receives the
 * fp32 partial sums [parts][T][H], and sparse_hip_combine_split finishes them (adds them in
 * their order, rounds, applies the shared gate) while it combines -- the same rounding steps
 * as the one-workgroup form, with the fp32 sum grouped differently.
 * `sh_gate_w_dev` and `sh_up_w_dev` may both be NULL: `sh_inter_ws_dev` then already holds the
 * shared expert's SiLU(gate x) * (up x) (sparse_hip_route_decode_packed_shared computes it beside
 * the routing) and only the routed experts' gate/up projections run here.
 */
size_t sparse_hip_decode_split_ws_bytes(int T, int H);
int sparse_hip_decode_split_parts(int Is);
int sparse_hip_moe_ffn_decode(const sparse_hip_experts* experts, const void* x_dev, const void* topv_dev,
                              const int32_t* perm_dev, const int32_t* seg_offsets_dev,
                              const sparse_hip_seglist* segs, int T, int K, void* inter_ws_dev,
                              void* parts_dev, const void* sh_gate_w_dev, const void* sh_up_w_dev,
                              const void* sh_down_w_dev, const void* shared_gate_dev, int Is,
                              void* sh_inter_ws_dev, void* shared_dev, void* split_ws_dev,
                              void* stream);

/*
 * sparse_hip_moe_ffn_decode followed by sparse_hip_combine_split, without the second launch:
 * in the down projection, the workgroup that finishes a 32-column tile last (counted per
 * tile) sums that tile's columns of every token -- the K routed rows in ascending expert id,
 * then the shared expert from its partial sums, with the rounding steps of
 * sparse_hip_combine_split, bit for bit -- and writes `out_dev` [T,H]
 * (utils/eval_core.py:16520-16526, :14690-14721, :523-538, :9455-9463).  Needs
 * sparse_hip_decode_split_parts(Is) > 1.  `split_ws_dev` holds
 * sparse_hip_decode_split_ws_bytes(T, H) bytes: the partial sums, then, from
 * sparse_hip_decode_split_counter_offset(T, H) on, one int32 counter per tile.  The call's first
 * launch puts the counters to zero, so the workspace may hold anything before (an earlier call with
 * another T, a call that did not finish); a finished call leaves them at zero.  Calls that share a
 * workspace must not overlap.  `parts_dev` is written as by sparse_hip_moe_ffn_decode.
 */
size_t sparse_hip_decode_split_counter_offset(int T, int H);
int sparse_hip_moe_ffn_decode_combine(const sparse_hip_experts* experts, const void* x_dev, const void* topv_dev,
                                      const int32_t* perm_dev, const int32_t* inv_perm_dev,
                                      const int32_t* seg_offsets_dev, const sparse_hip_seglist* segs, int T,
                                      int K, void* inter_ws_dev, void* parts_dev, const void* sh_gate_w_dev,
                                      const void* sh_up_w_dev, const void* sh_down_w_dev,
                                      const void* shared_gate_dev, int Is, void* sh_inter_ws_dev,
                                      void* split_ws_dev, void* out_dev, void* stream);

/* ---- A7: combine ----------------------------------------------------------- */

/*
 * out[t] = (((0 + parts[p_0]) + parts[p_1]) + ...) (+ shared[t]) with p_j the rows of
 * token t in ascending expert id and every add rounded to dtype: the accumulation
 * order of `final.index_add_` in `_experts_world1_exact` (utils/eval_core.py:14720)
 * and of `combine_expert_outputs` (utils/eval_core.py:523-538), followed by
 * `expert_out + shared_out` (utils/eval_core.py:16526).  `shared_dev` may be NULL.
 * parts [T*K,H], inv_perm [T*K], out [T,H].  H % 8 == 0.
 */
int sparse_hip_combine(const void* parts_dev, const int32_t* inv_perm_dev,
                       const void* shared_dev, int dtype, int T, int K, int H, void* out_dev,
                       void* stream);

/*
 * The same for a decode call whose shared expert was left as partial sums by
 * sparse_hip_moe_ffn_decode(split_ws_dev): shared[t] = r(r(sum of the `nparts` fp32
 * parts) * r(sigmoid(shared_gate[t]))) with r = rounding to `dtype` (no factor when
 * `shared_gate_dev` is NULL) -- the tail of `_shared_expert_forward`
 * (utils/eval_core.py:9455-9463) -- added after the routed parts as above.  bf16 or fp16.
 */
int sparse_hip_combine_split(const void* parts_dev, const int32_t* inv_perm_dev, const void* split_ws_dev,
                             int nparts, const void* shared_gate_dev, int dtype, int T, int K, int H,
                             void* out_dev, void* stream);

/* ---- A12: routing-scout predictor ------------------------------------------ */

/*
 * pred[T, E] = softmax(w2 relu(w1 float(x) + b1) + b2): the forward pass of the reference's
 * `RoutingScoutMLP` in eval mode (utils/eval_core.py:3402-3417: Linear, BatchNorm1d, ReLU, Dropout,
 * Linear, Softmax) as `_compute_and_schedule_next_layer_rs` runs it on the layer's input
 * (:10916-10960, `rs_in = x.float()`), for any number of token rows (a workgroup takes
 * SPARSE_HIP_DECODE_MAX_TOKENS of them).
 * All parameters are fp32 and row-major; the caller folds the BatchNorm's running statistics and affine
 * into w1 [D, H] and b1 [D] once, at load time (eval mode makes it a per-row scale and shift; Dropout is
 * the identity).  x is [T, H] in `dtype`; hidden_ws_dev holds T * D floats; w2 is [E, D].  Two launches.
 */
int sparse_hip_rs_predict(const void* x_dev, int dtype, int T, int H, const float* w1_dev, const float* b1_dev,
                          int D, const float* w2_dev, const float* b2_dev, int E, float* hidden_ws_dev,
                          float* pred_dev, void* stream);

/*
 * The pieces of the deeper predictor, `RoutingScoutResidualMLP` in eval mode
 * (utils/eval_core.py:3419-3461: LayerNorm, Linear, GELU; units of x + Linear(GELU(Linear(LayerNorm(x))));
 * LayerNorm, Linear, softmax) and of predictors that also read the layer's routing (:10903-10914), which
 * the host strings together; fp32 arithmetic and fp32 row-major parameters throughout.
 *
 * sparse_hip_rs_dense:     out[T, D] = act(x[T, H] w[D, H]^T + b[D]) (+ residual[T, D] when not NULL), with
 *                          act 0 = none, 1 = ReLU, 2 = GELU in its exact (erf) form; x in `dtype`, H a
 *                          multiple of 8 (pad rows and weight columns with zeros otherwise).
 * sparse_hip_rs_layernorm: out[t, :H] = (x[t, :H] - mean) / sqrt(var + eps) * gamma + beta with the biased
 *                          variance, as nn.LayerNorm; rows of x are ld_in elements apart, rows of out
 *                          ld_out, and out[t, H:ld_out] is set to zero.
 * sparse_hip_rs_features:  out[t, :] = [ float(x[t, :H]) | feat[t, :E] | zeros up to ld ], where feat holds
 *                          the token's K routing weights divided by max(their sum, 1e-12) at its K expert
 *                          ids (`idx`/`w` of :10903-10908; ids outside [0, E) are skipped).
 * sparse_hip_rs_softmax:   out[t, :] = softmax(in[t, :E]).
 */
int sparse_hip_rs_dense(const void* x_dev, int dtype, int T, int H, const float* w_dev, const float* b_dev, int D,
                        int act, const float* residual_dev, float* out_dev, void* stream);
int sparse_hip_rs_layernorm(const void* x_dev, int dtype, int T, int H, int ld_in, int ld_out,
                            const float* gamma_dev, const float* beta_dev, float eps, float* out_dev, void* stream);
int sparse_hip_rs_features(const void* x_dev, int dtype, int T, int H, const int64_t* topi_dev,
                           const void* topv_dev, int K, int E, int ld, float* out_dev, void* stream);
int sparse_hip_rs_softmax(const float* in_dev, int T, int E, float* out_dev, void* stream);

/* ---- A11/A12/A13: expert residency ----------------------------------------- */

/*
 * Enqueue a pinned-host -> HBM copy of one expert (`bytes` from `src_host` to
 * `dst_dev`) on `stream`, then record `event` (a hipEvent_t as void*, may be NULL) on
 * it.  Stands in for the three `pinned_cpu.to(device, non_blocking=True)` copies and
 * `_record_prefetch_event` (utils/eval_core.py:11427-11429, :9970-9984, :11234-11242,
 * :11621-11634).  Safe to call from a second host thread.
 */
int sparse_hip_expert_upload_async(void* dst_dev, const void* src_host, size_t bytes,
                                   void* stream, void* event);

/* Events and streams used to gate readiness (utils/eval_core.py:11176-11210,
 * :5028-5055).  Events are created without timing unless `timing` is non-zero. */
int sparse_hip_event_create(int timing, void** event_out);
int sparse_hip_event_destroy(void* event);
int sparse_hip_event_record(void* event, void* stream);
/* 0 = complete, SPARSE_HIP_ENOTREADY = still in flight. */
int sparse_hip_event_query(void* event);
/* Make `stream` wait for `event` without blocking the host. */
int sparse_hip_stream_wait_event(void* stream, void* event);
int sparse_hip_event_elapsed_ms(void* start, void* stop, float* ms_out);
/* Streams are created at the default priority. */
int sparse_hip_stream_create(void** stream_out);
int sparse_hip_stream_destroy(void* stream);
int sparse_hip_stream_synchronize(void* stream);
/* Pinned host arena for offloaded experts (hipHostMalloc / hipHostFree). */
int sparse_hip_host_alloc(size_t bytes, void** ptr_out);
int sparse_hip_host_free(void* ptr);

/* ---- weight layout ---------------------------------------------------------- */

/*
 * Convert one [rows, cols] matrix between row-major and the tiled layout described at the
 * top of this file (to_tiled != 0: row-major -> tiled).  src and dst must not alias.
 * The reference keeps weights row-major (utils/eval_core.py:5115-5123); packing is a
 * load-time step of this library's host.
 */
int sparse_hip_tile_weight(const void* src_dev, void* dst_dev, int rows, int cols, int dtype, int to_tiled,
                           void* stream);

/* Plain device copy of `bytes` (multiple of 16) by a grid-stride kernel: the known-size
 * reference point for scaling HBM traffic counters.  No counterpart in the reference. */
int sparse_hip_calib_copy(const void* src_dev, void* dst_dev, size_t bytes, void* stream);

/* ---- measurement ---------------------------------------------------------- */

/*
 * Per-kernel timing with HIP events on the stream each kernel is launched on (no
 * counterpart in the reference, which times whole segments with cuda.Event pairs,
 * utils/eval_core.py:14655-14688).  While enabled, every kernel launch made through
 * this library is bracketed by an event pair; `profile_read` waits for the recorded
 * pairs of one kernel and returns their summed duration and count.  Leave it off in
 * timed runs and under graph capture: the event records add launch gaps.
 */
#define SPARSE_HIP_K_ROUTER_LOGITS 0
#define SPARSE_HIP_K_GATE_TOPK 1
#define SPARSE_HIP_K_PERMUTE 2
#define SPARSE_HIP_K_DECODE_GATEUP 3
#define SPARSE_HIP_K_DECODE_DOWN 4
#define SPARSE_HIP_K_PREFILL_GATEUP 5
#define SPARSE_HIP_K_PREFILL_DOWN 6
#define SPARSE_HIP_K_TILED_GATEUP 7
#define SPARSE_HIP_K_TILED_DOWN 8
#define SPARSE_HIP_K_COMBINE 9
#define SPARSE_HIP_K_ROUTE_DECODE 10
#define SPARSE_HIP_K_COUNT 11
int sparse_hip_profile_enable(int on);
int sparse_hip_profile_reset(void);
int sparse_hip_profile_read(int kernel, double* total_ms_out, int64_t* launches_out);
/* Checking aid with no counterpart in the reference: while on, the prefill-size expert FFN
 * (sparse_hip_grouped_swiglu_prefill, sparse_hip_moe_ffn_prefill, sparse_hip_shared_expert at prefill sizes) runs the variant of its
 * kernel whose k loop drains every outstanding vector-memory operation where the normal one
 * waits for a counted number of them.  Same arithmetic, same bits, slower; a difference
 * between the two means the counted waits no longer match the code the compiler produced.
 * Process-wide; returns the previous setting. */
int sparse_hip_prefill_drain_waits(int on);
/* Measurement aid with no counterpart in the reference: the clock the matrix cores really run
 * at while the prefill-size expert FFN executes.  While `counters_dev` (two uint64 in device
 * memory, zeroed by the caller) is set, every workgroup of that kernel adds the shader-clock
 * cycles between its first and its last instruction to counters_dev[0] and the ticks of the
 * constant 100 MHz clock over the same interval to counters_dev[1]; 100 MHz x [0] / [1] is
 * the average shader clock of a busy compute unit, which under a power cap is well below the
 * peak clock the published MFMA rate assumes.  NULL turns it off.  Process-wide. */
int sparse_hip_prefill_clock_probe(void* counters_dev);
/* Measurement aid with no counterpart in the reference: what the matrix cores sustain on this part
 * for the prefill kernel's wavefront tile with nothing else going on.  Launches, twice (the first
 * untimed), one workgroup of eight wavefronts per compute unit, every wavefront multiplying a
 * 128 x 64 tile as eight by four bf16 16x16x32 MFMA tiles, `iters` (even) k steps of 32 on
 * pseudo-random operands held in registers (from_lds == 0) or with the eight activation fragments
 * of every k step read from LDS, as the prefill kernel's inner loop reads them (from_lds != 0).
 * `counters_dev`: 32 bytes of device memory, 8-byte aligned, which the call clears and uses.
 * Returns the rate of the timed launch (HIP events on `stream`) in TFLOP/s and the average shader
 * clock of the busy compute units in MHz.  Waits for the launch; not for use under graph capture. */
int sparse_hip_mfma_probe(int from_lds, int iters, void* counters_dev, double* tflops_out, double* clock_mhz_out,
                          void* stream);
/* Name of the __global__ function behind a kernel id (as rocprofv3 prints it, with the template
 * arguments that tell the kernels of one family apart: F stands for the 16-bit format, sparse::Bf16 or
 * sparse::Fp16; the tile-count arguments that follow are left out). */
const char* sparse_hip_kernel_name(int kernel);

#ifdef __cplusplus
}
#endif
#endif /* SPARSE_HIP_H */
