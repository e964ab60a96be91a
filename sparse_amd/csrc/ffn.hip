// C ABI entry points of the grouped SwiGLU FFN and the shared expert: argument
// checks, then dispatch to the decode (HBM-bound, bf16 MFMA 16x16x32), prefill
// (bf16 MFMA grouped GEMM) or fp32 tiled kernels.
#include "common.h"

namespace sparse {

int decode_routed_bf16(const sparse_hip_experts*, const void*, const void*, const int32_t*, const int32_t*,
                       const sparse_hip_seglist*, int, int, void*, void*, hipStream_t);
int decode_shared_bf16(const void*, const void*, const void*, const void*, const void*, int, int, int, int, void*,
                       void*, hipStream_t);
int decode_fused_bf16(const sparse_hip_experts*, const void*, const void*, const int32_t*, const int32_t*,
                      const sparse_hip_seglist*, int, int, void*, void*, const void*, const void*, const void*,
                      const void*, int, void*, void*, void*, const int32_t*, void*, hipStream_t);
size_t decode_split_ws_bytes(int, int);
size_t decode_split_counter_offset(int, int);
int decode_split_parts(int);
int prefill_routed_bf16(const sparse_hip_experts*, const void*, const void*, const int32_t*, const int32_t*,
                        const sparse_hip_seglist*, int, int, void*, void*, void*, hipStream_t);
size_t prefill_ws_bytes(int, int, int, int, int);
size_t prefill_merged_ws_bytes(int, int, int, int, int, int);
int prefill_merged(const sparse_hip_experts*, const void*, const void*, const int32_t*, const int32_t*,
                   const sparse_hip_seglist*, int, int, void*, void*, const void*, const void*, const void*,
                   const void*, int, void*, void*, void*, hipStream_t);
int prefill_set_drain_waits(int);
void prefill_set_clock_probe(void*);
int prefill_shared_bf16(const void*, const void*, const void*, const void*, const void*, int, int, int, int, void*,
                        void*, hipStream_t);
template <typename T>
int tiled_routed(const sparse_hip_experts*, const void*, const void*, const int32_t*, const int32_t*,
                 const sparse_hip_seglist*, int, int, void*, void*, hipStream_t);
template <typename T>
int tiled_shared(const void*, const void*, const void*, const void*, const void*, int, int, int, void*, void*,
                 hipStream_t);

static int check_routed(const char* fn, const sparse_hip_experts* ex, const void* x, const void* topv,
                        const int32_t* perm, const int32_t* seg_offsets, const sparse_hip_seglist* segs, int T,
                        int K, void* inter_ws, void* parts) {
  SP_REQUIRE(ex != nullptr && segs != nullptr, "%s: NULL descriptor", fn);
  SP_REQUIRE(valid_dtype(ex->dtype), "%s: unknown dtype %d", fn, ex->dtype);
  SP_REQUIRE(ex->num_experts >= 1 && ex->num_experts <= SPARSE_HIP_MAX_EXPERTS, "%s: E=%d outside [1,%d]", fn,
             ex->num_experts, SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(ex->hidden > 0 && ex->hidden % 64 == 0, "%s: H=%d must be a positive multiple of 64", fn,
             ex->hidden);
  SP_REQUIRE(ex->inter > 0 && ex->inter % 64 == 0, "%s: I=%d must be a positive multiple of 64", fn, ex->inter);
  SP_REQUIRE(ex->slot_stride >= 3ull * ex->hidden * ex->inter * elem_size(ex->dtype) &&
                 ex->slot_stride % 16 == 0,
             "%s: slot_stride=%llu too small or not 16-byte aligned", fn,
             static_cast<unsigned long long>(ex->slot_stride));
  SP_REQUIRE(ex->slab_dev != nullptr, "%s: NULL weight slab", fn);
  SP_REQUIRE((reinterpret_cast<uintptr_t>(ex->slab_dev) & 15) == 0, "%s: slab not 16-byte aligned", fn);
  SP_REQUIRE(T >= 1, "%s: T=%d must be >= 1", fn, T);
  SP_REQUIRE(K >= 1 && K <= SPARSE_HIP_MAX_TOPK, "%s: K=%d outside [1,%d]", fn, K, SPARSE_HIP_MAX_TOPK);
  SP_REQUIRE(x && topv && perm && seg_offsets && inter_ws && parts, "%s: NULL pointer", fn);
  SP_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(inter_ws) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(parts) & 15) == 0,
             "%s: activations must be 16-byte aligned", fn);
  SP_REQUIRE(segs->n >= 0 && segs->n <= SPARSE_HIP_MAX_EXPERTS, "%s: segment count %d outside [0,%d]", fn,
             segs->n, SPARSE_HIP_MAX_EXPERTS);
  SP_REQUIRE(segs->eids_dev == nullptr || segs->count_dev != nullptr, "%s: device segment list without count",
             fn);
  if (segs->eids_dev == nullptr) {
    for (int i = 0; i < segs->n; ++i) {
      SP_REQUIRE(segs->eids[i] >= 0 && segs->eids[i] < ex->num_experts, "%s: segment %d names expert %d", fn, i,
                 static_cast<int>(segs->eids[i]));
      SP_REQUIRE(segs->slots[i] >= 0, "%s: segment %d has slot %d", fn, i, static_cast<int>(segs->slots[i]));
    }
  } else {
    SP_REQUIRE(ex->expert_slot_dev != nullptr, "%s: device segment list needs expert_slot_dev", fn);
  }
  return SPARSE_HIP_OK;
}

}  // namespace sparse

using namespace sparse;

extern "C" {

int sparse_hip_prefill_drain_waits(int on) { return prefill_set_drain_waits(on); }

int sparse_hip_prefill_clock_probe(void* counters_dev) {
  prefill_set_clock_probe(counters_dev);
  return SPARSE_HIP_OK;
}

size_t sparse_hip_prefill_ws_bytes(int T, int K, int num_segments, int H, int I) {
  if (T <= 0 || K <= 0 || num_segments < 0 || H <= 0 || I <= 0) return 0;
  return prefill_ws_bytes(T, K, num_segments, H, I);
}

int sparse_hip_grouped_swiglu_decode(const sparse_hip_experts* experts, const void* x_dev, const void* topv_dev,
                                     const int32_t* perm_dev, const int32_t* seg_offsets_dev,
                                     const sparse_hip_seglist* segs, int T, int K, void* inter_ws_dev,
                                     void* parts_dev, void* stream) {
  int rc = check_routed("grouped_swiglu_decode", experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K,
                        inter_ws_dev, parts_dev);
  if (rc != SPARSE_HIP_OK) return rc;
  SP_REQUIRE(T <= SPARSE_HIP_DECODE_MAX_TOKENS, "grouped_swiglu_decode: T=%d exceeds %d; use the prefill entry",
             T, SPARSE_HIP_DECODE_MAX_TOKENS);
  if (segs->n == 0) return SPARSE_HIP_OK;
  hipStream_t st = as_stream(stream);
  if (is_16bit(experts->dtype))
    return decode_routed_bf16(experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K, inter_ws_dev,
                              parts_dev, st);
  return tiled_routed<float>(experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K, inter_ws_dev,
                             parts_dev, st);
}

int sparse_hip_grouped_swiglu_prefill(const sparse_hip_experts* experts, const void* x_dev, const void* topv_dev,
                                      const int32_t* perm_dev, const int32_t* seg_offsets_dev,
                                      const sparse_hip_seglist* segs, int T, int K, void* inter_ws_dev,
                                      void* parts_dev, void* tile_ws_dev, void* stream) {
  int rc = check_routed("grouped_swiglu_prefill", experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T,
                        K, inter_ws_dev, parts_dev);
  if (rc != SPARSE_HIP_OK) return rc;
  if (segs->n == 0) return SPARSE_HIP_OK;
  hipStream_t st = as_stream(stream);
  if (is_16bit(experts->dtype)) {
    SP_REQUIRE(tile_ws_dev != nullptr && (reinterpret_cast<uintptr_t>(tile_ws_dev) & 15) == 0,
               "grouped_swiglu_prefill: tile workspace is NULL or not 16-byte aligned");
    return prefill_routed_bf16(experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K, inter_ws_dev,
                               parts_dev, tile_ws_dev, st);
  }
  return tiled_routed<float>(experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K, inter_ws_dev,
                             parts_dev, st);
}

size_t sparse_hip_moe_ffn_prefill_ws_bytes(int T, int K, int num_segments, int H, int I, int Is) {
  if (T <= 0 || K <= 0 || num_segments < 0 || H <= 0 || I <= 0 || Is < 0) return 0;
  return prefill_merged_ws_bytes(T, K, num_segments, H, I, Is);
}

int sparse_hip_moe_ffn_prefill(const sparse_hip_experts* experts, const void* x_dev, const void* topv_dev,
                               const int32_t* perm_dev, const int32_t* seg_offsets_dev,
                               const sparse_hip_seglist* segs, int T, int K, void* inter_ws_dev, void* parts_dev,
                               const void* sh_gate_w_dev, const void* sh_up_w_dev, const void* sh_down_w_dev,
                               const void* shared_gate_dev, int Is, void* sh_inter_ws_dev, void* shared_dev,
                               void* tile_ws_dev, void* stream) {
  int rc = check_routed("moe_ffn_prefill", experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K,
                        inter_ws_dev, parts_dev);
  if (rc != SPARSE_HIP_OK) return rc;
  SP_REQUIRE(is_16bit(experts->dtype), "moe_ffn_prefill: bf16 / fp16 only; use the separate entry points");
  const bool shared = sh_down_w_dev != nullptr;
  if (shared) {
    SP_REQUIRE(Is > 0 && Is % 64 == 0, "moe_ffn_prefill: Is=%d must be a positive multiple of 64", Is);
    SP_REQUIRE(sh_gate_w_dev && sh_up_w_dev && sh_inter_ws_dev && shared_dev,
               "moe_ffn_prefill: NULL shared-expert pointer");
    SP_REQUIRE(((reinterpret_cast<uintptr_t>(sh_gate_w_dev) | reinterpret_cast<uintptr_t>(sh_up_w_dev) |
                 reinterpret_cast<uintptr_t>(sh_down_w_dev) | reinterpret_cast<uintptr_t>(sh_inter_ws_dev) |
                 reinterpret_cast<uintptr_t>(shared_dev)) &
                15) == 0,
               "moe_ffn_prefill: shared-expert pointers must be 16-byte aligned");
  }
  SP_REQUIRE(tile_ws_dev != nullptr && (reinterpret_cast<uintptr_t>(tile_ws_dev) & 255) == 0,
             "moe_ffn_prefill: tile workspace is NULL or not 256-byte aligned");
  // lane offsets into an activation matrix are 32-bit byte counts
  const uint64_t widest = static_cast<uint64_t>(experts->hidden > experts->inter ? experts->hidden : experts->inter);
  SP_REQUIRE(static_cast<uint64_t>(T) * K * widest * 2 < (1ull << 32) &&
                 static_cast<uint64_t>(T) * (shared ? static_cast<uint64_t>(Is > experts->hidden ? Is : experts->hidden) : 1) * 2 < (1ull << 32),
             "moe_ffn_prefill: T=%d is too large for 32-bit row offsets; split the call", T);
  SP_REQUIRE(static_cast<uint64_t>(T) * K < (1ull << 32) / static_cast<uint64_t>(K), "moe_ffn_prefill: T*K too large");
  if (segs->n == 0 && !shared) return SPARSE_HIP_OK;
  return prefill_merged(experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K, inter_ws_dev, parts_dev,
                        sh_gate_w_dev, sh_up_w_dev, sh_down_w_dev, shared_gate_dev, Is, sh_inter_ws_dev,
                        shared_dev, tile_ws_dev, as_stream(stream));
}

int sparse_hip_moe_ffn_decode(const sparse_hip_experts* experts, const void* x_dev, const void* topv_dev,
                              const int32_t* perm_dev, const int32_t* seg_offsets_dev,
                              const sparse_hip_seglist* segs, int T, int K, void* inter_ws_dev, void* parts_dev,
                              const void* sh_gate_w_dev, const void* sh_up_w_dev, const void* sh_down_w_dev,
                              const void* shared_gate_dev, int Is, void* sh_inter_ws_dev, void* shared_dev,
                              void* split_ws_dev, void* stream) {
  int rc = check_routed("moe_ffn_decode", experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K,
                        inter_ws_dev, parts_dev);
  if (rc != SPARSE_HIP_OK) return rc;
  SP_REQUIRE(is_16bit(experts->dtype), "moe_ffn_decode: bf16 / fp16 only; use the separate entry points");
  SP_REQUIRE(T <= SPARSE_HIP_DECODE_MAX_TOKENS, "moe_ffn_decode: T=%d exceeds %d", T,
             SPARSE_HIP_DECODE_MAX_TOKENS);
  SP_REQUIRE(Is > 0 && Is % 64 == 0, "moe_ffn_decode: Is=%d must be a positive multiple of 64", Is);
  SP_REQUIRE(sh_down_w_dev && sh_inter_ws_dev && shared_dev, "moe_ffn_decode: NULL shared-expert pointer");
  SP_REQUIRE((sh_gate_w_dev == nullptr) == (sh_up_w_dev == nullptr),
             "moe_ffn_decode: shared gate and up projections are given together or not at all");
  SP_REQUIRE(((reinterpret_cast<uintptr_t>(sh_gate_w_dev) | reinterpret_cast<uintptr_t>(sh_up_w_dev) |
               reinterpret_cast<uintptr_t>(sh_down_w_dev) | reinterpret_cast<uintptr_t>(sh_inter_ws_dev) |
               reinterpret_cast<uintptr_t>(shared_dev) | reinterpret_cast<uintptr_t>(split_ws_dev)) &
              15) == 0,
             "moe_ffn_decode: shared-expert pointers must be 16-byte aligned");
  return decode_fused_bf16(experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K, inter_ws_dev,
                           parts_dev, sh_gate_w_dev, sh_up_w_dev, sh_down_w_dev, shared_gate_dev, Is,
                           sh_inter_ws_dev, shared_dev, split_ws_dev, nullptr, nullptr, as_stream(stream));
}

int sparse_hip_moe_ffn_decode_combine(const sparse_hip_experts* experts, const void* x_dev, const void* topv_dev,
                                      const int32_t* perm_dev, const int32_t* inv_perm_dev,
                                      const int32_t* seg_offsets_dev, const sparse_hip_seglist* segs, int T, int K,
                                      void* inter_ws_dev, void* parts_dev, const void* sh_gate_w_dev,
                                      const void* sh_up_w_dev, const void* sh_down_w_dev, const void* shared_gate_dev,
                                      int Is, void* sh_inter_ws_dev, void* split_ws_dev, void* out_dev, void* stream) {
  int rc = check_routed("moe_ffn_decode_combine", experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K,
                        inter_ws_dev, parts_dev);
  if (rc != SPARSE_HIP_OK) return rc;
  SP_REQUIRE(is_16bit(experts->dtype), "moe_ffn_decode_combine: bf16 / fp16 only");
  SP_REQUIRE(T <= SPARSE_HIP_DECODE_MAX_TOKENS, "moe_ffn_decode_combine: T=%d exceeds %d", T,
             SPARSE_HIP_DECODE_MAX_TOKENS);
  SP_REQUIRE(Is > 0 && Is % 64 == 0, "moe_ffn_decode_combine: Is=%d must be a positive multiple of 64", Is);
  SP_REQUIRE(decode_split_parts(Is) > 1,
             "moe_ffn_decode_combine: Is=%d cannot be cut into parts; use sparse_hip_moe_ffn_decode + sparse_hip_combine", Is);
  SP_REQUIRE(sh_down_w_dev && sh_inter_ws_dev && split_ws_dev && inv_perm_dev && out_dev,
             "moe_ffn_decode_combine: NULL pointer");
  SP_REQUIRE((sh_gate_w_dev == nullptr) == (sh_up_w_dev == nullptr),
             "moe_ffn_decode_combine: shared gate and up projections are given together or not at all");
  SP_REQUIRE(((reinterpret_cast<uintptr_t>(sh_gate_w_dev) | reinterpret_cast<uintptr_t>(sh_up_w_dev) |
               reinterpret_cast<uintptr_t>(sh_down_w_dev) | reinterpret_cast<uintptr_t>(sh_inter_ws_dev) |
               reinterpret_cast<uintptr_t>(out_dev) | reinterpret_cast<uintptr_t>(split_ws_dev)) &
              15) == 0,
             "moe_ffn_decode_combine: pointers must be 16-byte aligned");
  return decode_fused_bf16(experts, x_dev, topv_dev, perm_dev, seg_offsets_dev, segs, T, K, inter_ws_dev,
                           parts_dev, sh_gate_w_dev, sh_up_w_dev, sh_down_w_dev, shared_gate_dev, Is,
                           sh_inter_ws_dev, /*shared_out=*/out_dev, split_ws_dev, inv_perm_dev, out_dev,
                           as_stream(stream));
}

size_t sparse_hip_decode_split_counter_offset(int T, int H) {
  if (T < 1 || H < 1) return 0;
  return decode_split_counter_offset(T, H);
}

size_t sparse_hip_decode_split_ws_bytes(int T, int H) {
  if (T < 1 || H < 1) return 0;
  return decode_split_ws_bytes(T, H);
}

int sparse_hip_decode_split_parts(int Is) { return Is > 0 && Is % 64 == 0 ? decode_split_parts(Is) : 1; }

int sparse_hip_shared_expert(const void* x_dev, const void* gate_w_dev, const void* up_w_dev,
                             const void* down_w_dev, const void* shared_gate_dev, int dtype, int T, int H,
                             int Is, void* inter_ws_dev, void* shared_dev, void* stream) {
  SP_REQUIRE(valid_dtype(dtype), "shared_expert: unknown dtype %d", dtype);
  SP_REQUIRE(T >= 1, "shared_expert: T=%d must be >= 1", T);
  SP_REQUIRE(H > 0 && H % 64 == 0 && Is > 0 && Is % 64 == 0,
             "shared_expert: H=%d and Is=%d must be positive multiples of 64", H, Is);
  SP_REQUIRE(x_dev && down_w_dev && inter_ws_dev && shared_dev, "shared_expert: NULL pointer");
  SP_REQUIRE((gate_w_dev == nullptr) == (up_w_dev == nullptr),
             "shared_expert: gate and up projections are given together or not at all");
  SP_REQUIRE(gate_w_dev != nullptr || (is_16bit(dtype) && T <= SPARSE_HIP_DECODE_MAX_TOKENS),
             "shared_expert: only a 16-bit call of up to %d tokens can take a ready inter_ws", SPARSE_HIP_DECODE_MAX_TOKENS);
  SP_REQUIRE(((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(gate_w_dev) |
               reinterpret_cast<uintptr_t>(up_w_dev) | reinterpret_cast<uintptr_t>(down_w_dev) |
               reinterpret_cast<uintptr_t>(inter_ws_dev) | reinterpret_cast<uintptr_t>(shared_dev)) &
              15) == 0,
             "shared_expert: pointers must be 16-byte aligned");
  hipStream_t st = as_stream(stream);
  if (is_16bit(dtype)) {
    if (T <= SPARSE_HIP_DECODE_MAX_TOKENS)
      return decode_shared_bf16(x_dev, gate_w_dev, up_w_dev, down_w_dev, shared_gate_dev, dtype, T, H, Is,
                                inter_ws_dev, shared_dev, st);
    return prefill_shared_bf16(x_dev, gate_w_dev, up_w_dev, down_w_dev, shared_gate_dev, dtype, T, H, Is,
                               inter_ws_dev, shared_dev, st);
  }
  return tiled_shared<float>(x_dev, gate_w_dev, up_w_dev, down_w_dev, shared_gate_dev, T, H, Is, inter_ws_dev,
                             shared_dev, st);
}

}  // extern "C"
