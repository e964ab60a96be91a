// Library identity, error reporting, and the residency primitives of the C ABI:
// pinned-host -> HBM expert uploads on a caller-chosen stream, and the event/stream
// wrappers that gate readiness without host synchronisation.
#include "common.h"

#include <string.h>

#include <mutex>
#include <vector>

namespace sparse {

static thread_local char g_err[512] = {0};

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t err, const char* what) {
  set_error("%s: %s (%d)", what, hipGetErrorString(err), static_cast<int>(err));
  return SPARSE_HIP_ELAUNCH;
}

// ---- per-kernel event timing ---------------------------------------------------
struct ProfRec {
  hipEvent_t start, stop;
};
static std::mutex g_prof_mu;
static bool g_prof_on = false;
static std::vector<ProfRec> g_prof_recs[SPARSE_HIP_K_COUNT];
static std::vector<hipEvent_t> g_prof_free;

static hipEvent_t prof_take_event() {
  if (!g_prof_free.empty()) {
    hipEvent_t e = g_prof_free.back();
    g_prof_free.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}

ProfScope::ProfScope(int kernel, hipStream_t stream, bool dispatch_events)
    : kernel_(kernel), stream_(stream), start_(nullptr), stop_(nullptr) {
  if (!g_prof_on) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  start_ = prof_take_event();
  if (start_ == nullptr) return;
  if (dispatch_events) {
    stop_ = prof_take_event();
    if (stop_ == nullptr) {
      g_prof_free.push_back(start_);
      start_ = nullptr;
    }
    return;
  }
  (void)hipEventRecord(start_, stream_);
}

ProfScope::~ProfScope() {
  if (start_ == nullptr) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  if (stop_ != nullptr) {  // stamped by the launch itself
    g_prof_recs[kernel_].push_back(ProfRec{start_, stop_});
    return;
  }
  hipEvent_t stop = prof_take_event();
  if (stop == nullptr) {
    g_prof_free.push_back(start_);
    return;
  }
  (void)hipEventRecord(stop, stream_);
  g_prof_recs[kernel_].push_back(ProfRec{start_, stop});
}

}  // namespace sparse

using namespace sparse;

extern "C" {

int sparse_hip_version(void) { return SPARSE_HIP_ABI_VERSION; }

const char* sparse_hip_arch(void) { return "gfx950"; }

const char* sparse_hip_last_error(void) { return g_err; }

int sparse_hip_expert_upload_async(void* dst_dev, const void* src_host, size_t bytes, void* stream,
                                   void* event) {
  SP_REQUIRE(dst_dev != nullptr && src_host != nullptr, "expert_upload_async: NULL pointer");
  SP_REQUIRE(bytes > 0, "expert_upload_async: bytes must be > 0");
  SP_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, as_stream(stream)));
  if (event != nullptr) SP_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(stream)));
  return SPARSE_HIP_OK;
}

int sparse_hip_event_create(int timing, void** event_out) {
  SP_REQUIRE(event_out != nullptr, "event_create: NULL out pointer");
  hipEvent_t ev;
  SP_HIP(hipEventCreateWithFlags(&ev, timing ? hipEventDefault : hipEventDisableTiming));
  *event_out = ev;
  return SPARSE_HIP_OK;
}

int sparse_hip_event_destroy(void* event) {
  SP_REQUIRE(event != nullptr, "event_destroy: NULL event");
  SP_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
  return SPARSE_HIP_OK;
}

int sparse_hip_event_record(void* event, void* stream) {
  SP_REQUIRE(event != nullptr, "event_record: NULL event");
  SP_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(stream)));
  return SPARSE_HIP_OK;
}

int sparse_hip_event_query(void* event) {
  SP_REQUIRE(event != nullptr, "event_query: NULL event");
  hipError_t e = hipEventQuery(reinterpret_cast<hipEvent_t>(event));
  if (e == hipSuccess) return SPARSE_HIP_OK;
  if (e == hipErrorNotReady) return SPARSE_HIP_ENOTREADY;
  return hip_fail(e, "hipEventQuery");
}

int sparse_hip_stream_wait_event(void* stream, void* event) {
  SP_REQUIRE(event != nullptr, "stream_wait_event: NULL event");
  SP_HIP(hipStreamWaitEvent(as_stream(stream), reinterpret_cast<hipEvent_t>(event), 0));
  return SPARSE_HIP_OK;
}

int sparse_hip_event_elapsed_ms(void* start, void* stop, float* ms_out) {
  SP_REQUIRE(start != nullptr && stop != nullptr && ms_out != nullptr, "event_elapsed_ms: NULL argument");
  SP_HIP(hipEventElapsedTime(ms_out, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)));
  return SPARSE_HIP_OK;
}

int sparse_hip_stream_create(void** stream_out) {
  SP_REQUIRE(stream_out != nullptr, "stream_create: NULL out pointer");
  hipStream_t s;
  SP_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream_out = s;
  return SPARSE_HIP_OK;
}

int sparse_hip_stream_destroy(void* stream) {
  SP_REQUIRE(stream != nullptr, "stream_destroy: NULL stream");
  SP_HIP(hipStreamDestroy(as_stream(stream)));
  return SPARSE_HIP_OK;
}

int sparse_hip_stream_synchronize(void* stream) {
  SP_HIP(hipStreamSynchronize(as_stream(stream)));
  return SPARSE_HIP_OK;
}

int sparse_hip_host_alloc(size_t bytes, void** ptr_out) {
  SP_REQUIRE(ptr_out != nullptr && bytes > 0, "host_alloc: bad argument");
  void* p = nullptr;
  SP_HIP(hipHostMalloc(&p, bytes, hipHostMallocDefault));
  *ptr_out = p;
  return SPARSE_HIP_OK;
}

int sparse_hip_host_free(void* ptr) {
  SP_REQUIRE(ptr != nullptr, "host_free: NULL pointer");
  SP_HIP(hipHostFree(ptr));
  return SPARSE_HIP_OK;
}

int sparse_hip_profile_enable(int on) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  g_prof_on = on != 0;
  return SPARSE_HIP_OK;
}

int sparse_hip_profile_reset(void) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  for (auto& recs : g_prof_recs) {
    for (auto& r : recs) {
      g_prof_free.push_back(r.start);
      g_prof_free.push_back(r.stop);
    }
    recs.clear();
  }
  return SPARSE_HIP_OK;
}

int sparse_hip_profile_read(int kernel, double* total_ms_out, int64_t* launches_out) {
  SP_REQUIRE(kernel >= 0 && kernel < SPARSE_HIP_K_COUNT, "profile_read: kernel id %d outside [0,%d)", kernel,
             SPARSE_HIP_K_COUNT);
  SP_REQUIRE(total_ms_out != nullptr && launches_out != nullptr, "profile_read: NULL output");
  std::lock_guard<std::mutex> lk(g_prof_mu);
  double total = 0.0;
  for (auto& r : g_prof_recs[kernel]) {
    SP_HIP(hipEventSynchronize(r.stop));
    float ms = 0.f;
    SP_HIP(hipEventElapsedTime(&ms, r.start, r.stop));
    total += ms;
  }
  *total_ms_out = total;
  *launches_out = static_cast<int64_t>(g_prof_recs[kernel].size());
  return SPARSE_HIP_OK;
}

const char* sparse_hip_kernel_name(int kernel) {
  static const char* names[SPARSE_HIP_K_COUNT] = {
      "router_logits_kernel", "gate_topk_kernel",   "permute_scatter_kernel", "decode_ffn_kernel<F, true>",
      "decode_ffn_kernel<F, false>", "prefill_ffn_kernel<F, true>", "prefill_ffn_kernel<F, false>",
      "ffn_tiled_kernel<gate_up>", "ffn_tiled_kernel<down>", "combine_kernel", "route_decode_kernel"};
  if (kernel < 0 || kernel >= SPARSE_HIP_K_COUNT) return "";
  return names[kernel];
}

}  // extern "C"
