// Optional per-kernel timing with HIP events recorded on the launch stream.
// Off by default; when on, every tagged launch site records an event before
// and after its kernel(s).  Reading a tag synchronises on its events.
#include <atomic>
#include <mutex>
#include <vector>

#include "zen_common.h"

namespace zen {
namespace {

struct Span {
  int tag;
  hipEvent_t start, stop;
};

std::mutex g_mu;
std::atomic<bool> g_on{false};  // read without the mutex at every tagged launch site
int g_only = -1;  // >= 0: only launches with this tag are timed
int g_every = 1;  // of which every g_every-th one
int64_t g_seen[kProfCount];  // launches per tag since recording began
std::vector<Span> g_spans;
std::vector<hipEvent_t> g_spare;  // created ahead of the timed launches: creating an event costs host time

constexpr size_t kSpareEvents = 2048;

hipEvent_t take_event() {
  if (!g_spare.empty()) {
    hipEvent_t e = g_spare.back();
    g_spare.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  return hipEventCreate(&e) == hipSuccess ? e : nullptr;
}

const char *const kNames[kProfCount] = {
    "k_topk_hist", "k_select_compact", "k_insert_list", "k_final_key", "sort_pairs",
    "k_gather",    "k_merge_prep",     "k_merge_reduce", "k_compress", "k_insert_dense",
    "k_select_stage", "k_coarse_scatter+k_fine_scatter", "k_slab_sort", "k_slab_chains+classify", "k_slab_place",
    "merge: k_coarse_scatter+k_fine_scatter", "k_merge_bucket", "k_sample_hist", "k_decode_fused",
    "k_wide_tail", "k_wide_scatter", "k_wide_merge",
};

void drop_spans() {  // the events go back to the spare list (a read has waited for them, or nobody will)
  for (Span &s : g_spans) {
    g_spare.push_back(s.start);
    g_spare.push_back(s.stop);
  }
  g_spans.clear();
}

}  // namespace

ProfScope::ProfScope(int tag, hipStream_t stream) : tag_(tag), stream_(stream), start_(nullptr), stop_(nullptr) {
  if (!g_on.load(std::memory_order_relaxed)) return;  // off: host threads that enqueue side by side do not meet here
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_on.load(std::memory_order_relaxed) || (g_only >= 0 && tag != g_only)) return;
  if (g_seen[tag]++ % g_every != 0) return;
  start_ = take_event();
  stop_ = start_ ? take_event() : nullptr;
  if (!stop_) {
    if (start_) g_spare.push_back(start_);
    start_ = nullptr;
    return;
  }
  (void)hipEventRecord(start_, stream_);
}

ProfScope::~ProfScope() {
  if (!start_) return;
  (void)hipEventRecord(stop_, stream_);
  std::lock_guard<std::mutex> lock(g_mu);
  g_spans.push_back(Span{tag_, start_, stop_});
}

}  // namespace zen

extern "C" {

int zen_profile_enable(int on) {
  std::lock_guard<std::mutex> lock(zen::g_mu);
  zen::drop_spans();
  zen::g_on.store(on != 0, std::memory_order_relaxed);
  for (int64_t &c : zen::g_seen) c = 0;
  while (on != 0 && zen::g_spare.size() < zen::kSpareEvents) {
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) break;
    zen::g_spare.push_back(e);
  }
  return ZEN_OK;
}

int zen_profile_only(int tag) {
  if (tag >= zen::kProfCount) return zen::fail(ZEN_EINVAL, "zen_profile_only: no such tag");
  std::lock_guard<std::mutex> lock(zen::g_mu);
  zen::g_only = tag < 0 ? -1 : tag;
  return ZEN_OK;
}

int zen_profile_every(int n) {
  if (n < 1) return zen::fail(ZEN_EINVAL, "zen_profile_every: n must be at least 1");
  std::lock_guard<std::mutex> lock(zen::g_mu);
  zen::g_every = n;
  return ZEN_OK;
}

int zen_profile_tags(void) { return zen::kProfCount; }

const char *zen_profile_name(int tag) {
  return tag >= 0 && tag < zen::kProfCount ? zen::kNames[tag] : "";
}

int zen_profile_read(int tag, double *total_ms, int64_t *launches) {
  using namespace zen;
  if (!total_ms || !launches || tag < 0 || tag >= kProfCount) return fail(ZEN_EINVAL, "zen_profile_read: bad argument");
  std::lock_guard<std::mutex> lock(g_mu);
  double sum = 0;
  int64_t count = 0;
  for (const Span &s : g_spans) {
    if (s.tag != tag) continue;
    ZEN_HIP_CHECK(hipEventSynchronize(s.stop));
    float ms = 0;
    ZEN_HIP_CHECK(hipEventElapsedTime(&ms, s.start, s.stop));
    sum += ms;
    ++count;
  }
  *total_ms = sum;
  *launches = count;
  return ZEN_OK;
}

}  // extern "C"
