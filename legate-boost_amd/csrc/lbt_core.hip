// Error reporting, version and the event-based profiler of liblbtree.so.
#include "lbt_internal.h"

#include <cstring>

namespace lbt {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...)
{
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

ThreadResources& thread_resources()
{
  static thread_local ThreadResources tr;
  return tr;
}

Profiler& profiler()
{
  static Profiler p;
  return p;
}

void Profiler::begin(int cls, int level, double bytes, hipStream_t s)
{
  ProfSpan sp{};
  sp.cls   = cls;
  sp.level = level;
  sp.bytes = bytes;
  // events are kept and reused: creating a pair per span costs more than recording it
  auto take = [&](hipEvent_t* e) {
    if (!pool.empty()) {
      *e = pool.back();
      pool.pop_back();
      return true;
    }
    return hipEventCreate(e) == hipSuccess;
  };
  if (!take(&sp.start)) return;
  if (!take(&sp.stop)) {
    pool.push_back(sp.start);
    return;
  }
  (void)hipEventRecord(sp.start, s);
  open.push_back(sp);
}

void Profiler::end(hipStream_t s)
{
  if (open.empty()) return;
  (void)hipEventRecord(open.back().stop, s);
}

void Profiler::collect()
{
  for (auto& sp : open) {
    float ms = 0.f;
    if (hipEventSynchronize(sp.stop) == hipSuccess &&
        hipEventElapsedTime(&ms, sp.start, sp.stop) == hipSuccess) {
      acc.launches[sp.cls] += 1;
      acc.ms[sp.cls] += ms;
      acc.bytes[sp.cls] += sp.bytes;
      if (sp.cls == LBT_PROF_HISTOGRAM && sp.level >= 0 && sp.level < 64) {
        if (sp.level + 1 > acc.n_levels) acc.n_levels = sp.level + 1;
        acc.level_ms[sp.level] += ms;
        acc.level_bytes[sp.level] += sp.bytes;
      }
    }
    pool.push_back(sp.start);
    pool.push_back(sp.stop);
  }
  open.clear();
  for (auto& lv : levels) {
    if (hipEventSynchronize(lv.arrived) == hipSuccess) {
      for (int d = 0; d < lv.levels && d < 64; d++) {
        const LevelCounts& c = lv.host[d];
        // algorithmic bytes of the histogram launches of the level: the feature values and packed
        // gradients of the rows of built nodes, one position per row, the built histograms once
        double by = static_cast<double>(c.built_instances) * lv.bytes_per_built_row +
                    static_cast<double>(c.built_nodes) * lv.bytes_per_built_node + (d == 0 ? lv.root_extra_bytes : 0.0);
        acc.level_bytes[d] += by;
        acc.level_instances[d] += static_cast<double>(c.instances);
        acc.level_built_instances[d] += static_cast<double>(c.built_instances);
        acc.level_built_nodes[d] += static_cast<double>(c.built_nodes);
        acc.bytes[LBT_PROF_HISTOGRAM] += by;
      }
    }
    pool.push_back(lv.arrived);
    level_pool.push_back(lv.host);
  }
  levels.clear();
}

ProfLevels* Profiler::begin_levels(int n_levels, double per_row, double per_node, double root_extra)
{
  ProfLevels lv{};
  if (!level_pool.empty()) {
    lv.host = level_pool.back();
    level_pool.pop_back();
  } else if (hipHostMalloc(reinterpret_cast<void**>(&lv.host), sizeof(LevelCounts) * 64, hipHostMallocDefault) !=
             hipSuccess) {
    return nullptr;
  }
  if (!pool.empty()) {
    lv.arrived = pool.back();
    pool.pop_back();
  } else if (hipEventCreate(&lv.arrived) != hipSuccess) {
    level_pool.push_back(lv.host);
    return nullptr;
  }
  lv.levels               = n_levels;
  lv.bytes_per_built_row  = per_row;
  lv.bytes_per_built_node = per_node;
  lv.root_extra_bytes     = root_extra;
  levels.push_back(lv);
  return &levels.back();
}

// Takes the thread's handles out of its record first and then releases every one of them, also
// after a failure in between: nothing that was freed or destroyed stays reachable for a later
// call. The first failure is what is reported.
int release_thread_resources()
{
  ThreadResources& tr = thread_resources();
  const ThreadResources old = tr;
  tr = ThreadResources{};
  hipError_t first = hipSuccess;
  const char* what = "";
  auto note = [&](hipError_t e, const char* call) {
    if (e != hipSuccess && first == hipSuccess) {
      first = e;
      what  = call;
    }
  };
  // the buffers may still feed or receive copies of calls that did not wait
  if (old.stage_free != nullptr) note(hipEventSynchronize(old.stage_free), "hipEventSynchronize");
  if (old.counts_here != nullptr) note(hipEventSynchronize(old.counts_here), "hipEventSynchronize");
  if (old.stats_here != nullptr) note(hipEventSynchronize(old.stats_here), "hipEventSynchronize");
  if (old.stage != nullptr) note(hipHostFree(old.stage), "hipHostFree");
  if (old.mirror != nullptr) note(hipHostFree(old.mirror), "hipHostFree");
  if (old.stage_free != nullptr) note(hipEventDestroy(old.stage_free), "hipEventDestroy");
  if (old.counts_here != nullptr) note(hipEventDestroy(old.counts_here), "hipEventDestroy");
  if (old.stats_here != nullptr) note(hipEventDestroy(old.stats_here), "hipEventDestroy");
  if (first != hipSuccess) {
    set_error("%s failed while the thread's resources were released: %s", what, hipGetErrorString(first));
    return LBT_ERR_HIP;
  }
  return LBT_OK;
}

// The thread's resources for the current device: events and pinned buffers belong to the device
// they were created on, so a thread that has moved to another device starts afresh.
int thread_resources_here(ThreadResources** out)
{
  int device = 0;
  LBT_HIP(hipGetDevice(&device));
  ThreadResources& tr = thread_resources();
  const bool holds = tr.mirror != nullptr || tr.stage != nullptr || tr.counts_here != nullptr ||
                     tr.stats_here != nullptr || tr.stage_free != nullptr;
  if (holds && tr.device != device) {
    const int now = device;
    LBT_HIP(hipSetDevice(tr.device));
    const int rc = release_thread_resources();
    LBT_HIP(hipSetDevice(now));
    LBT_TRY(rc);
  }
  thread_resources().device = device;
  *out = &thread_resources();
  return LBT_OK;
}

}  // namespace lbt

extern "C" {

const char* lbt_last_error(void) { return lbt::g_error; }

int lbt_version(void) { return 3; }

int lbt_release_thread_resources(void) { return lbt::release_thread_resources(); }

void lbt_profile_enable(int on) { lbt::profiler().mode = on < 0 ? 0 : on; }

void lbt_profile_reset(void)
{
  auto& p = lbt::profiler();
  p.collect();
  std::memset(&p.acc, 0, sizeof(p.acc));
}

void lbt_profile_get(lbt_profile* out)
{
  // waits for the calls that returned without synchronising
  lbt::profiler().collect();
  if (out) *out = lbt::profiler().acc;
}

}  // extern "C"
