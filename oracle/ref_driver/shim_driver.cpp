/*
 * shim_driver.cpp — replays a stream through the GpuChromeTraceLogger shim
 * (kineto_amd/shim/) exactly as ref_driver.cpp replays it through the real ChromeTraceLogger,
 * so that a test can compare the two files byte for byte.  The logger is obtained the way
 * libkineto obtains it: from an ActivityLoggerFactory (src/ActivityLoggerFactory.h:25-78) by
 * protocol prefix.
 *
 * TEST INFRASTRUCTURE ONLY; this repository's own code.
 */
#include <chrono>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "ActivityLoggerFactory.h"
#include "Logger.h"
#include "output_json.h"

#include "GpuChromeTraceLogger.h"
#include "mat_activity.h"

using namespace ktj_ref_driver;

namespace {
struct ShimLogger : public ktj_shim::GpuChromeTraceLogger {
  using GpuChromeTraceLogger::GpuChromeTraceLogger;
  using GpuChromeTraceLogger::finalizeTrace;
};
}  // namespace

extern "C" {

int64_t ktj_shim_base_time(void) { return ChromeTraceBaseTime::singleton().get(); }

// url is "<protocol>://<path>"; the protocol is registered here with a factory that builds the
// shim.  Returns 0, -2 for a base-time mismatch, -3 if the factory did not produce the shim,
// else the shim's engine status.  *unsupported receives the number of dropped activities.
// bulk_threads > 0: the activities are handed over in one handleActivities() call with that many
// workers, as GenericTraceActivity objects (so that the workers pack them).
// huge_device_mod > 0: every activity whose arrival index is 1 modulo it reports a deviceId
// beyond 32 bits (replay_stream's wide_device_mod); *unsupported stays 0 for them.
// call_order: see replay_stream (0: the buffering logger's replay; 2: the calls as
// GenericActivityProfiler issues them, activities unsorted and split around the CPU span).
int ktj_shim_render(const ktj_stream* s, const ktj_mat_activity* acts, uint64_t n_acts, string_fn fn,
                    const void* ctx, const char* url, int hip_device, uint64_t* unsupported, int bulk_threads,
                    int huge_device_mod, int call_order) {
  SET_LOG_SEVERITY_LEVEL(3);
  if (s->base_time_ns != ChromeTraceBaseTime::singleton().get()) return -2;
  ActivityLoggerFactory factory;
  factory.addProtocol("GpuJson", [hip_device](const std::string& path) {
    return std::unique_ptr<ActivityLogger>(new ShimLogger(path, hip_device));
  });
  std::unique_ptr<ActivityLogger> logger;
  try {
    logger = factory.makeLogger(url);
  } catch (const std::invalid_argument&) {
    return -3;
  }
  auto* shim = dynamic_cast<ShimLogger*>(logger.get());
  if (shim == nullptr) return -3;
  if (bulk_threads > 0) {
    replay_stream(*shim, s, acts, n_acts, fn, ctx, [&](ShimLogger& l, const std::vector<const MatActivity*>& order) {
      std::vector<GenericMatActivity> generic;
      generic.reserve(order.size());
      std::vector<const ITraceActivity*> all;
      all.reserve(order.size());
      for (size_t i = 0; i < order.size(); ++i) {
        if (i % 7 == 3) all.push_back(order[i]); /* some stay plain ITraceActivity: packed by the calling thread */
        else { generic.emplace_back(order[i]); all.push_back(&generic.back()); }
      }
      l.handleActivities(all, static_cast<unsigned>(bulk_threads));
    }, call_order, huge_device_mod);
  } else if (huge_device_mod > 0) {
    replay_stream(*shim, s, acts, n_acts, fn, ctx, [&](ShimLogger& l, const std::vector<const MatActivity*>& order) {
      for (const MatActivity* a : order) {
        if (a->wideDevice) { const GenericMatActivity g(a); l.handleActivity(g); }
        else a->log(l);
      }
    }, call_order, huge_device_mod);
  } else {
    replay_stream(*shim, s, acts, n_acts, fn, ctx, call_order);
  }
  if (unsupported) *unsupported = shim->unsupportedActivities();
  return shim->engineStatus();
}

// Times handleActivities() alone (host-side packing, merge and hand-over to the engine; no
// finalizeTrace) on n CPU-op activities with typed metadata, as a profiler's CpuTraceBuffer holds
// them.  Returns the engine status; *seconds receives the wall time of the call.
int ktj_shim_time_bulk(uint64_t n, int threads, const char* path, int hip_device, double* seconds) {
  SET_LOG_SEVERITY_LEVEL(3);
  ShimLogger shim(path, hip_device);
  shim.handleTraceStart({}, "");
  TraceSpan span(0, 0, "bench");
  std::vector<GenericTraceActivity> acts;
  acts.reserve(n);
  const int64_t base = ChromeTraceBaseTime::singleton().get();
  for (uint64_t i = 0; i < n; ++i) {
    acts.emplace_back(span, ActivityType::CPU_OP, "aten::op_" + std::to_string(i % 997));
    GenericTraceActivity& a = acts.back();
    a.startTime = base + static_cast<int64_t>(i) * 1000;
    a.endTime = a.startTime + 500;
    a.device = 4000;
    a.resource = 4001 + static_cast<int32_t>(i % 8);
    a.id = static_cast<int32_t>(i + 1);
    a.addMetadata("Sequence number", static_cast<int64_t>(i));
    a.addMetadata("Fwd thread id", 0);
    a.addMetadataQuoted("Input type", "float");
  }
  std::vector<const ITraceActivity*> all;
  all.reserve(n);
  for (const auto& a : acts) all.push_back(&a);
  const auto t0 = std::chrono::steady_clock::now();
  shim.handleActivities(all, static_cast<unsigned>(threads));
  const auto t1 = std::chrono::steady_clock::now();
  if (seconds) *seconds = std::chrono::duration<double>(t1 - t0).count();
  shim.finalizeTrace(base + static_cast<int64_t>(n) * 1000 + 1000);
  return shim.engineStatus();
}

}  // extern "C"
