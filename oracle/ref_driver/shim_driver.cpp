/*
 * shim_driver.cpp — replays a stream through the GpuChromeTraceLogger shim
 * (kineto_amd/shim/) exactly as ref_driver.cpp replays it through the real ChromeTraceLogger,
 * so that a test can compare the two files byte for byte.  The logger is obtained the way
 * libkineto obtains it: from an ActivityLoggerFactory (src/ActivityLoggerFactory.h:25-78) by
 * protocol prefix.
 *
 * TEST INFRASTRUCTURE ONLY; this repository's own code.
 */
#include <memory>
#include <stdexcept>
#include <string>

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
int ktj_shim_render(const ktj_stream* s, const ktj_mat_activity* acts, uint64_t n_acts, string_fn fn,
                    const void* ctx, const char* url, int hip_device, uint64_t* unsupported) {
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
  replay_stream(*shim, s, acts, n_acts, fn, ctx);
  if (unsupported) *unsupported = shim->unsupportedActivities();
  return shim->engineStatus();
}

}  // extern "C"
