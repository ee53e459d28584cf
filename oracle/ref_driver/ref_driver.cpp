/*
 * ref_driver.cpp — drives the *real* libkineto ChromeTraceLogger (compiled from the reference
 * sources where they lie, see ../Makefile) with activities described by plain structs.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is this repository's own code: adaptor structs that
 * implement libkineto::ITraceActivity over ktj_mat_activity, and C entry points for the tests.
 * All formatting is done by the reference: ChromeTraceLogger (src/output_json.cpp),
 * JsonTypedMetadataVisitor (include/TypedMetadataJson.h), GenericTraceActivity
 * (src/GenericTraceActivity.cpp) and fmt.
 */
#include <algorithm>
#include <cstring>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "ActivityType.h"
#include "Config.h"
#include "GenericTraceActivity.h"
#include "ITraceActivity.h"
#include "Logger.h"
#include "TraceSpan.h"
#include "TypedMetadataJson.h"
#include "output_json.h"

#include "../ktj_oracle.h"

using namespace libkineto;

#include "mat_activity.h"

using namespace ktj_ref_driver;

namespace {

// Exposes the protected finalizeTrace(int64_t) so that no Config object is needed.
struct RefLogger : public ChromeTraceLogger {
  using ChromeTraceLogger::ChromeTraceLogger;
  using ChromeTraceLogger::finalizeTrace;
};

}  // namespace

extern "C" {

int64_t ktj_ref_base_time(void) { return ChromeTraceBaseTime::singleton().get(); }

// Renders the stream's header/infos/spans and the given activities with the real logger into
// out_path, with the activities stable-sorted by (deviceId, resourceId, timestamp); call_order as
// described at replay_stream (0: the buffering logger's replay, 1: the profiler's own order), and
// so is wide_device_mod (activities that report a deviceId beyond 32 bits).
int ktj_ref_render(const ktj_stream* s, const ktj_mat_activity* acts, uint64_t n_acts, string_fn fn,
                   const void* ctx, const char* out_path, int call_order, int wide_device_mod) {
  SET_LOG_SEVERITY_LEVEL(3);  // ERROR: silence per-name WARNING lines
  if (s->base_time_ns != ChromeTraceBaseTime::singleton().get()) return -2;
  RefLogger logger{std::string(out_path)};
  replay_stream(logger, s, acts, n_acts, fn, ctx, call_order, wide_device_mod);
  return 0;
}

// fmt "{}" on a double, as TypedMetadataJson.h:172-178 and GenericTraceActivity.h:107-109 use it.
size_t ktj_ref_fmt_double(double v, char* out) {
  std::string r = fmt::format("{}", v);
  std::memcpy(out, r.data(), r.size());
  out[r.size()] = 0;
  return r.size();
}

// Inserts n typed int64 entries with the given keys, in the given order, into a real
// GenericTraceActivity and returns the metadataJson() the reference produces; the key order in
// that string is the iteration order of its unordered_map.
size_t ktj_ref_metadata_order(const char* const* keys, uint64_t n, char* out, size_t cap) {
  TraceSpan span(0, 0, "s");
  GenericTraceActivity act(span, ActivityType::CPU_OP, "x");
  for (uint64_t i = 0; i < n; ++i) act.addTypedMetadata(keys[i], TypedValue{static_cast<int64_t>(i)});
  std::string r = act.metadataJson();
  if (r.size() + 1 > cap) return 0;
  std::memcpy(out, r.data(), r.size() + 1);
  return r.size();
}

// A real GenericTraceActivity with string-keyed addMetadata / addMetadataQuoted values, logged
// through the real ChromeTraceLogger; used to pin the RawJson path of
// test/GenericTraceActivityMetadataTest.cpp.
size_t ktj_ref_generic_metadata(int n, const char* const* keys, const int* kinds, const int64_t* ivals,
                                const double* dvals, const char* const* svals, char* out, size_t cap) {
  TraceSpan span(0, 0, "s");
  GenericTraceActivity act(span, ActivityType::CPU_OP, "x");
  for (int i = 0; i < n; ++i) {
    switch (kinds[i]) {
      case 0: act.addMetadata(keys[i], ivals[i]); break;
      case 1: act.addMetadata(keys[i], dvals[i]); break;
      case 2: act.addMetadataQuoted(keys[i], svals[i]); break;
      case 3: act.addMetadata(keys[i], ivals[i] != 0); break;
      case 4: act.addMetadata(keys[i], static_cast<uint64_t>(ivals[i])); break;
      default: break;
    }
  }
  std::string r = act.metadataJson();
  if (r.size() + 1 > cap) return 0;
  std::memcpy(out, r.data(), r.size() + 1);
  return r.size();
}

}  // extern "C"
