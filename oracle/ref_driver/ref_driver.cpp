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

namespace {

typedef void (*string_fn)(const void* ctx, uint32_t id, const char** p, uint64_t* n);

struct StringTable {
  string_fn fn;
  const void* ctx;
  std::string get(uint32_t id) const {
    const char* p = nullptr;
    uint64_t n = 0;
    fn(ctx, id, &p, &n);
    return std::string(p, n);
  }
};

// ITraceActivity over one materialised activity.  metadataJson() feeds the typed values, in
// visit order, through the reference's JsonTypedMetadataVisitor.
struct MatActivity : public ITraceActivity {
  const ktj_mat_activity* a;
  const StringTable* st;
  mutable GenericTraceActivity linkedStub;  // only correlationId()/name() are read from it
  bool hasLinked;

  MatActivity(const ktj_mat_activity* act, const StringTable* s) : a(act), st(s), hasLinked(act->has_linked != 0) {
    linkedStub.id = static_cast<int32_t>(act->linked_corr);
    linkedStub.activityName = "linked_op";
  }
  int64_t deviceId() const override { return a->device; }
  int64_t resourceId() const override { return a->resource; }
  int32_t getThreadId() const override { return 0; }
  int64_t timestamp() const override { return a->ts; }
  int64_t duration() const override { return a->dur; }
  int64_t correlationId() const override { return a->corr; }
  int flowType() const override { return a->flow_type; }
  int64_t flowId() const override { return a->flow_id; }
  bool flowStart() const override { return a->flow_start != 0; }
  ActivityType type() const override { return static_cast<ActivityType>(a->type); }
  const std::string name() const override { return st->get(a->name_id); }
  const ITraceActivity* linkedActivity() const override { return hasLinked ? &linkedStub : nullptr; }
  const TraceSpan* traceSpan() const override { return nullptr; }
  void log(ActivityLogger& logger) const override { logger.handleActivity(*this); }

  void visitTypedMetadata(ITypedMetadataVisitor& visitor) const override {
    const uint64_t* slot = a->slots;
    std::vector<std::string> keep;  // MetadataField holds a string_view
    keep.reserve(a->n_fields);
    for (uint32_t f = 0; f < a->n_fields; ++f) {
      const ktj_field& fd = a->fields[f];
      keep.push_back(fd.key_id == KTJ_NONE ? std::string() : st->get(fd.key_id));
      const std::string& key = keep.back();
      switch (fd.type) {
        case KTJ_F_I64:
          visitor.visit(MetadataField<int64_t>{key}, static_cast<int64_t>(slot[0]));
          break;
        case KTJ_F_U64:
          visitor.visit(MetadataField<uint64_t>{key}, static_cast<uint64_t>(slot[0]));
          break;
        case KTJ_F_F64: {
          double d;
          std::memcpy(&d, &slot[0], 8);
          visitor.visit(MetadataField<double>{key}, d);
          break;
        }
        case KTJ_F_BOOL:
          visitor.visit(MetadataField<bool>{key}, slot[0] != 0);
          break;
        case KTJ_F_STR:
          visitor.visit(MetadataField<std::string>{key}, st->get(static_cast<uint32_t>(slot[0])));
          break;
        case KTJ_F_RAW:
          visitor.visit(MetadataField<RawJson>{key}, RawJson{st->get(static_cast<uint32_t>(slot[0]))});
          break;
        case KTJ_F_I64_ARRAY: {
          std::vector<int64_t> v(fd.count);
          for (uint32_t k = 0; k < fd.count; ++k) v[k] = static_cast<int64_t>(slot[k]);
          visitor.visit(MetadataField<std::vector<int64_t>>{key}, v);
          break;
        }
        default:
          break;
      }
      slot += fd.count;
    }
  }
  const std::string metadataJson() const override {
    // A field without a key stands for a whole pre-rendered fragment (what an activity's own
    // metadataJson() returned); it is passed through untouched.
    if (a->n_fields == 1 && a->fields[0].key_id == KTJ_NONE) {
      return st->get(static_cast<uint32_t>(a->slots[0]));
    }
    libkineto::internal::JsonTypedMetadataVisitor visitor;
    visitTypedMetadata(visitor);
    return std::move(visitor).json();
  }
};

// Exposes the protected finalizeTrace(int64_t) so that no Config object is needed.
struct RefLogger : public ChromeTraceLogger {
  using ChromeTraceLogger::ChromeTraceLogger;
  using ChromeTraceLogger::finalizeTrace;
};

}  // namespace

extern "C" {

int64_t ktj_ref_base_time(void) { return ChromeTraceBaseTime::singleton().get(); }

// Renders the stream's header/infos/spans and the given activities with the real logger into
// out_path, in the order of the reference's buffering logger (src/output_membuf.h:91-107) with
// the activities stable-sorted by (deviceId, resourceId, timestamp).
int ktj_ref_render(const ktj_stream* s, const ktj_mat_activity* acts, uint64_t n_acts, string_fn fn,
                   const void* ctx, const char* out_path) {
  SET_LOG_SEVERITY_LEVEL(3);  // ERROR: silence per-name WARNING lines
  if (s->base_time_ns != ChromeTraceBaseTime::singleton().get()) return -2;
  StringTable st{fn, ctx};
  std::vector<MatActivity> wrapped;
  wrapped.reserve(n_acts);
  for (uint64_t i = 0; i < n_acts; ++i) wrapped.emplace_back(&acts[i], &st);
  std::vector<const MatActivity*> order(n_acts);
  for (uint64_t i = 0; i < n_acts; ++i) order[i] = &wrapped[i];
  std::stable_sort(order.begin(), order.end(), [](const MatActivity* x, const MatActivity* y) {
    return std::make_tuple(x->deviceId(), x->resourceId(), x->timestamp()) <
        std::make_tuple(y->deviceId(), y->resourceId(), y->timestamp());
  });

  RefLogger logger{std::string(out_path)};
  std::unordered_map<std::string, std::string> metadata;  // env metadata (host_name) is added by the logger
  logger.handleTraceStart(metadata, s->device_properties ? s->device_properties : "");
  for (uint64_t i = 0; i < s->n_device_infos; ++i) {
    const ktj_device_info& d = s->device_infos[i];
    logger.handleDeviceInfo({d.id, d.sort_index, d.name, d.label}, d.time_ns);
  }
  for (uint64_t i = 0; i < s->n_resource_infos; ++i) {
    const ktj_resource_info& r = s->resource_infos[i];
    logger.handleResourceInfo(
        {r.id, r.sort_index, r.device_id, r.name, r.host_thread ? ResourceType::HOST_THREAD : ResourceType::UNKNOWN},
        r.time_ns);
  }
  for (uint64_t i = 0; i < s->n_overhead_infos; ++i) {
    logger.handleOverheadInfo(ActivityLogger::OverheadInfo(s->overhead_infos[i].name), s->overhead_infos[i].time_ns);
  }
  for (const MatActivity* a : order) a->log(logger);
  for (uint64_t i = 0; i < s->n_spans; ++i) {
    const ktj_trace_span& sp = s->spans[i];
    TraceSpan span(sp.op_count, sp.iteration, sp.name, sp.prefix);
    span.startTime = sp.start_ns;
    span.endTime = sp.end_ns;
    logger.handleTraceSpan(span);
  }
  logger.finalizeTrace(s->end_time_ns);
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
