/*
 * mat_activity.h — libkineto::ITraceActivity over one materialised activity of the CPU checker
 * (ktj_mat_activity), shared by the drivers of the real ChromeTraceLogger and of the
 * GpuChromeTraceLogger shim.  TEST INFRASTRUCTURE ONLY; this repository's own code.
 */
#pragma once

#include <algorithm>
#include <cstring>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "ActivityType.h"
#include "GenericTraceActivity.h"
#include "ITraceActivity.h"
#include "TraceSpan.h"
#include "TypedMetadataJson.h"
#include "output_base.h"

#include "../ktj_oracle.h"

namespace ktj_ref_driver {
using namespace libkineto;

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
  bool wideDevice = false;  // reports a deviceId beyond 32 bits (set by replay_stream)

  // collectives: ktj_stream::collectives; an activity whose linked op carries collective metadata
  // gets a record_param_comms op with those values as its linked activity
  MatActivity(const ktj_mat_activity* act, const StringTable* s, const ktj_collective_meta* collectives = nullptr)
      : a(act), st(s), hasLinked(act->has_linked != 0) {
    linkedStub.id = static_cast<int32_t>(act->linked_corr);
    linkedStub.activityName = "linked_op";
    if (act->collective != 0 && collectives != nullptr) {
      const ktj_collective_meta& m = collectives[act->collective - 1];
      linkedStub.activityName = "record_param_comms";
      const std::pair<const char*, const char*> kv[] = {
          {"Collective name", m.collective_name}, {"In msg nelems", m.in_msg_nelems}, {"Out msg nelems", m.out_msg_nelems},
          {"Group size", m.group_size}, {"dtype", m.dtype}, {"Input Tensors start", m.in_tensors_start},
          {"Output Tensors start", m.out_tensors_start}, {"In split size", m.in_split}, {"Out split size", m.out_split},
          {"Process Group Name", m.pg_name}, {"Process Group Description", m.pg_desc},
          {"Process Group Ranks", m.group_ranks}, {"Dst Rank", m.dst_rank}, {"Src Rank", m.src_rank}, {"Seq", m.seq},
          {"Comms Id", m.comms_id}, {"Rank", m.rank}};
      for (const auto& e : kv)
        if (e.second != nullptr && e.second[0] != 0) linkedStub.addMetadata(std::string(e.first), std::string(e.second));
    }
  }
  int64_t deviceId() const override { return wideDevice ? kWideDeviceId : a->device; }
  static constexpr int64_t kWideDeviceId = int64_t{1} << 40;
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
    std::vector<std::string> keep;  // MetadataField holds a string_view
    keep.reserve(a->n_fields);
    uint32_t f = 0;
    const uint64_t* slot = a->slots;
    visitFields(visitor, f, slot, keep);
  }
  // Visits fields from index f on; returns after the KTJ_F_DICT_END that closes the dict this
  // call was made for (or at the end of the fields).
  void visitFields(ITypedMetadataVisitor& visitor, uint32_t& f, const uint64_t*& slot, std::vector<std::string>& keep) const {
    while (f < a->n_fields) {
      const ktj_field& fd = a->fields[f++];
      keep.push_back(fd.key_id == KTJ_NONE ? std::string() : st->get(fd.key_id));
      const std::string& key = keep.back();
      const uint64_t* v = slot;
      slot += fd.count;
      switch (fd.type) {
        case KTJ_F_I64:
          visitor.visit(MetadataField<int64_t>{key}, static_cast<int64_t>(v[0]));
          break;
        case KTJ_F_U64:
          visitor.visit(MetadataField<uint64_t>{key}, static_cast<uint64_t>(v[0]));
          break;
        case KTJ_F_F64: {
          double d;
          std::memcpy(&d, &v[0], 8);
          visitor.visit(MetadataField<double>{key}, d);
          break;
        }
        case KTJ_F_BOOL:
          visitor.visit(MetadataField<bool>{key}, v[0] != 0);
          break;
        case KTJ_F_STR:
          visitor.visit(MetadataField<std::string>{key}, st->get(static_cast<uint32_t>(v[0])));
          break;
        case KTJ_F_RAW:
          visitor.visit(MetadataField<RawJson>{key}, RawJson{st->get(static_cast<uint32_t>(v[0]))});
          break;
        case KTJ_F_I64_ARRAY: {
          std::vector<int64_t> arr(fd.count);
          for (uint32_t k = 0; k < fd.count; ++k) arr[k] = static_cast<int64_t>(v[k]);
          visitor.visit(MetadataField<std::vector<int64_t>>{key}, arr);
          break;
        }
        case KTJ_F_STR_ARRAY: {
          std::vector<std::string> arr;
          for (uint32_t k = 0; k < fd.count; ++k) arr.push_back(st->get(static_cast<uint32_t>(v[k])));
          visitor.visit(MetadataField<std::vector<std::string>>{key}, arr);
          break;
        }
        case KTJ_F_DICT_BEGIN:
          visitor.visit(MetadataDict{key}, [&](ITypedMetadataVisitor& d) { visitFields(d, f, slot, keep); });
          break;
        case KTJ_F_DICT_END:
          return;
        case KTJ_F_UNSUPPORTED:  // a field type the visitor has no overload for
          visitor.visit(MetadataField<std::pair<int64_t, int64_t>>{key}, std::pair<int64_t, int64_t>{1, 2});
          break;
        case KTJ_F_SHAPES: {  // the checker hands the encoding over inline (see include/ktj.h)
          InputShapes shapes;
          const uint64_t* q = v;
          const uint64_t* end = v + fd.count;
          const uint64_t entries = q < end ? *q++ : 0;
          auto shape = [&](uint64_t rank) {
            std::vector<int64_t> dims;
            for (uint64_t k = 0; k < rank; ++k) { dims.push_back(q < end ? static_cast<int64_t>(*q) : 0); if (q < end) ++q; }
            return dims;
          };
          for (uint64_t e = 0; e < entries && q < end; ++e) {
            const uint64_t head = *q++, m = head & 0xFFFFFFFFull;
            if (head & KTJ_SHAPE_LIST) {
              TensorListShapes list;
              for (uint64_t t = 0; t < m && q < end; ++t) { const uint64_t rank = *q++ & 0xFFFFFFFFull; list.push_back(shape(rank)); }
              shapes.emplace_back(std::move(list));
            } else shapes.emplace_back(shape(m));
          }
          visitor.visit(MetadataField<InputShapes>{key}, shapes);
          break;
        }
        default:
          break;
      }
    }
  }
  // The keyed double fields are the activity's counter values (read for counter kinds only).
  mutable std::vector<std::pair<std::string, double>> counters;
  mutable bool countersBuilt = false;
  const std::vector<std::pair<std::string, double>>& counterValues() const override {
    if (!countersBuilt) {
      countersBuilt = true;
      const uint64_t* slot = a->slots;
      for (uint32_t f = 0; f < a->n_fields; slot += a->fields[f].count, ++f) {
        const ktj_field& fd = a->fields[f];
        if (fd.type != KTJ_F_F64 || fd.key_id == KTJ_NONE) continue;
        double d;
        std::memcpy(&d, &slot[0], 8);
        counters.emplace_back(st->get(fd.key_id), d);
      }
    }
    return counters;
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

// The same activity as a GenericTraceActivity (what a buffering logger's replay loop mostly holds):
// every accessor forwards to the MatActivity.
struct GenericMatActivity : public GenericTraceActivity {
  const MatActivity* m;
  explicit GenericMatActivity(const MatActivity* mat) : m(mat) {}
  int64_t deviceId() const override { return m->deviceId(); }
  int64_t resourceId() const override { return m->resourceId(); }
  int32_t getThreadId() const override { return m->getThreadId(); }
  int64_t timestamp() const override { return m->timestamp(); }
  int64_t duration() const override { return m->duration(); }
  int64_t correlationId() const override { return m->correlationId(); }
  int flowType() const override { return m->flowType(); }
  int64_t flowId() const override { return m->flowId(); }
  bool flowStart() const override { return m->flowStart(); }
  ActivityType type() const override { return m->type(); }
  const std::string name() const override { return m->name(); }
  const ITraceActivity* linkedActivity() const override { return m->linkedActivity(); }
  const TraceSpan* traceSpan() const override { return nullptr; }
  void log(ActivityLogger& logger) const override { logger.handleActivity(*this); }
  const std::string metadataJson() const override { return m->metadataJson(); }
  const std::vector<std::pair<std::string, double>>& counterValues() const override { return m->counterValues(); }
};

// Replays one stream into a logger in the order of the reference's buffering logger
// (src/output_membuf.h:91-107): trace start, device / resource / overhead infos, the activities
// stable-sorted by (deviceId, resourceId, timestamp), spans, finalizeTrace(endTime).  L must
// expose finalizeTrace(int64_t).  `log_all` hands a list of activities to the logger; the default
// is the replay loop of src/output_membuf.h:101-103, one log() call each.
//
// call_order 0: the order of the buffering logger's replay (src/output_membuf.h:91-107): trace
//   start, device infos, resource infos, (overhead infos,) the activities stable-sorted by
//   (deviceId, resourceId, timestamp), the spans, finalizeTrace.
// call_order 1: the order in which GenericActivityProfiler drives a logger directly
//   (src/GenericActivityProfiler.cpp:178-224 processTraceInternal, :655-740 finalizeTrace): trace
//   start, the activities, the CPU buffer's span, resource infos, device infos, the GPU spans,
//   overhead infos, finalizeTrace — with the activity segment sorted as above, so that it is what
//   a logger that keeps its activities in one sorted section must write.
// call_order 2: the same calls as 1 but with the activities where the profiler issues them and in
//   arrival order: CPU-side activities, the CPU buffer's span, then the GPU-side activities and the
//   rest.  Only a logger that sorts by itself writes the file of call_order 1 from it.
template <class L, class LogAll>
void replay_stream(L& logger, const ktj_stream* s, const ktj_mat_activity* acts, uint64_t n_acts, string_fn fn,
                   const void* ctx, LogAll log_all, int call_order = 0, int wide_device_mod = 0) {
  StringTable st{fn, ctx};
  std::vector<MatActivity> wrapped;
  wrapped.reserve(n_acts);
  for (uint64_t i = 0; i < n_acts; ++i) {
    wrapped.emplace_back(&acts[i], &st, s->collectives);
    wrapped.back().wideDevice = wide_device_mod > 0 && acts[i].arrival % static_cast<uint64_t>(wide_device_mod) == 1;
  }
  std::vector<const MatActivity*> order(n_acts);
  for (uint64_t i = 0; i < n_acts; ++i) order[i] = &wrapped[i];
  if (call_order != 2)
    std::stable_sort(order.begin(), order.end(), [](const MatActivity* x, const MatActivity* y) {
      return std::make_tuple(x->deviceId(), x->resourceId(), x->timestamp()) <
          std::make_tuple(y->deviceId(), y->resourceId(), y->timestamp());
    });
  auto device_infos = [&] {
    for (uint64_t i = 0; i < s->n_device_infos; ++i) {
      const ktj_device_info& d = s->device_infos[i];
      logger.handleDeviceInfo({d.id, d.sort_index, d.name, d.label}, d.time_ns);
    }
  };
  auto resource_infos = [&] {
    for (uint64_t i = 0; i < s->n_resource_infos; ++i) {
      const ktj_resource_info& r = s->resource_infos[i];
      logger.handleResourceInfo(
          {r.id, r.sort_index, r.device_id, r.name, r.host_thread ? ResourceType::HOST_THREAD : ResourceType::UNKNOWN},
          r.time_ns);
    }
  };
  auto overhead_infos = [&] {
    for (uint64_t i = 0; i < s->n_overhead_infos; ++i)
      logger.handleOverheadInfo(ActivityLogger::OverheadInfo(s->overhead_infos[i].name), s->overhead_infos[i].time_ns);
  };
  auto spans = [&](uint64_t from, uint64_t to) {
    for (uint64_t i = from; i < to && i < s->n_spans; ++i) {
      const ktj_trace_span& sp = s->spans[i];
      TraceSpan span(sp.op_count, sp.iteration, sp.name, sp.prefix);
      span.startTime = sp.start_ns;
      span.endTime = sp.end_ns;
      logger.handleTraceSpan(span);
    }
  };

  std::unordered_map<std::string, std::string> metadata;  // env metadata (host_name) is added by the logger
  logger.handleTraceStart(metadata, s->device_properties ? s->device_properties : "");
  if (call_order == 0) {
    device_infos();
    resource_infos();
    overhead_infos();
    log_all(logger, order);
    spans(0, s->n_spans);
  } else {
    if (call_order == 1) {
      log_all(logger, order);
      spans(0, 1);
    } else { /* CPU-side activities (processCpuTrace), their span, then everything else (processGpuActivities) */
      std::vector<const MatActivity*> cpu_side, gpu_side;
      for (const MatActivity* a : order) {
        const ActivityType t = a->type();
        (t == ActivityType::CPU_OP || t == ActivityType::USER_ANNOTATION || t == ActivityType::CPU_INSTANT_EVENT ||
                 t == ActivityType::PYTHON_FUNCTION
             ? cpu_side : gpu_side).push_back(a);
      }
      if (cpu_side.empty() && !gpu_side.empty()) { cpu_side.push_back(gpu_side.front()); gpu_side.erase(gpu_side.begin()); }
      log_all(logger, cpu_side);
      spans(0, 1);
      log_all(logger, gpu_side);
    }
    resource_infos();
    device_infos();
    spans(1, s->n_spans);
    overhead_infos();
  }
  logger.finalizeTrace(s->end_time_ns);
}

template <class L>
void replay_stream(L& logger, const ktj_stream* s, const ktj_mat_activity* acts, uint64_t n_acts, string_fn fn,
                   const void* ctx, int call_order = 0, int wide_device_mod = 0) {
  replay_stream(logger, s, acts, n_acts, fn, ctx, [](L& l, const std::vector<const MatActivity*>& order) {
    for (const MatActivity* a : order) a->log(l);
  }, call_order, wide_device_mod);
}

}  // namespace ktj_ref_driver
