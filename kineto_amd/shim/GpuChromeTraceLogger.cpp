/*
 * GpuChromeTraceLogger.cpp — see GpuChromeTraceLogger.h.
 *
 * Per-record work on the host is limited to reading the activity's accessors once, interning
 * its name in a string dictionary, appending its metadataJson() text to a blob, and appending one
 * 64-byte packed record; sorting, sizing and all formatting happen on the GPU in ktj_finalize.
 */
#include "GpuChromeTraceLogger.h"

#include <algorithm>
#include <cstring>
#include <limits>
#include <thread>

#include "EnvMetadata.h"
#include "GenericTraceActivity.h"
#include "ITraceActivity.h"
#include "Logger.h"
#include "TraceSpan.h"
#include "output_json.h" /* ChromeTraceBaseTime */

using namespace libkineto;

namespace ktj_shim {

namespace {
constexpr size_t kRecordBatch = 1u << 16;       /* records per ktj_submit_records call */
constexpr size_t kStringBatchBytes = 16u << 20; /* dictionary bytes per ktj_intern_strings call */
constexpr const char* kParamCommsName = "record_param_comms"; /* output_json.cpp: kParamCommsCallName */
}  // namespace

/* ---- packing: activity -> 64-byte record, with ids local to the packer ---- */

namespace {
const char* const kCollectiveKeys[] = {"Collective name", "In msg nelems", "Out msg nelems", "Group size", "dtype",
                                       "Input Tensors start", "Output Tensors start", "In split size", "Out split size",
                                       "Process Group Name", "Process Group Description", "Process Group Ranks",
                                       "Dst Rank", "Src Rank", "Seq", "Comms Id", "Rank"};
constexpr size_t kCollectiveKeyCount = sizeof(kCollectiveKeys) / sizeof(kCollectiveKeys[0]);
static_assert(kCollectiveKeyCount * sizeof(const char*) == sizeof(ktj_collective_meta), "one key per field of ktj_collective_meta");

/* schema codes inside a Packed (KTJ_NONE = no metadata) */
constexpr uint32_t kLocalFragment = 0, kLocalCollective = 1, kLocalCollectiveFragment = 2, kLocalCounterBase = 3;
/* what a slot holds, for the translation to engine ids */
constexpr uint8_t kSlotPlain = 0, kSlotFragment = 1, kSlotCollective = 2;
}  // namespace

/* The output of one packer: records whose string ids, schema ids, collective indices and slot
 * offsets are local to it, plus the local dictionaries.  A packer touches no logger state, so
 * several can run at once on disjoint activities; merge() translates to engine ids. */
struct GpuChromeTraceLogger::Packed {
  std::vector<ktj_generic_rec> records;
  std::vector<uint64_t> origin;    /* position of each record in the caller's sequence */
  std::vector<uint64_t> slots;
  std::vector<uint8_t> slotKind;
  std::vector<std::string> names; /* activity and counter names: few distinct ones, kept once */
  std::unordered_map<std::string, uint32_t> nameIndex;
  std::string fragmentBlob;       /* metadataJson() texts: nearly all distinct (sequence numbers, */
  std::vector<uint64_t> fragmentOff{0}; /* correlation ids), so they are stored as they come; n + 1 offsets */
  std::vector<std::string> collectives; /* the 17 values of an op, each followed by NUL */
  std::unordered_map<std::string, uint32_t> collectiveIndex;
  std::vector<std::vector<uint32_t>> counterSchemas; /* local ids of the counter names */
  std::unordered_map<std::string, uint32_t> counterIndex;
  /* engine ids of the local entries translated so far (merge) */
  std::vector<uint32_t> nameGlobal, collectiveGlobal, counterGlobal;
  uint32_t fragmentBase = 0; /* engine id of local fragment 0 */

  uint32_t name(const std::string& s) {
    auto it = nameIndex.find(s);
    if (it != nameIndex.end()) return it->second;
    const uint32_t id = static_cast<uint32_t>(names.size());
    nameIndex.emplace(s, id);
    names.push_back(s);
    return id;
  }
  uint32_t fragment(const std::string& s) {
    fragmentBlob.append(s);
    fragmentOff.push_back(fragmentBlob.size());
    return static_cast<uint32_t>(fragmentOff.size() - 2);
  }
  void slot(uint64_t v, uint8_t kind) { slots.push_back(v); slotKind.push_back(kind); }
  void clearRecords() {
    records.clear(); origin.clear(); slots.clear(); slotKind.clear(); fragmentBlob.clear(); fragmentOff.assign(1, 0);
  }
};

GpuChromeTraceLogger::GpuChromeTraceLogger(const std::string& traceFileName, int hipDevice)
    : fileName_(traceFileName), staging_(new Packed) {
  /* the engine applies the default-file-name rule (output_json.cpp:481-483) for an empty name */
  uint32_t flags = KTJ_CREATE_NO_STAGE_TIMES; /* a logger reports no stage times */
#ifdef DISPLAY_TRACE_IN_NS /* the reference's compile-time switch (output_json.cpp:451-454) */
  flags |= KTJ_CREATE_DISPLAY_NS;
#endif
  const int rc = ktj_create(&engine_, traceFileName.c_str(), ChromeTraceBaseTime::singleton().get(), hipDevice, flags);
  if (rc != KTJ_OK) {
    LOG(ERROR) << "GPU trace engine unavailable (ktj_create rc=" << rc << "): "
               << (engine_ ? ktj_last_error(engine_) : "no engine");
    if (engine_) ktj_destroy(engine_);
    engine_ = nullptr;
    status_ = rc;
    return;
  }
  const ktj_field fragment = {KTJ_NONE, KTJ_F_RAW, 1}; /* one slot: string id of a whole args fragment */
  note(ktj_register_schema(engine_, &fragment, 1, &fragmentSchema_), "ktj_register_schema");
  const ktj_field withCollective[2] = {{KTJ_NONE, KTJ_F_COLLECTIVE, 1}, fragment};
  note(ktj_register_schema(engine_, withCollective, 1, &collectiveSchema_), "ktj_register_schema");
  note(ktj_register_schema(engine_, withCollective, 2, &collectiveFragmentSchema_), "ktj_register_schema");
  pendingOffsets_.push_back(0);
}

GpuChromeTraceLogger::~GpuChromeTraceLogger() {
  if (engine_) ktj_destroy(engine_);
}

void GpuChromeTraceLogger::note(int rc, const char* what) {
  if (rc == KTJ_OK || status_ != 0) return;
  status_ = rc;
  LOG(ERROR) << what << " failed (rc=" << rc << "): " << (engine_ ? ktj_last_error(engine_) : "");
}

/* ---- packing: one activity -> one record in a Packed ---- */

/* Reads the activity's accessors once and appends one record (what ChromeTraceLogger::handleActivity
 * reads, output_json.cpp:837-963). */
void GpuChromeTraceLogger::pack(const ITraceActivity& op, uint64_t origin, Packed& out) {
  const ActivityType type = op.type();
  const std::string name = op.name();
  const ITraceActivity* linked = op.linkedActivity();
  const int64_t device = op.deviceId();
  const bool counter = type == ActivityType::HARDWARE_COUNTERS || type == ActivityType::MTIA_COUNTERS ||
      type == ActivityType::XPU_SCOPE_PROFILER; /* output_json.cpp:847-856 */
  /* collective metadata comes from a linked record_param_comms op (output_json.cpp:899-908) */
  const bool collective = !counter && linked != nullptr &&
      (type == ActivityType::CONCURRENT_KERNEL || (type == ActivityType::MTIA_CCP_EVENTS && name.rfind("hccl::", 0) == 0)) &&
      linked->name() == kParamCommsName;
  const bool wideDevice = device < std::numeric_limits<int32_t>::min() || device > std::numeric_limits<int32_t>::max();
  ktj_generic_rec r{};
  r.start_ns = op.timestamp();
  r.end_ns = r.start_ns + op.duration();
  r.resource = op.resourceId();
  r.device = wideDevice ? 0 : static_cast<int32_t>(device);
  r.id = static_cast<int32_t>(op.correlationId()); /* `int external_id = op.correlationId()`, :893 */
  r.type = static_cast<uint8_t>(type);
  r.name_id = out.name(name);
  r.flow_id = op.flowId();
  const int flowType = op.flowType(); /* anything but the two known kinds prints no flow event (:979-994) */
  r.flow_type = (flowType == static_cast<int>(KTJ_LINK_FWDBWD) || flowType == static_cast<int>(KTJ_LINK_ASYNC_CPU_GPU)) ? static_cast<uint8_t>(flowType) : 0;
  r.flags = op.flowStart() ? KTJ_GF_FLOW_START : 0;
  if (linked != nullptr) {
    r.flags |= KTJ_GF_LINKED;
    r.linked_id = static_cast<int32_t>(linked->correlationId()); /* `int external_id = …`, :873 */
  }
  r.schema_id = KTJ_NONE;
  if (wideDevice) { /* the record's device field is 32 bits: the value goes into the slot before the record's values */
    r.flags |= KTJ_GF_WIDE_DEVICE;
    out.slot(static_cast<uint64_t>(device), kSlotPlain);
  }
  r.args_off = out.slots.size();
  if (counter) { /* handleCounterEvent (:679-716) prints counterValues() and nothing else */
    const auto& values = op.counterValues();
    if (!values.empty()) { /* one schema per distinct list of counter names: a keyed double field for each */
      std::vector<uint32_t> names;
      names.reserve(values.size());
      for (const auto& kv : values) names.push_back(out.name(kv.first));
      const std::string key(reinterpret_cast<const char*>(names.data()), names.size() * sizeof(uint32_t));
      auto it = out.counterIndex.find(key);
      if (it == out.counterIndex.end()) {
        it = out.counterIndex.emplace(key, static_cast<uint32_t>(out.counterSchemas.size())).first;
        out.counterSchemas.push_back(std::move(names));
      }
      r.schema_id = kLocalCounterBase + it->second;
      for (const auto& kv : values) {
        uint64_t bits;
        static_assert(sizeof(bits) == sizeof(kv.second), "double is 64 bits");
        std::memcpy(&bits, &kv.second, sizeof(bits));
        out.slot(bits, kSlotPlain);
      }
    }
  } else {
    const std::string metadata = op.metadataJson();
    if (collective) { /* the first slot names the linked op's collective metadata */
      std::string key;
      for (size_t i = 0; i < kCollectiveKeyCount; ++i) {
        key += linked->getMetadataValue(kCollectiveKeys[i]);
        key += '\0';
      }
      auto it = out.collectiveIndex.find(key);
      if (it == out.collectiveIndex.end()) {
        it = out.collectiveIndex.emplace(key, static_cast<uint32_t>(out.collectives.size())).first;
        out.collectives.push_back(key);
      }
      r.schema_id = metadata.empty() ? kLocalCollective : kLocalCollectiveFragment;
      out.slot(it->second, kSlotCollective);
    } else if (!metadata.empty()) {
      r.schema_id = kLocalFragment;
    }
    if (!metadata.empty()) out.slot(out.fragment(metadata), kSlotFragment);
  }
  out.records.push_back(r);
  out.origin.push_back(origin);
}

/* ---- merging: local ids -> engine ids ---- */

uint32_t GpuChromeTraceLogger::intern(const std::string& s) {
  auto it = strings_.find(s);
  if (it != strings_.end()) return it->second;
  const uint32_t id = nextStringId_++;
  strings_.emplace(s, id);
  pendingBlob_.append(s);
  pendingOffsets_.push_back(pendingBlob_.size());
  if (pendingBlob_.size() >= kStringBatchBytes) flushStrings();
  return id;
}

/* Brings the packer's dictionaries up to date with the engine's: every local string, collective
 * entry and counter schema that has no engine id yet gets one. */
void GpuChromeTraceLogger::translate(Packed& p) {
  for (size_t i = p.nameGlobal.size(); i < p.names.size(); ++i) p.nameGlobal.push_back(intern(p.names[i]));
  /* the fragments of this batch get consecutive ids */
  const size_t nFragments = p.fragmentOff.size() - 1;
  if (nFragments != 0 && p.fragmentBlob.size() >= kStringBatchBytes) {
    /* a batch of its own: handed to the engine where it lies, after whatever is pending */
    flushStrings();
    p.fragmentBase = nextStringId_;
    uint32_t first = 0;
    if (ok()) {
      note(ktj_intern_strings(engine_, p.fragmentBlob.data(), p.fragmentOff.data(), nFragments, &first), "ktj_intern_strings");
      if (status_ == 0 && first != p.fragmentBase) note(KTJ_ERR_STATE, "string id bookkeeping");
    }
    nextStringId_ += static_cast<uint32_t>(nFragments);
    pendingFirstId_ = nextStringId_;
  } else {
    p.fragmentBase = nextStringId_;
    if (nFragments != 0) {
      const uint64_t at = pendingBlob_.size();
      pendingBlob_.append(p.fragmentBlob);
      pendingOffsets_.reserve(pendingOffsets_.size() + nFragments);
      for (size_t i = 1; i <= nFragments; ++i) pendingOffsets_.push_back(at + p.fragmentOff[i]);
      nextStringId_ += static_cast<uint32_t>(nFragments);
      if (pendingBlob_.size() >= kStringBatchBytes) flushStrings();
    }
  }
  for (size_t i = p.collectiveGlobal.size(); i < p.collectives.size(); ++i) {
    const std::string& key = p.collectives[i];
    auto it = collectives_.find(key);
    if (it == collectives_.end()) {
      /* the values ChromeTraceLogger::appendCollectiveMetadata reads (output_json.cpp:718-835), handed
       * to the engine once per distinct set */
      const char* v[kCollectiveKeyCount];
      const char* q = key.c_str();
      for (size_t k = 0; k < kCollectiveKeyCount; ++k) { v[k] = q; q += std::strlen(q) + 1; }
      const ktj_collective_meta meta = {v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8],
                                        v[9], v[10], v[11], v[12], v[13], v[14], v[15], v[16]}; /* kCollectiveKeys order */
      uint32_t index = 0;
      note(ktj_add_collective(engine_, &meta, &index), "ktj_add_collective");
      it = collectives_.emplace(key, index).first;
    }
    p.collectiveGlobal.push_back(it->second);
  }
  for (size_t i = p.counterGlobal.size(); i < p.counterSchemas.size(); ++i) {
    std::vector<ktj_field> fields;
    fields.reserve(p.counterSchemas[i].size());
    for (uint32_t local : p.counterSchemas[i]) fields.push_back(ktj_field{p.nameGlobal[local], KTJ_F_F64, 1});
    const std::string key(reinterpret_cast<const char*>(fields.data()), fields.size() * sizeof(ktj_field));
    auto it = counterSchemas_.find(key);
    if (it == counterSchemas_.end()) {
      uint32_t sid = KTJ_NONE;
      note(ktj_register_schema(engine_, fields.data(), fields.size(), &sid), "ktj_register_schema");
      it = counterSchemas_.emplace(key, sid).first;
    }
    p.counterGlobal.push_back(it->second);
  }
}

/* Appends the packer's slots to the pending args and returns where they start. */
uint64_t GpuChromeTraceLogger::appendSlots(const Packed& p) {
  const uint64_t base = nextSlot_;
  slots_.reserve(slots_.size() + p.slots.size());
  for (size_t i = 0; i < p.slots.size(); ++i) {
    const uint64_t v = p.slots[i];
    slots_.push_back(p.slotKind[i] == kSlotFragment ? p.fragmentBase + v : p.slotKind[i] == kSlotCollective ? p.collectiveGlobal[v] : v);
  }
  nextSlot_ += p.slots.size();
  return base;
}

ktj_generic_rec GpuChromeTraceLogger::translated(const Packed& p, size_t i, uint64_t slotBase) const {
  ktj_generic_rec r = p.records[i];
  r.name_id = p.nameGlobal[r.name_id];
  r.args_off += slotBase;
  if (r.schema_id == kLocalFragment) r.schema_id = fragmentSchema_;
  else if (r.schema_id == kLocalCollective) r.schema_id = collectiveSchema_;
  else if (r.schema_id == kLocalCollectiveFragment) r.schema_id = collectiveFragmentSchema_;
  else if (r.schema_id != KTJ_NONE) r.schema_id = p.counterGlobal[r.schema_id - kLocalCounterBase];
  return r;
}

/* One packer whose records are already in arrival order. */
void GpuChromeTraceLogger::mergeInOrder(Packed& p) {
  translate(p);
  const uint64_t base = appendSlots(p);
  records_.reserve(records_.size() + p.records.size());
  for (size_t i = 0; i < p.records.size(); ++i) records_.push_back(translated(p, i, base));
  p.clearRecords();
  flushStrings();
  flushRecords();
}

void GpuChromeTraceLogger::flushStrings() {
  const size_t n = pendingOffsets_.size() - 1;
  if (n == 0 || !ok()) return;
  uint32_t first = 0;
  note(ktj_intern_strings(engine_, pendingBlob_.data(), pendingOffsets_.data(), n, &first), "ktj_intern_strings");
  if (status_ == 0 && first != pendingFirstId_) note(KTJ_ERR_STATE, "string id bookkeeping");
  pendingFirstId_ = nextStringId_;
  pendingBlob_.clear();
  pendingOffsets_.assign(1, 0);
}

void GpuChromeTraceLogger::flushRecords() {
  submitRecords(records_.data(), records_.size());
  records_.clear();
}

/* the pending args slots, then the records that refer to them */
void GpuChromeTraceLogger::submitRecords(const ktj_generic_rec* records, size_t count) {
  if (count != 0 && ok()) {
    uint64_t first = 0;
    note(ktj_submit_args(engine_, slots_.data(), slots_.size(), &first), "ktj_submit_args");
    if (status_ == 0 && first + slots_.size() != nextSlot_) note(KTJ_ERR_STATE, "args slot bookkeeping");
    note(ktj_submit_records(engine_, KTJ_REC_GENERIC, records, count), "ktj_submit_records");
  }
  slots_.clear(); /* slots only ever come with records */
}

void GpuChromeTraceLogger::handleTraceStart(const std::unordered_map<std::string, std::string>& metadata,
                                            const std::string& device_properties) {
  if (!ok()) return;
  /* ChromeTraceLogger::addEnvVarsToMetadata (output_json.cpp:433-443): environment first, the
   * caller's entries override; the header lists them in this map's iteration order */
  auto combined = libkineto::getEnvMetadata();
  for (const auto& [k, v] : metadata) combined[k] = v;
  std::vector<const char*> kv;
  kv.reserve(combined.size() * 2);
  for (const auto& [k, v] : combined) {
    kv.push_back(k.c_str());
    kv.push_back(v.c_str());
  }
  note(ktj_trace_start(engine_, kv.data(), combined.size(), device_properties.c_str()), "ktj_trace_start");
}

void GpuChromeTraceLogger::handleDeviceInfo(const DeviceInfo& info, int64_t time) {
  if (!ok()) return;
  const ktj_device_info d = {info.id, info.sortIndex, info.name.c_str(), info.label.c_str(), time};
  note(ktj_submit_info(engine_, KTJ_INFO_DEVICE, &d), "ktj_submit_info(device)");
}

void GpuChromeTraceLogger::handleResourceInfo(const ResourceInfo& info, int64_t time) {
  if (!ok()) return;
  const ktj_resource_info r = {info.id, info.sortIndex, info.deviceId, info.name.c_str(),
                               info.resourceType == ResourceType::HOST_THREAD ? 1 : 0, 0, time};
  note(ktj_submit_info(engine_, KTJ_INFO_RESOURCE, &r), "ktj_submit_info(resource)");
}

void GpuChromeTraceLogger::handleOverheadInfo(const OverheadInfo& info, int64_t time) {
  if (!ok()) return;
  const ktj_overhead_info o = {info.name.c_str(), time};
  note(ktj_submit_info(engine_, KTJ_INFO_OVERHEAD, &o), "ktj_submit_info(overhead)");
}

void GpuChromeTraceLogger::handleTraceSpan(const TraceSpan& span) {
  if (!ok()) return;
  const ktj_trace_span s = {span.startTime, span.endTime, span.opCount, span.iteration, span.name.c_str(),
                            span.prefix.c_str()};
  note(ktj_submit_info(engine_, KTJ_INFO_SPAN, &s), "ktj_submit_info(span)");
}

/* The records are batched and reach the engine later; the engine is told now that the activities
 * have begun, so that infos and spans that follow go behind the activity section, as they do in
 * the reference logger's file when it is driven by GenericActivityProfiler::processTraceInternal. */
void GpuChromeTraceLogger::noteFirstActivity() {
  if (activitiesBegun_) return;
  activitiesBegun_ = true;
  note(ktj_begin_activities(engine_), "ktj_begin_activities");
}

void GpuChromeTraceLogger::handleActivity(const ITraceActivity& op) {
  if (!ok()) return;
  noteFirstActivity();
  pack(op, 0, *staging_);
  if (staging_->records.size() >= kRecordBatch) mergeInOrder(*staging_);
}

/* The replay loop of a buffering logger (MemoryTraceLogger::log, libkineto/src/output_membuf.h:91-107:
 * `for (auto& activity : activities_) activity->log(logger)`) as one call.  The host gather runs
 * on `threads` workers: each packs the GenericTraceActivity objects of one contiguous slice.  Every
 * other kind of activity is packed by the calling thread, in order: the ROCm wrappers hand grid,
 * block and size from the runtime row to the device row through thread_local maps inside
 * metadataJson() (libkineto/src/RocprofActivity_inl.h:28-30, 163-180, 221-232), so they must stay on
 * one thread and in sequence.  The records reach the engine in the order of `activities`. */
void GpuChromeTraceLogger::handleActivities(const std::vector<const ITraceActivity*>& activities, unsigned threads) {
  if (!ok() || activities.empty()) return;
  noteFirstActivity();
  mergeInOrder(*staging_); /* what single calls left behind comes first */
  const size_t n = activities.size();
  if (threads == 0) threads = std::max(1u, std::thread::hardware_concurrency());
  threads = static_cast<unsigned>(std::min<size_t>(threads, (n + 4095) / 4096));
  std::vector<Packed> parts(threads + 1); /* parts[threads]: the calling thread's, everything that is not generic */
  auto run = [threads](auto&& job) { /* job(w) for every w < threads, w = 0 on the calling thread */
    std::vector<std::thread> pool;
    for (unsigned w = 1; w < threads; ++w) pool.emplace_back(job, w);
    job(0u);
    for (auto& t : pool) t.join();
  };
  auto is_generic = [](const ITraceActivity* a) { return dynamic_cast<const GenericTraceActivity*>(a) != nullptr; };
  {
    std::vector<std::thread> pool;
    for (unsigned w = 0; w < threads; ++w)
      pool.emplace_back([&, w] {
        const size_t lo = n * w / threads, hi = n * (w + 1) / threads;
        for (size_t i = lo; i < hi; ++i)
          if (is_generic(activities[i])) pack(*activities[i], i, parts[w]);
      });
    for (size_t i = 0; i < n; ++i) /* meanwhile, here and in order: everything else */
      if (!is_generic(activities[i])) pack(*activities[i], i, parts[threads]);
    for (auto& t : pool) t.join();
  }

  /* merge.  In sequence: the local dictionaries become engine ids and every part learns where its
   * slots go.  Then, part by part on the workers: slots and records move to their final places
   * (a record's place is its activity's position). */
  std::vector<uint64_t> base(parts.size());
  size_t nRecords = 0, nSlots = 0;
  for (size_t w = 0; w < parts.size(); ++w) {
    translate(parts[w]);
    base[w] = nextSlot_ + nSlots;
    nSlots += parts[w].slots.size();
    nRecords += parts[w].records.size();
  }
  if (nRecords != n) { note(KTJ_ERR_STATE, "record bookkeeping"); return; } /* every activity packs into one record */
  const size_t slot0 = slots_.size();
  slots_.resize(slot0 + nSlots);
  std::unique_ptr<ktj_generic_rec[]> placed(new ktj_generic_rec[n]); /* not zero-filled: every place is written */
  const unsigned nParts = static_cast<unsigned>(parts.size());
  const uint64_t firstSlot = nextSlot_;
  run([&](unsigned w0) {
    for (unsigned w = w0; w < nParts; w += threads) {
      const Packed& p = parts[w];
      uint64_t* out = slots_.data() + slot0 + (base[w] - firstSlot);
      for (size_t i = 0; i < p.slots.size(); ++i) {
        const uint64_t v = p.slots[i];
        out[i] = p.slotKind[i] == kSlotFragment ? p.fragmentBase + v : p.slotKind[i] == kSlotCollective ? p.collectiveGlobal[v] : v;
      }
      for (size_t j = 0; j < p.records.size(); ++j) placed[p.origin[j]] = translated(p, j, base[w]);
    }
  });
  nextSlot_ += nSlots;
  flushStrings();
  submitRecords(placed.get(), n); /* records_ is empty here: mergeInOrder above flushed it */
}

void GpuChromeTraceLogger::handleGenericActivity(const GenericTraceActivity& op) {
  handleActivity(op); /* output_json.cpp:965-971 */
}

void GpuChromeTraceLogger::finalizeMemoryTrace(const std::string&, const Config&) {
  LOG(INFO) << "finalizeMemoryTrace not implemented for GpuChromeTraceLogger";
}

void GpuChromeTraceLogger::finalizeTrace(const Config&, std::unique_ptr<ActivityBuffers> /*buffers*/, int64_t endTime) {
  /* everything the engine needs was copied in handleActivity; the buffers are not kept */
  finalizeTrace(endTime);
}

void GpuChromeTraceLogger::finalizeTrace(int64_t endTime) {
  if (!ok()) {
    LOG(ERROR) << "Failed to write to log file!";
    return;
  }
  mergeInOrder(*staging_);
  uint64_t written = 0;
  if (status_ == 0) note(ktj_finalize(engine_, endTime, &written), "ktj_finalize");
  if (status_ != 0) {
    LOG(ERROR) << "Failed to write to log file!";
    return;
  }
  LOG(INFO) << "Chrome Trace written to " << fileName_ << " (" << written << " bytes)";
}

}  // namespace ktj_shim
