/*
 * GpuChromeTraceLogger.cpp — see GpuChromeTraceLogger.h.
 *
 * Per-record work on the host is limited to reading the activity's accessors once, interning
 * its name and its metadataJson() text in a string dictionary, and appending one 64-byte packed
 * record; sorting, sizing and all formatting happen on the GPU in ktj_finalize.
 */
#include "GpuChromeTraceLogger.h"

#include <cstring>
#include <limits>

#include "EnvMetadata.h"
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

GpuChromeTraceLogger::GpuChromeTraceLogger(const std::string& traceFileName, int hipDevice) : fileName_(traceFileName) {
  /* the engine applies the default-file-name rule (output_json.cpp:481-483) for an empty name */
  const int rc = ktj_create(&engine_, traceFileName.c_str(), ChromeTraceBaseTime::singleton().get(), hipDevice, 0);
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

uint32_t GpuChromeTraceLogger::intern(std::unordered_map<std::string, uint32_t>& index, const std::string& s) {
  auto it = index.find(s);
  if (it != index.end()) return it->second;
  const uint32_t id = nextStringId_++;
  index.emplace(s, id);
  pendingBlob_.append(s);
  pendingOffsets_.push_back(pendingBlob_.size());
  if (pendingBlob_.size() >= kStringBatchBytes) flushStrings();
  return id;
}

/* The values ChromeTraceLogger::appendCollectiveMetadata reads from a record_param_comms op
 * (output_json.cpp:718-835), handed to the engine once per distinct set of values. */
uint32_t GpuChromeTraceLogger::collectiveIndex(const ITraceActivity& op) {
  static const char* const kKeys[] = {"Collective name", "In msg nelems", "Out msg nelems", "Group size", "dtype",
                                      "Input Tensors start", "Output Tensors start", "In split size", "Out split size",
                                      "Process Group Name", "Process Group Description", "Process Group Ranks",
                                      "Dst Rank", "Src Rank", "Seq", "Comms Id", "Rank"};
  constexpr size_t kCount = sizeof(kKeys) / sizeof(kKeys[0]);
  static_assert(kCount * sizeof(const char*) == sizeof(ktj_collective_meta), "one key per field of ktj_collective_meta");
  std::string values[kCount];
  std::string key;
  for (size_t i = 0; i < kCount; ++i) {
    values[i] = op.getMetadataValue(kKeys[i]);
    key += values[i];
    key += '\0';
  }
  auto it = collectives_.find(key);
  if (it != collectives_.end()) return it->second;
  const ktj_collective_meta meta = {
      values[0].c_str(),  values[1].c_str(),  values[2].c_str(),  values[3].c_str(),  values[4].c_str(),  values[5].c_str(),
      values[6].c_str(),  values[7].c_str(),  values[8].c_str(),  values[9].c_str(),  values[10].c_str(), values[11].c_str(),
      values[12].c_str(), values[13].c_str(), values[14].c_str(), values[15].c_str(), values[16].c_str()}; /* kKeys order */
  uint32_t index = 0;
  note(ktj_add_collective(engine_, &meta, &index), "ktj_add_collective");
  collectives_.emplace(std::move(key), index);
  return index;
}

/* One schema per distinct list of counter names: a keyed double field for each. */
uint32_t GpuChromeTraceLogger::counterSchema(const std::vector<std::pair<std::string, double>>& values) {
  if (values.empty()) return KTJ_NONE;
  std::string key;
  std::vector<ktj_field> fields;
  fields.reserve(values.size());
  for (const auto& kv : values) {
    const uint32_t id = intern(names_, kv.first);
    fields.push_back(ktj_field{id, KTJ_F_F64, 1});
    key.append(reinterpret_cast<const char*>(&id), sizeof(id));
  }
  auto it = counterSchemas_.find(key);
  if (it != counterSchemas_.end()) return it->second;
  uint32_t sid = KTJ_NONE;
  note(ktj_register_schema(engine_, fields.data(), fields.size(), &sid), "ktj_register_schema");
  counterSchemas_.emplace(std::move(key), sid);
  return sid;
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
  if (records_.empty() || !ok()) return;
  uint64_t first = 0;
  note(ktj_submit_args(engine_, slots_.data(), slots_.size(), &first), "ktj_submit_args");
  if (status_ == 0 && first + slots_.size() != nextSlot_) note(KTJ_ERR_STATE, "args slot bookkeeping");
  note(ktj_submit_records(engine_, KTJ_REC_GENERIC, records_.data(), records_.size()), "ktj_submit_records");
  records_.clear();
  slots_.clear();
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

void GpuChromeTraceLogger::handleActivity(const ITraceActivity& op) {
  if (!ok()) return;
  const ActivityType type = op.type();
  const std::string name = op.name();
  const ITraceActivity* linked = op.linkedActivity();
  const int64_t device = op.deviceId();
  const int64_t flowId = op.flowId();
  const bool counter = type == ActivityType::HARDWARE_COUNTERS || type == ActivityType::MTIA_COUNTERS ||
      type == ActivityType::XPU_SCOPE_PROFILER; /* output_json.cpp:847-856 */
  /* collective metadata comes from a linked record_param_comms op (output_json.cpp:899-908) */
  const bool collective = !counter && linked != nullptr &&
      (type == ActivityType::CONCURRENT_KERNEL || (type == ActivityType::MTIA_CCP_EVENTS && name.rfind("hccl::", 0) == 0)) &&
      linked->name() == kParamCommsName;
  const bool unsupported = device < std::numeric_limits<int32_t>::min() || device > std::numeric_limits<int32_t>::max();
  if (unsupported) {
    if (unsupported_++ == 0) {
      LOG(WARNING) << "GpuChromeTraceLogger: activity '" << name << "' of type " << toString(type)
                   << " is of a kind the GPU engine does not render; such activities are dropped";
    }
    return;
  }

  ktj_generic_rec r{};
  r.start_ns = op.timestamp();
  r.end_ns = r.start_ns + op.duration();
  r.resource = op.resourceId();
  r.device = static_cast<int32_t>(device);
  r.id = static_cast<int32_t>(op.correlationId()); /* `int external_id = op.correlationId()`, :893 */
  r.type = static_cast<uint8_t>(type);
  r.name_id = intern(names_, name);
  r.flow_id = flowId;
  const int flowType = op.flowType(); /* anything but the two known kinds prints no flow event (:979-994) */
  r.flow_type = (flowType == static_cast<int>(KTJ_LINK_FWDBWD) || flowType == static_cast<int>(KTJ_LINK_ASYNC_CPU_GPU)) ? static_cast<uint8_t>(flowType) : 0;
  r.flags = op.flowStart() ? KTJ_GF_FLOW_START : 0;
  if (linked != nullptr) {
    r.flags |= KTJ_GF_LINKED;
    r.linked_id = static_cast<int32_t>(linked->correlationId()); /* `int external_id = …`, :873 */
  }
  if (counter) { /* handleCounterEvent (:679-716) prints counterValues() and nothing else */
    const auto& values = op.counterValues();
    r.schema_id = counterSchema(values);
    r.args_off = nextSlot_;
    nextSlot_ += values.size();
    for (const auto& kv : values) {
      uint64_t bits;
      static_assert(sizeof(bits) == sizeof(kv.second), "double is 64 bits");
      std::memcpy(&bits, &kv.second, sizeof(bits));
      slots_.push_back(bits);
    }
    records_.push_back(r);
    if (records_.size() >= kRecordBatch) flushRecords();
    return;
  }
  const std::string metadata = op.metadataJson();
  if (collective) { /* the first slot names the linked op's collective metadata */
    r.schema_id = metadata.empty() ? collectiveSchema_ : collectiveFragmentSchema_;
    r.args_off = nextSlot_++;
    slots_.push_back(collectiveIndex(*linked));
    if (!metadata.empty()) {
      ++nextSlot_;
      slots_.push_back(intern(fragments_, metadata));
    }
  } else if (metadata.empty()) {
    r.schema_id = KTJ_NONE;
  } else {
    r.schema_id = fragmentSchema_;
    r.args_off = nextSlot_++;
    slots_.push_back(intern(fragments_, metadata));
  }
  records_.push_back(r);
  if (records_.size() >= kRecordBatch) flushRecords();
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
  flushStrings();
  flushRecords();
  uint64_t written = 0;
  if (status_ == 0) note(ktj_finalize(engine_, endTime, &written), "ktj_finalize");
  if (status_ != 0) {
    LOG(ERROR) << "Failed to write to log file!";
    return;
  }
  LOG(INFO) << "Chrome Trace written to " << fileName_ << " (" << written << " bytes)";
}

}  // namespace ktj_shim
