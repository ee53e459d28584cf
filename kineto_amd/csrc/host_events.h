/*
 * host_events.h — the few events of a trace that are not per-activity: header, process/thread
 * metadata, trace spans, footer.  O(#devices + #streams) strings, formatted on the host and
 * placed before and after the GPU-formatted activity section.
 */
#ifndef KTJ_HOST_EVENTS_H_
#define KTJ_HOST_EVENTS_H_

#include <string>
#include <vector>

#include "../../include/ktj.h"

namespace ktj {

/* ChromeTraceLogger::handleTraceStart + metadataToJSON (libkineto/src/output_json.cpp:414-479) */
void append_trace_start(std::string& out, const char* const* meta_kv, size_t n_kv,
                        const char* device_properties, int64_t base_time_ns, bool display_ns = false);
/* handleDeviceInfo (output_json.cpp:507-542) */
void append_device_info(std::string& out, const ktj_device_info& info, int64_t base_time_ns);
/* handleResourceInfo (output_json.cpp:544-577) */
void append_resource_info(std::string& out, const ktj_resource_info& info, int64_t base_time_ns);
/* handleOverheadInfo (output_json.cpp:579-607) */
void append_overhead_info(std::string& out, const ktj_overhead_info& info, int64_t base_time_ns);
/* handleTraceSpan + addIterationMarker (output_json.cpp:609-658) */
void append_trace_span(std::string& out, const ktj_trace_span& span, int64_t base_time_ns);
/* finalizeTrace (output_json.cpp:1066-1096): "Record Window End", array close, the
 * "distributedInfo" entry if there is one, traceName */
void append_trace_end(std::string& out, int64_t end_time_ns, int64_t base_time_ns, const std::string& file_name,
                      const std::string& distributed_info = std::string());

/* What the logger keeps of one record_param_comms op. */
struct CollectiveInfo {
  std::string args;                                 /* appendCollectiveArgs (output_json.cpp:718-797), comma-joined */
  std::string pg_name, pg_desc, group_size, ranks;  /* process-group table entry (:818-834)                         */
  std::string rank;                                 /* "Rank" as handed over (:812)                                  */
};
CollectiveInfo make_collective(const ktj_collective_meta& meta);
/* One activity that printed collective metadata; `hccl` selects backend "hccl"/"mtia:hccl"
 * instead of "nccl"/"cuda:nccl" (output_json.cpp:901-907). */
struct CollectiveUse {
  uint32_t index;
  bool hccl;
};
/* appendCollectiveMetadata's bookkeeping replayed over the uses in emission order, then
 * addOnDemandDistMetadata (output_json.cpp:799-835, 1030-1064).  Empty if no use names the
 * default process group.  Process groups are listed in the iteration order of a
 * std::unordered_map keyed by group name, as the logger's own table is. */
std::string distributed_info_text(const std::vector<CollectiveInfo>& collectives, const std::vector<CollectiveUse>& uses);

}  // namespace ktj
#endif
