/*
 * sdk_records.cpp — TEST INFRASTRUCTURE ONLY.
 *
 * Builds what rocprofiler-sdk hands to a buffer callback (an array of rocprofiler_record_header_t*
 * whose payloads are the SDK's own record structs) from a list of device rows, so that tests can
 * drive ktj_submit_sdk_buffer without a live profiling session.  Fields the logger does not read
 * (thread id, dispatch id, sizes, addresses, source agent, byte count) are filled with arbitrary
 * values; with `noise` records of other kinds and categories are mixed in.
 */
#include <rocprofiler-sdk/buffer_tracing.h>

#include <cstdint>
#include <cstring>
#include <deque>
#include <vector>

#include "../../include/ktj.h"
#include "../../kineto_amd/csrc/sdk_api_rows.h"

namespace {
struct SdkBuffer {
  std::deque<rocprofiler_buffer_tracing_kernel_dispatch_record_t> dispatches;
  std::deque<rocprofiler_buffer_tracing_memory_copy_record_t> copies;
  std::deque<rocprofiler_buffer_tracing_hip_api_record_t> apis;
  std::deque<rocprofiler_record_header_t> headers;
  std::vector<void*> header_ptrs;
};
}  // namespace

extern "C" {

/* agent handle of a row = agent_base + device + 1 (device -1 gives agent_base itself, which the
 * caller leaves out of its agent table); kernel id = kernel_base + name_id, and kernel_base - 1
 * for a row whose name is `unknown_name_id`. */
void* ktjsim_sdk_buffer_create(const ktj_device_rec* rows, uint64_t n, uint64_t agent_base, uint64_t kernel_base,
                               uint32_t unknown_name_id, int noise) {
  SdkBuffer* b = new SdkBuffer;
  auto add = [b](uint32_t category, uint32_t kind, void* payload) {
    rocprofiler_record_header_t h;
    std::memset(&h, 0, sizeof h);
    h.category = category;
    h.kind = kind;
    h.payload = payload;
    b->headers.push_back(h);
  };
  for (uint64_t i = 0; i < n; ++i) {
    const ktj_device_rec& r = rows[i];
    if (noise && i % 5 == 2) { /* a HIP runtime API record in the same buffer: not a device row */
      rocprofiler_buffer_tracing_hip_api_record_t a;
      std::memset(&a, 0x5A, sizeof a);
      a.size = sizeof a;
      a.kind = ROCPROFILER_BUFFER_TRACING_HIP_RUNTIME_API;
      b->apis.push_back(a);
      add(ROCPROFILER_BUFFER_CATEGORY_TRACING, ROCPROFILER_BUFFER_TRACING_HIP_RUNTIME_API, &b->apis.back());
    }
    if (r.domain == KTJ_DOM_MEMORY_COPY) {
      rocprofiler_buffer_tracing_memory_copy_record_t c;
      std::memset(&c, 0xC3, sizeof c);
      c.size = sizeof c;
      c.kind = ROCPROFILER_BUFFER_TRACING_MEMORY_COPY;
      c.operation = static_cast<rocprofiler_memory_copy_operation_t>(r.op);
      c.correlation_id.internal = r.id;
      c.start_timestamp = r.begin;
      c.end_timestamp = r.end;
      c.dst_agent_id.handle = agent_base + static_cast<uint64_t>(static_cast<int64_t>(r.device) + 1);
      c.src_agent_id.handle = agent_base + 77;
      b->copies.push_back(c);
      add(ROCPROFILER_BUFFER_CATEGORY_TRACING, ROCPROFILER_BUFFER_TRACING_MEMORY_COPY, &b->copies.back());
      if (noise && i % 7 == 1) /* same payload under a non-tracing category: skipped */
        add(ROCPROFILER_BUFFER_CATEGORY_COUNTERS, ROCPROFILER_BUFFER_TRACING_MEMORY_COPY, &b->copies.back());
    } else {
      rocprofiler_buffer_tracing_kernel_dispatch_record_t d;
      std::memset(&d, 0x3C, sizeof d);
      d.size = sizeof d;
      d.kind = ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH;
      d.operation = static_cast<rocprofiler_kernel_dispatch_operation_t>(r.op);
      d.correlation_id.internal = r.id;
      d.start_timestamp = r.begin;
      d.end_timestamp = r.end;
      d.dispatch_info.agent_id.handle = agent_base + static_cast<uint64_t>(static_cast<int64_t>(r.device) + 1);
      d.dispatch_info.queue_id.handle = r.queue;
      d.dispatch_info.kernel_id = r.name_id == unknown_name_id ? kernel_base - 1 : kernel_base + r.name_id;
      b->dispatches.push_back(d);
      add(ROCPROFILER_BUFFER_CATEGORY_TRACING, ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH, &b->dispatches.back());
    }
  }
  b->header_ptrs.reserve(b->headers.size());
  for (auto& h : b->headers) b->header_ptrs.push_back(&h);
  return b;
}
void* const* ktjsim_sdk_buffer_headers(void* buf) { return static_cast<SdkBuffer*>(buf)->header_ptrs.data(); }
uint64_t ktjsim_sdk_buffer_count(void* buf) { return static_cast<SdkBuffer*>(buf)->header_ptrs.size(); }
void ktjsim_sdk_buffer_free(void* buf) { delete static_cast<SdkBuffer*>(buf); }

/* ---- HIP runtime API callback records (ktj_submit_sdk_api_record) ---- */
uint64_t ktjsim_sdk_api_args_size(void) { return sizeof(rocprofiler_hip_api_args_t); }
uint32_t ktjsim_sdk_api_last_op(void) { return ROCPROFILER_HIP_RUNTIME_API_ID_LAST; }
/* the engine's conversion (kineto_amd/csrc/sdk_api_rows.h) of one call whose argument union holds
 * the given bytes */
uint32_t ktjsim_sdk_api_row(uint32_t operation, uint64_t correlation_id, const void* args_bytes, uint64_t begin, uint64_t end,
                            uint32_t pid, uint32_t tid, ktj_runtime_rec* out) {
  rocprofiler_hip_api_args_t args;
  std::memcpy(&args, args_bytes, sizeof args);
  return ktj::sdk_api::runtime_row(operation, correlation_id, args, begin, end, pid, tid, out);
}
/* a callback record as the SDK hands it over, around the same bytes (for ktj_submit_sdk_api_record);
 * freed with ktjsim_sdk_api_record_free */
struct ApiRecordHolder { rocprofiler_callback_tracing_record_t rec; rocprofiler_callback_tracing_hip_api_data_t data; };
void* ktjsim_sdk_api_record_create(uint32_t kind, uint32_t operation, uint64_t correlation_id, const void* args_bytes) {
  typedef ApiRecordHolder Holder;
  Holder* h = new Holder;
  std::memset(h, 0, sizeof *h);
  h->data.size = sizeof h->data;
  std::memcpy(&h->data.args, args_bytes, sizeof h->data.args);
  h->rec.kind = static_cast<rocprofiler_callback_tracing_kind_t>(kind);
  h->rec.operation = static_cast<rocprofiler_tracing_operation_t>(operation);
  h->rec.correlation_id.internal = correlation_id;
  h->rec.phase = ROCPROFILER_CALLBACK_PHASE_EXIT;
  h->rec.payload = &h->data;
  return h;
}
void ktjsim_sdk_api_record_free(void* p) { delete static_cast<ApiRecordHolder*>(p); }
uint32_t ktjsim_sdk_api_kind_hip_runtime(void) { return ROCPROFILER_CALLBACK_TRACING_HIP_RUNTIME_API; }
int ktjsim_sdk_api_is_flow_start(uint32_t operation) { return ktj::sdk_api::is_flow_start(operation) ? 1 : 0; }
/* the SDK's number of a few operations the tests name */
int64_t ktjsim_sdk_api_op_id(const char* name) {
#define X(op) if (std::strcmp(name, #op) == 0) return ROCPROFILER_HIP_RUNTIME_API_ID_##op;
  KTJ_SDK_FLOW_START_APIS(X) X(hipMemcpyDtoD) X(hipDeviceSynchronize) X(hipGetDevice)
#undef X
  return -1;
}

}  // extern "C"
