/*
 * sdk_rows.c — TEST INFRASTRUCTURE ONLY, part of the CPU checker.
 *
 * Restates RocprofLogger::buffer_callback (libkineto/src/RocprofLogger.cpp:681-749): which
 * rocprofiler-sdk buffer records become rocprofAsyncRow objects (src/RocLogger.h:216-240) and
 * with which fields.  The rows come out as ktj_device_rec, the packed form of rocprofAsyncRow.
 *
 * Pinned against the reference's own function: oracle/_ref/sdk_ref_driver compiles
 * RocprofLogger.cpp where it lies, fills the logger's agent and kernel-name tables and calls
 * buffer_callback on the same SDK records; tests/test_sdk_ingest.py compares the rows field by
 * field (hand-written records and the device rows of four synthetic configurations, with and
 * without records of other kinds mixed in).
 */
#include <rocprofiler-sdk/buffer_tracing.h>
#include <stdint.h>
#include <string.h>

#include "../include/ktj.h"

/* agents / kernel names: parallel arrays standing in for the logger's two maps.  Returns the
 * number of rows written to out (room for num_headers). */
uint64_t ktj_oracle_sdk_rows(void* const* headers, uint64_t num_headers, const uint64_t* agent_handles,
                             const int32_t* agent_devices, uint64_t n_agents, const uint64_t* kernel_ids,
                             const uint32_t* kernel_name_ids, uint64_t n_kernels, uint32_t unknown_name_id,
                             ktj_device_rec* out) {
  uint64_t n = 0;
  for (uint64_t i = 0; i < num_headers; ++i) {
    const rocprofiler_record_header_t* header = (const rocprofiler_record_header_t*)headers[i];
    if (header->category != ROCPROFILER_BUFFER_CATEGORY_TRACING) continue;        /* :692 */
    ktj_device_rec r;
    memset(&r, 0, sizeof r);
    uint64_t agent;
    if (header->kind == ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH) {              /* :693-724 */
      const rocprofiler_buffer_tracing_kernel_dispatch_record_t* rec =
          (const rocprofiler_buffer_tracing_kernel_dispatch_record_t*)header->payload;
      agent = rec->dispatch_info.agent_id.handle;
      r.id = rec->correlation_id.internal;
      r.domain = KTJ_DOM_KERNEL_DISPATCH;                                          /* record.kind */
      r.op = (uint32_t)rec->operation;
      r.queue = rec->dispatch_info.queue_id.handle;
      r.begin = rec->start_timestamp;
      r.end = rec->end_timestamp;
      r.name_id = unknown_name_id;                                                 /* "<unknown kernel>" :709-714 */
      for (uint64_t k = 0; k < n_kernels; ++k)
        if (kernel_ids[k] == rec->dispatch_info.kernel_id) r.name_id = kernel_name_ids[k]; /* last entry of an id wins */
    } else if (header->kind == ROCPROFILER_BUFFER_TRACING_MEMORY_COPY) {           /* :725-746 */
      const rocprofiler_buffer_tracing_memory_copy_record_t* rec =
          (const rocprofiler_buffer_tracing_memory_copy_record_t*)header->payload;
      agent = rec->dst_agent_id.handle;
      r.id = rec->correlation_id.internal;
      r.domain = KTJ_DOM_MEMORY_COPY;
      r.op = (uint32_t)rec->operation;
      r.queue = 0;
      r.begin = rec->start_timestamp;
      r.end = rec->end_timestamp;
      r.name_id = KTJ_NONE;                                                        /* "" */
    } else {
      continue;
    }
    r.device = -1;                                                                 /* :703-707, 733-737 */
    for (uint64_t k = 0; k < n_agents; ++k)
      if (agent_handles[k] == agent) r.device = agent_devices[k];
    out[n++] = r;
  }
  return n;
}
