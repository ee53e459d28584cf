/*
 * ktj_rocprofiler.h — rocprofiler-sdk records straight into the engine: the buffer records of
 * kernel dispatches and memory copies (device rows) and the callback records of HIP runtime API
 * calls (runtime rows).
 *
 * Replaces the body of RocprofLogger::buffer_callback (libkineto/src/RocprofLogger.cpp:681-749),
 * which turns every kernel-dispatch and memory-copy record of an SDK buffer into a heap-allocated
 * rocprofAsyncRow with a copied kernel-name string.  Here the same fields go into packed device
 * rows (ktj_device_rec) in one pass over the headers, and from there to the GPU; the two lookups of
 * that function (agent handle -> device index, kernel id -> kernel name) use tables the caller
 * keeps up to date from the SDK's agent query and code-object callbacks
 * (RocprofLogger.cpp: globalContext.agents, globalContext.kernel_names).
 *
 * The header does not include the SDK's: `headers` is the `rocprofiler_record_header_t**` the
 * SDK passes to its buffer callback.
 */
#ifndef KTJ_ROCPROFILER_H_
#define KTJ_ROCPROFILER_H_

#include "ktj.h"

#ifdef __cplusplus
extern "C" {
#endif

/* globalContext.agents: agent handle -> logical_node_type_id.  An agent that is not listed gives
 * device -1 (RocprofLogger.cpp:703-707).  Replaces the table. */
int ktj_set_sdk_agents(ktj_engine* e, const uint64_t* agent_handles, const int32_t* device_ids, size_t n);

/* globalContext.kernel_names: kernel id -> string id of the kernel's name.  A kernel that is not
 * listed gets unknown_name_id, the string id of "<unknown kernel>" (RocprofLogger.cpp:709-714).
 * Adds to the table; a kernel id given again takes the new name. */
int ktj_set_sdk_kernel_names(ktj_engine* e, const uint64_t* kernel_ids, const uint32_t* name_ids, size_t n,
                             uint32_t unknown_name_id);

/* One call of the SDK's buffer callback.  Records of category ROCPROFILER_BUFFER_CATEGORY_TRACING
 * and kind ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH or ROCPROFILER_BUFFER_TRACING_MEMORY_COPY
 * become device rows, in header order, after the rows submitted so far; every other record is
 * skipped, as the reference skips it.  *n_rows receives the number of rows taken.  The SDK's
 * buffer may be released when the call returns. */
int ktj_submit_sdk_buffer(ktj_engine* e, void* const* headers, size_t num_headers, uint64_t* n_rows);

/* One HIP runtime API call, at ROCPROFILER_CALLBACK_PHASE_EXIT of the SDK's callback tracing
 * service: replaces the row construction of RocprofLogger::api_callback
 * (libkineto/src/RocprofLogger.cpp:561-679).  `record` is the SDK's
 * `const rocprofiler_callback_tracing_record_t*` (kind ROCPROFILER_CALLBACK_TRACING_HIP_RUNTIME_API,
 * anything else is ignored as the reference ignores it; its payload is the SDK's
 * rocprofiler_callback_tracing_hip_api_data_t).  begin / end are the caller's timestamps of the
 * enter and exit phases (the reference takes getApproximateTime() in both, :569-574), pid / tid the
 * calling process and thread.  The call becomes one runtime row (ktj_runtime_rec: kernel launch,
 * copy, malloc/free or plain, by operation) after the rows submitted so far; its arguments are read
 * from the SDK's argument union by the names the reference looks for.  external_id /
 * user_external_id: the innermost id of the caller's external-correlation stack of domain 0 / 1, or
 * NULL where that stack is empty (:661-672): each gives one KTJ_REC_EXTCORR / KTJ_REC_USERCORR pair
 * for the call's correlation id.  Rows are buffered on the host and reach the device in batches:
 * when 65536 have gathered, before a ktj_submit_records / ktj_submit_records_device call of the
 * KTJ_REC_RUNTIME, KTJ_REC_EXTCORR or KTJ_REC_USERCORR class appends (so arrival order is call
 * order), with ktj_flush, and with the next ktj_process / ktj_finalize.  ktj_process_noalloc does
 * not take them (growing the device arrays allocates): call ktj_flush before it. */
int ktj_submit_sdk_api_record(ktj_engine* e, const void* record, uint64_t begin, uint64_t end, uint32_t pid,
                              uint32_t tid, const uint64_t* external_id, const uint64_t* user_external_id);

/* Sends the rows that ktj_submit_sdk_api_record has buffered on the host to the device, without
 * processing anything.  No counterpart in the reference (its rows stay in host vectors,
 * RocprofLogger.h:84). */
int ktj_flush(ktj_engine* e);

#ifdef __cplusplus
}
#endif
#endif /* KTJ_ROCPROFILER_H_ */
