/*
 * ktj.h — C ABI of the MI355X trace post-processing engine ("ktj" = kineto trace → JSON).
 *
 * The engine turns raw activity records into Chrome-trace JSON that is byte-identical to what
 * libkineto's ChromeTraceLogger writes for the same records.  Everything below is plain C:
 * opaque handle, pointers and sizes, int status codes (0 = ok, negative = error).  Nothing
 * throws or aborts across this boundary.  One producer thread per engine, like the reference
 * logger (libkineto/src/output_json.h:62-63).
 *
 * Reference interfaces each entry point replaces are cited as file:line relative to the
 * pytorch/kineto tree.
 */
#ifndef KTJ_H_
#define KTJ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * Status codes
 * ---------------------------------------------------------------------------------------- */
#define KTJ_OK 0
#define KTJ_ERR_ARG (-1)      /* bad argument (null pointer, unknown id, out-of-range index)   */
#define KTJ_ERR_STATE (-2)    /* call order violated (e.g. submit after finalize)               */
#define KTJ_ERR_HIP (-3)      /* a HIP call failed; ktj_last_error() has the text               */
#define KTJ_ERR_IO (-4)       /* output file could not be opened / written / renamed            */
#define KTJ_ERR_NOMEM (-5)    /* host or device allocation failed                               */
#define KTJ_ERR_LIMIT (-6)    /* input exceeds a documented limit                               */

/* ------------------------------------------------------------------------------------------
 * Limits of one trace.  A trace beyond one of them is refused by ktj_process with KTJ_ERR_LIMIT
 * and a ktj_last_error() text that names the limit; nothing is written.  The reference keeps
 * these in node-based maps and has no such limits.
 *   - (device, stream) pairs among the device records (the pairs that RocprofActivity's dense
 *     stream index numbers, libkineto/src/RocprofActivity_inl.h:118-146);
 *   - distinct hardware queue ids among the device records (used where a device record's stream
 *     has to be found through its queue);
 *   - (deviceId, resourceId) pairs of "Stream Sync" CUDA_SYNC activities (output_json.cpp:913-943).
 * The number of distinct deviceId and resourceId values is not limited; above 4096 of either the
 * sort works on the raw 64-bit values instead of ranks, which is several times slower.
 * Record counts are limited by device memory and by 32-bit row indices (fewer than 2^32 - 16 rows).
 * ---------------------------------------------------------------------------------------- */
#define KTJ_MAX_STREAM_PAIRS 4096u
#define KTJ_MAX_QUEUES 32768u
#define KTJ_MAX_SYNC_ROWS 32768u

#define KTJ_NONE 0xFFFFFFFFu  /* "no string" / "no schema" sentinel for 32-bit ids              */

/* ------------------------------------------------------------------------------------------
 * Activity types: numeric values and category strings of libkineto::ActivityType
 * (libkineto/include/ActivityType.h:19-62, names :80-111).
 * ---------------------------------------------------------------------------------------- */
enum {
  KTJ_TYPE_CPU_OP = 0,
  KTJ_TYPE_USER_ANNOTATION = 1,
  KTJ_TYPE_GPU_USER_ANNOTATION = 2,
  KTJ_TYPE_GPU_MEMCPY = 3,
  KTJ_TYPE_GPU_MEMSET = 4,
  KTJ_TYPE_CONCURRENT_KERNEL = 5,
  KTJ_TYPE_EXTERNAL_CORRELATION = 6,
  KTJ_TYPE_CUDA_RUNTIME = 7,
  KTJ_TYPE_CUDA_DRIVER = 8,
  KTJ_TYPE_CPU_INSTANT_EVENT = 9,
  KTJ_TYPE_PYTHON_FUNCTION = 10,
  KTJ_TYPE_OVERHEAD = 11,
  KTJ_TYPE_MTIA_RUNTIME = 12,
  KTJ_TYPE_MTIA_CCP_EVENTS = 13,
  KTJ_TYPE_MTIA_INSIGHT = 14,
  KTJ_TYPE_CUDA_SYNC = 15,
  KTJ_TYPE_CUDA_EVENT = 16,
  KTJ_TYPE_MTIA_COUNTERS = 17,
  KTJ_TYPE_GLOW_RUNTIME = 18,
  KTJ_TYPE_CUDA_PROFILER_RANGE = 19,
  KTJ_TYPE_HPU_OP = 20,
  KTJ_TYPE_XPU_RUNTIME = 21,
  KTJ_TYPE_XPU_DRIVER = 22,
  KTJ_TYPE_COLLECTIVE_COMM = 23,
  KTJ_TYPE_PRIVATEUSE1_RUNTIME = 24,
  KTJ_TYPE_PRIVATEUSE1_DRIVER = 25,
  KTJ_TYPE_XPU_SCOPE_PROFILER = 26,
  KTJ_TYPE_XPU_SYNC = 27,
  KTJ_TYPE_HARDWARE_COUNTERS = 28,
  KTJ_TYPE_COUNT = 29
};

/* Flow link types (libkineto/include/GenericTraceActivity.h:29-30). */
#define KTJ_LINK_FWDBWD 1u
#define KTJ_LINK_ASYNC_CPU_GPU 2u

/* ------------------------------------------------------------------------------------------
 * Raw activity records (the engine's input "activity buffers").  Packed arrays of fixed-size
 * little-endian structs; sizes are multiples of 16 so that one lane reads 16 bytes at a time.
 * ---------------------------------------------------------------------------------------- */

/* Record classes for ktj_submit_records(). */
enum {
  KTJ_REC_GENERIC = 0,  /* ktj_generic_rec  */
  KTJ_REC_RUNTIME = 1,  /* ktj_runtime_rec  */
  KTJ_REC_DEVICE = 2,   /* ktj_device_rec   */
  KTJ_REC_EXTCORR = 3,  /* ktj_extcorr_rec, domain 0: correlation id -> CPU op              */
  KTJ_REC_USERCORR = 4  /* ktj_extcorr_rec, domain 1: correlation id -> user annotation     */
};

/*
 * Generic activity: the fields of libkineto::GenericTraceActivity
 * (libkineto/include/GenericTraceActivity.h:174-195) plus what ChromeTraceLogger reads from a
 * linked activity (libkineto/src/output_json.cpp:871-874).  CPU-op spans submitted by a
 * profiler client and every activity that arrives through ActivityLogger::handleActivity use
 * this shape.
 *
 * Two kinds are not complete events.  KTJ_TYPE_CPU_INSTANT_EVENT prints an instant event
 * (output_json.cpp:660-677).  KTJ_TYPE_HARDWARE_COUNTERS, KTJ_TYPE_MTIA_COUNTERS and
 * KTJ_TYPE_XPU_SCOPE_PROFILER print counter events (output_json.cpp:679-716): the record's
 * counterValues() are the keyed KTJ_F_F64 fields of its schema in schema order, its other fields
 * are not printed.  Neither kind prints an External id or a flow event.
 */
typedef struct ktj_generic_rec {
  int64_t start_ns;      /* startTime (absolute ns)                                            */
  int64_t end_ns;        /* endTime; duration() = end_ns - start_ns                            */
  int64_t resource;      /* resourceId(): thread id or stream id                               */
  int64_t flow_id;       /* flowId(): flow.id of a GenericTraceActivity, the correlation id of
                            runtime / device wrappers; a flow event follows when it is > 0     */
  uint64_t args_off;     /* first 8-byte slot of this record's values in the args blob         */
  int32_t id;            /* correlationId() as the logger reads it: `int external_id`
                            (output_json.cpp:871-893); GenericTraceActivity::id is int32       */
  int32_t device;        /* deviceId() — process id for CPU ops.  A deviceId that does not fit 32
                            bits goes into the args slot before args_off, with KTJ_GF_WIDE_DEVICE */
  uint32_t name_id;      /* string id of name()                                                */
  int32_t linked_id;     /* linkedActivity()->correlationId(), int-truncated like the logger's
                            `int external_id`; read only if KTJ_GF_LINKED                      */
  uint32_t schema_id;    /* args schema, KTJ_NONE = no metadata                                */
  uint8_t type;          /* KTJ_TYPE_*                                                         */
  uint8_t flow_type;     /* flow.type (4 bits)                                                 */
  uint8_t flags;         /* KTJ_GF_*                                                           */
  uint8_t pad0;
} ktj_generic_rec;       /* 64 bytes; getThreadId() is never printed and is not carried */

#define KTJ_GF_FLOW_START 0x01u /* flow.start                                                  */
#define KTJ_GF_LINKED 0x02u     /* linkedActivity() != nullptr                                 */
#define KTJ_GF_WIDE_DEVICE 0x04u /* deviceId() is args[args_off - 1] (an int64), `device` is unused */

/* Kinds of runtime rows: libkineto/src/RocLogger.h:74-81 (rocprof_activity_types). */
enum {
  KTJ_RT_DEFAULT = 0, /* rocprofRow        (RocLogger.h:101-118) */
  KTJ_RT_KERNEL = 1,  /* rocprofKernelRow  (RocLogger.h:120-165) */
  KTJ_RT_COPY = 2,    /* rocprofCopyRow    (RocLogger.h:167-194) */
  KTJ_RT_MALLOC = 3   /* rocprofMallocRow  (RocLogger.h:196-214) */
};

/*
 * Runtime-API row: union of rocprofRow / rocprofKernelRow / rocprofCopyRow / rocprofMallocRow.
 * begin/end are in the host's approximate-clock domain and go through the clock model
 * (libkineto/src/RocprofActivityApi.cpp:171-174).
 */
typedef struct ktj_runtime_rec {
  uint64_t id;     /* correlation id                                                          */
  uint64_t begin;
  uint64_t end;
  uint32_t cid;    /* runtime API operation id; name and flow-start come from the API table   */
  uint32_t pid;
  uint32_t tid;
  uint32_t kind;   /* KTJ_RT_*                                                                */
  union {
    struct {
      uint32_t grid[3];
      uint32_t workgroup[3];
      uint64_t group_segment_size;
      uint64_t stream;          /* hipStream_t as integer; 0 = null stream                     */
      uint32_t kernel_name_id;  /* "kernel" arg when the function pointer is known, else KTJ_NONE */
      uint32_t pad;
    } kernel;
    struct {
      uint64_t src;
      uint64_t dst;
      uint64_t size;
      uint64_t stream;
      uint32_t copy_kind;       /* hipMemcpyKind as integer                                    */
      uint32_t pad;
    } copy;
    struct {
      uint64_t ptr;
      uint64_t size;
    } malloc_;
    uint64_t raw[7];
  } u;
} ktj_runtime_rec; /* 96 bytes */

/* Device-row domains. */
enum {
  KTJ_DOM_KERNEL_DISPATCH = 0, /* rocprofAsyncRow, ROCPROFILER_BUFFER_TRACING_KERNEL_DISPATCH */
  KTJ_DOM_MEMORY_COPY = 1,     /* rocprofAsyncRow, ROCPROFILER_BUFFER_TRACING_MEMORY_COPY     */
  KTJ_DOM_MEMSET = 2           /* memset record shaped like CUpti_ActivityMemset
                                  (libkineto/src/CuptiActivity.h:682-713)                      */
};

/* Copy directions: numeric values of rocprofiler_memory_copy_operation_t. */
enum {
  KTJ_COPY_NONE = 0,
  KTJ_COPY_H2H = 1,
  KTJ_COPY_H2D = 2,
  KTJ_COPY_D2H = 3,
  KTJ_COPY_D2D = 4
};

/*
 * Device (asynchronous) row: rocprofAsyncRow (libkineto/src/RocLogger.h:216-240).  The kernel
 * name std::string becomes a string id.  A KTJ_DOM_MEMSET row is read through ktj_memset_rec below.
 */
typedef struct ktj_device_rec {
  uint64_t id;       /* correlation id                                                        */
  uint64_t begin;    /* device clock                                                          */
  uint64_t end;
  uint32_t domain;   /* KTJ_DOM_* in the low 16 bits (KTJ_ROW_DOMAIN); the upper 16 bits are read
                        on memset rows only                                                   */
  uint32_t op;       /* KTJ_COPY_* for copies                                                 */
  int32_t device;
  uint32_t name_id;  /* kernel name, KTJ_NONE = empty                                         */
  uint64_t queue;    /* HSA queue id                                                          */
  uint64_t stream;   /* 0 = unknown: back-filled from the correlated runtime row              */
  uint64_t bytes;    /* KTJ_DOM_MEMSET only                                                   */
} ktj_device_rec;    /* 64 bytes */
#define KTJ_ROW_DOMAIN(raw) ((uint32_t)(raw) & 0xFFFFu)

/*
 * The KTJ_DOM_MEMSET view of a device row: the fields of CUpti_ActivityMemset4 that
 * GpuActivity<CUpti_ActivityMemsetType> reads (libkineto/src/CuptiActivity.h:682-719, with
 * :424-458 for the graph and channel keys).  Same 64 bytes as ktj_device_rec, member by member:
 * `domain` splits into domain / channel_type / memory_kind, `op` and `name_id` hold the two halves
 * of the graph node id, `queue` holds context and channel id, `stream` holds stream and graph id.
 * No ROCm producer makes such a row (the reference's ROCm GpuActivity never takes the GPU_MEMSET
 * type, libkineto/src/RocprofActivity.h:84-98); it exists for CUDA-shaped record streams.
 * The name is "Memset (<memory kind>)" (cupti_strings.cpp:42-66); timestamp() = begin and
 * duration() = end - begin; the stream is not back-filled.  The args are
 *   "device", "context", "stream", "correlation", "bytes"[, "memory bandwidth (GB/s)" unless the
 *   duration is 0] — what a reference built against CUDA < 12 prints — and, in an engine created
 *   with KTJ_CREATE_CUDA12_ARGS, also "graph id", "graph node id", "channel", "channel_type", as a
 *   reference built against CUDA >= 12 prints them.
 */
typedef struct ktj_memset_rec {
  uint64_t id;            /* correlationId (32 bits in CUPTI; all 64 are joined and printed)    */
  uint64_t begin;         /* start                                                              */
  uint64_t end;
  uint16_t domain;        /* KTJ_DOM_MEMSET                                                     */
  uint8_t channel_type;   /* CUpti_ChannelType                                                  */
  uint8_t memory_kind;    /* CUpti_ActivityMemoryKind: KTJ_MEMKIND_*                            */
  uint32_t graph_node_lo; /* graphNodeId, low half                                              */
  int32_t device;         /* deviceId                                                           */
  uint32_t graph_node_hi; /* graphNodeId, high half                                             */
  uint32_t context;       /* contextId                                                          */
  uint32_t channel_id;    /* channelID                                                          */
  uint32_t stream;        /* streamId                                                           */
  uint32_t graph_id;      /* graphId                                                            */
  uint64_t bytes;
} ktj_memset_rec;         /* 64 bytes */

/* CUpti_ActivityMemoryKind as memoryKindString names it (libkineto/src/cupti_strings.cpp:42-66);
 * any other value prints "Unrecognized". */
enum {
  KTJ_MEMKIND_UNKNOWN = 0,        /* "Unknown"        */
  KTJ_MEMKIND_PAGEABLE = 1,       /* "Pageable"       */
  KTJ_MEMKIND_PINNED = 2,         /* "Pinned"         */
  KTJ_MEMKIND_DEVICE = 3,         /* "Device"         */
  KTJ_MEMKIND_ARRAY = 4,          /* "Array"          */
  KTJ_MEMKIND_MANAGED = 5,        /* "Managed"        */
  KTJ_MEMKIND_DEVICE_STATIC = 6,  /* "Device Static"  */
  KTJ_MEMKIND_MANAGED_STATIC = 7  /* "Managed Static" */
};

/* External-correlation pair (libkineto/src/RocmActivityProfiler.cpp:135-148).  Domain 0
 * (KTJ_REC_EXTCORR, cpuCorrelationMap_): correlation id -> CPU-op id, the "External id" link.
 * Domain 1 (KTJ_REC_USERCORR, userCorrelationMap_): correlation id -> id of a user annotation; when
 * any are submitted, every (device, stream) on which device rows of one annotation ran gets a
 * GPU_USER_ANNOTATION activity that spans them (GenericActivityProfiler.cpp:277-327, 425-433, 726). */
typedef struct ktj_extcorr_rec {
  uint64_t correlation;
  uint64_t external_id;
} ktj_extcorr_rec; /* 16 bytes */

/* ------------------------------------------------------------------------------------------
 * Args schemas: the typed metadata of a generic activity, in emission order
 * (libkineto/include/TypedMetadataJson.h:38-205).  A record's values live in the args blob as
 * consecutive 8-byte slots starting at args_off; each field consumes `count` slots.
 * ---------------------------------------------------------------------------------------- */
enum {
  KTJ_F_I64 = 0,   /* int64 via to_chars                                  (1 slot)            */
  KTJ_F_U64 = 1,   /* uint64 via to_chars                                 (1 slot)            */
  KTJ_F_F64 = 2,   /* double via fmt "{}"; non-finite values are quoted   (1 slot)            */
  KTJ_F_BOOL = 3,  /* true / false                                        (1 slot)            */
  KTJ_F_STR = 4,   /* slot = string id, emitted in double quotes          (1 slot)            */
  KTJ_F_RAW = 5,   /* slot = string id, emitted verbatim (RawJson)        (1 slot)            */
  KTJ_F_I64_ARRAY = 6, /* [a, b, c] with `count` int64 elements           (count slots)       */
  KTJ_F_COLLECTIVE = 7, /* slot = index from ktj_add_collective; keyless, recognised only as the
                          first field of a schema; prints nothing in the fragment (1 slot)    */
  KTJ_F_STR_ARRAY = 8, /* ["a", "b"] with `count` quoted strings, slots = string ids
                          (std::vector<std::string>, TypedMetadataJson.h:52-64) (count slots) */
  KTJ_F_DICT_BEGIN = 9, /* "key": { — the fields up to the matching KTJ_F_DICT_END are the dict's
                          children (beginDict, TypedMetadataJson.h:128-132); dicts nest (0 slots) */
  KTJ_F_DICT_END = 10, /* } (endDict, TypedMetadataJson.h:134-137); keyless             (0 slots) */
  KTJ_F_SHAPES = 11,   /* InputShapes ("Input Dims": [[2, 2], [[4, 1], [4, 1]]], TypedMetadata.h:
                          39-47): the slot holds the index of the first slot of the value's
                          encoding elsewhere in the args blob, see below              (1 slot) */
  KTJ_F_UNSUPPORTED = 12 /* "key": "<unsupported metadata type>" (visitUnsupported,
                          TypedMetadataJson.h:122-126)                                (0 slots) */
};
/* Encoding of a KTJ_F_SHAPES value in 8-byte slots: [n] then n entries; an entry is either
 * [KTJ_SHAPE_TENSOR | rank][rank dims] (one tensor's shape, printed [d0, d1]) or
 * [KTJ_SHAPE_LIST | m] followed by m times [rank][rank dims] (a TensorList argument, printed
 * [[..], [..]]).  Dims are int64. */
#define KTJ_SHAPE_TENSOR 0ull
#define KTJ_SHAPE_LIST (1ull << 32)

typedef struct ktj_field {
  uint32_t key_id; /* string id of the key; KTJ_NONE = the slot's string is a whole fragment   */
  uint16_t type;   /* KTJ_F_*                                                                 */
  uint16_t count;  /* slots consumed: 1, the element count of an array, 0 for dict brackets and
                      KTJ_F_UNSUPPORTED                                                        */
} ktj_field;

#define KTJ_MAX_SCHEMA_FIELDS 1024

/* ------------------------------------------------------------------------------------------
 * Collective metadata (ChromeTraceLogger::appendCollectiveMetadata, output_json.cpp:718-835,
 * 899-908, and the "distributedInfo" entry of the footer, :1030-1064).  The logger copies it from
 * the `record_param_comms` CPU op an activity is linked to; here the caller hands the op's
 * values over once (ktj_add_collective) and refers to them from records by index, through a
 * leading KTJ_F_COLLECTIVE field:
 *   - on a generic record of type KTJ_TYPE_CONCURRENT_KERNEL or KTJ_TYPE_MTIA_CCP_EVENTS
 *     (backends "nccl" / "hccl"): the record prints the collective arguments after its own
 *     metadata — the case of an activity that arrives with its linked op resolved;
 *   - on any other generic record (the record_param_comms CPU op itself): kernel rows of
 *     KTJ_REC_DEVICE that the join links to this record print them (backend "nccl").
 * Every value is the text getMetadataValue() returns for the key (strings may keep their
 * surrounding quotes); NULL or "" = the op does not carry the key.
 * ---------------------------------------------------------------------------------------- */
typedef struct ktj_collective_meta {
  const char* collective_name;   /* "Collective name"            */
  const char* in_msg_nelems;     /* "In msg nelems"              */
  const char* out_msg_nelems;    /* "Out msg nelems"             */
  const char* group_size;        /* "Group size"                 */
  const char* dtype;             /* "dtype"                      */
  const char* in_tensors_start;  /* "Input Tensors start"        */
  const char* out_tensors_start; /* "Output Tensors start"       */
  const char* in_split;          /* "In split size"              */
  const char* out_split;         /* "Out split size"             */
  const char* pg_name;           /* "Process Group Name"         */
  const char* pg_desc;           /* "Process Group Description"  */
  const char* group_ranks;       /* "Process Group Ranks"        */
  const char* dst_rank;          /* "Dst Rank"                   */
  const char* src_rank;          /* "Src Rank"                   */
  const char* seq;               /* "Seq"                        */
  const char* comms_id;          /* "Comms Id"                   */
  const char* rank;              /* "Rank" (distributedInfo only) */
} ktj_collective_meta;

/* ------------------------------------------------------------------------------------------
 * Small host-side events (formatted by the host part of the library; O(#devices + #streams)).
 * ---------------------------------------------------------------------------------------- */
enum {
  KTJ_INFO_DEVICE = 0,   /* ktj_device_info   */
  KTJ_INFO_RESOURCE = 1, /* ktj_resource_info */
  KTJ_INFO_OVERHEAD = 2, /* ktj_overhead_info */
  KTJ_INFO_SPAN = 3      /* ktj_trace_span    */
};

typedef struct ktj_device_info {    /* libkineto/include/IActivityProfiler.h:48-53 */
  int64_t id;
  int64_t sort_index;
  const char* name;
  const char* label;
  int64_t time_ns;
} ktj_device_info;

typedef struct ktj_resource_info {  /* libkineto/include/IActivityProfiler.h:63-70 */
  int64_t id;
  int64_t sort_index;
  int64_t device_id;
  const char* name;
  int32_t host_thread;              /* ResourceType::HOST_THREAD */
  int32_t pad;
  int64_t time_ns;
} ktj_resource_info;

typedef struct ktj_overhead_info {  /* libkineto/include/output_base.h:41-44 */
  const char* name;
  int64_t time_ns;
} ktj_overhead_info;

typedef struct ktj_trace_span {     /* libkineto/include/TraceSpan.h:17-36 */
  int64_t start_ns;
  int64_t end_ns;
  int32_t op_count;
  int32_t iteration;
  const char* name;
  const char* prefix;
} ktj_trace_span;

/* Clock model for raw → wall-clock conversion. */
typedef struct ktj_clock_model {
  uint64_t t0_approx;   /* libkineto/src/ApproximateClock.cpp:83-90: for t > t0_approx the       */
  int64_t t0;           /*   converter returns (int64)((double)(t - t0_approx) * scale) + t0     */
  double scale;         /*   with the product taken in x87 extended precision; else 0           */
  int64_t async_offset; /* added to device-row begin/end (RocprofActivityApi.cpp:166-170)       */
  uint32_t runtime_mode; /* KTJ_CLOCK_* applied to runtime rows                                 */
  uint32_t device_mode;  /* KTJ_CLOCK_* applied to device rows                                  */
} ktj_clock_model;

enum {
  KTJ_CLOCK_IDENTITY = 0, /* timestamps already are wall-clock ns                               */
  KTJ_CLOCK_CONVERT = 1,  /* apply the converter to begin and end separately
                             (libkineto/src/CuptiTimestamp.h:29-51)                             */
  KTJ_CLOCK_OFFSET = 2    /* add async_offset                                                   */
};

/* Counters of the post-processing stage (libkineto/src/GenericActivityProfiler.cpp:91-102,
 * 329-340, 363-395) and per-stage timing measured with HIP events on the engine's stream. */
#define KTJ_N_STAGES 12
typedef struct ktj_stats {
  uint64_t n_generic, n_runtime, n_device, n_extcorr;
  uint64_t n_emitted;              /* activities written                                        */
  uint64_t out_of_range_events;
  uint64_t gpu_and_cpu_op_out_of_order;
  uint64_t n_flow_events;
  uint64_t n_linked;               /* activities that found a CPU op via external correlation   */
  uint64_t n_blank_names;          /* names replaced by "unknown"                               */
  uint64_t output_bytes;
  uint64_t activity_bytes;         /* bytes of the sorted activity section                      */
  float stage_ms[KTJ_N_STAGES];    /* see KTJ_STAGE_*                                           */
  uint64_t stage_bytes[KTJ_N_STAGES]; /* algorithmic bytes moved by that stage                  */
} ktj_stats;

enum {
  KTJ_STAGE_DICT = 0,     /* name / string dictionary sanitising                               */
  KTJ_STAGE_DECODE = 1,   /* raw records → columns                                             */
  KTJ_STAGE_CONVERT = 2,  /* clock conversion + window filter: part of KTJ_STAGE_DECODE, always 0     */
  KTJ_STAGE_JOIN = 3,     /* hash build + probe (ext-corr, runtime↔device, streams)            */
  KTJ_STAGE_SORT = 4,     /* key build + stable radix sort                                     */
  KTJ_STAGE_SIZE = 5,     /* exact byte length per record                                      */
  KTJ_STAGE_SCAN = 6,     /* device-wide exclusive scan                                        */
  KTJ_STAGE_EMIT = 7,     /* JSON formatting into the output buffer                            */
  KTJ_STAGE_D2H = 8,      /* device → pinned host copy (file sink: time spent waiting for it)  */
  KTJ_STAGE_FILE = 9,     /* write + rename (host)                                             */
  KTJ_STAGE_TOTAL_GPU = 10 /* first kernel start → last kernel end                             */
};

typedef struct ktj_engine ktj_engine;

/* ------------------------------------------------------------------------------------------
 * Life cycle.  Replaces ChromeTraceLogger::ChromeTraceLogger / openTraceFile
 * (libkineto/src/output_json.cpp:485-505): opens "<out_path>.tmp"; empty or NULL path means
 * "/tmp/libkineto_activities_<pid>.json".  If the file cannot be opened the engine is still
 * created and every later call is a silent no-op returning KTJ_OK, like the reference's
 * `if (!traceOf_) return;`; ktj_finalize then returns KTJ_ERR_IO.
 * With KTJ_CREATE_NO_FILE no file is opened or written: the document stays in the engine's
 * buffers (ktj_output_device / ktj_output_host) and out_path is only the "traceName".
 * KTJ_CREATE_TILE_EMIT selects the output-partitioned emit kernel (one workgroup per tile of
 * output bytes, staged in LDS) instead of the default one-lane-per-activity kernel; both produce
 * the same bytes.
 * KTJ_CREATE_HASH_JOIN keeps the join tables in hash mode even when the correlation ids are dense
 * enough for direct addressing (the engine chooses per table otherwise); same results, slower.
 * KTJ_CREATE_DISPLAY_NS writes "displayTimeUnit": "ns" instead of "ms" in the header, as a reference
 * built with DISPLAY_TRACE_IN_NS does (output_json.cpp:451-454); nothing else changes.
 * KTJ_CREATE_PAIR_SORT sorts (key, arrival index) pairs also where key and index fit one 64-bit
 * word (the engine sorts single words then otherwise); same results, slower.
 * KTJ_CREATE_CUDA12_ARGS prints the "graph id", "graph node id", "channel" and "channel_type" keys
 * of memset rows (ktj_memset_rec), which the reference compiles in for CUDA >= 12 only
 * (CuptiActivity.h:424-458).
 * KTJ_CREATE_NO_STAGE_TIMES leaves the events between the stages of a pass out: ktj_stats then
 * reports the time of the whole pass only (stage_ms[KTJ_STAGE_TOTAL_GPU]), and a trace of a few
 * records is finished a tenth sooner.
 *
 * ktj_destroy leaves what every engine needs before its first record (its stream and events, the
 * small page-locked buffers, 1 MiB of device memory for the inputs of small traces), the 64 MiB of
 * page-locked staging for large submissions if the engine made one, and, while they are small
 * (64 MiB together), the working memory and the document buffer of its last pass behind
 * for the next ktj_create on the same device, which starts from them instead of allocating: one
 * such set per device, held until the process ends.  A trace of a few records otherwise spends
 * more time creating and destroying these than on the GPU.  Nothing is kept of an engine that saw
 * a HIP error.
 * ---------------------------------------------------------------------------------------- */
#define KTJ_CREATE_NO_FILE 0x1u
#define KTJ_CREATE_TILE_EMIT 0x2u
#define KTJ_CREATE_HASH_JOIN 0x4u
#define KTJ_CREATE_PAIR_SORT 0x8u
#define KTJ_CREATE_DISPLAY_NS 0x10u
#define KTJ_CREATE_CUDA12_ARGS 0x20u
#define KTJ_CREATE_NO_STAGE_TIMES 0x40u
int ktj_create(ktj_engine** out, const char* out_path, int64_t base_time_ns, int hip_device,
               uint32_t flags);
void ktj_destroy(ktj_engine* e);
const char* ktj_last_error(const ktj_engine* e);

/* ChromeTraceLogger::handleTraceStart (output_json.cpp:445-479).  meta_kv holds n_kv key/value
 * string pairs (2*n_kv pointers) in the order the caller's metadata map iterates, already merged
 * with the environment metadata (output_json.cpp:433-443). */
int ktj_trace_start(ktj_engine* e, const char* const* meta_kv, size_t n_kv,
                    const char* device_properties);

/* String dictionary: names, arg keys, arg string values, raw fragments.  offsets has n+1
 * entries into blob.  *first_id receives the id of the first string; ids are consecutive. */
int ktj_intern_strings(ktj_engine* e, const char* blob, const uint64_t* offsets, size_t n,
                       uint32_t* first_id);

/* Args schema registration (fields in emission order). */
int ktj_register_schema(ktj_engine* e, const ktj_field* fields, size_t n_fields,
                        uint32_t* schema_id);

/* One record_param_comms op's collective metadata; *index receives the value for the slot of a
 * KTJ_F_COLLECTIVE field.  The strings are copied. */
int ktj_add_collective(ktj_engine* e, const ktj_collective_meta* meta, uint32_t* index);

/* Args blob (8-byte slots) referenced by ktj_generic_rec::args_off.  Appends; *first_slot
 * receives the slot index of the first appended value. */
int ktj_submit_args(ktj_engine* e, const uint64_t* slots, size_t n_slots, uint64_t* first_slot);

/* Runtime API table: RocprofLogger::opString (libkineto/src/RocprofLogger.cpp:751-760) and
 * RuntimeActivity::flowStart (libkineto/src/RocprofActivity_inl.h:185-200).
 * cid_name_ids[cid] = string id of the API name; flow_start_cids lists the cids that start an
 * ac2g flow; malloc_cid is the cid of hipMalloc, whose rows carry a "bytes" arg
 * (RocprofActivity_inl.h:265-277), or KTJ_NONE. */
int ktj_set_api_table(ktj_engine* e, const uint32_t* cid_name_ids, size_t n_cids,
                      const uint32_t* flow_start_cids, size_t n_flow_start, uint32_t malloc_cid);

int ktj_set_clock_model(ktj_engine* e, const ktj_clock_model* model);

/* Capture window for the out-of-range filter (GenericActivityProfiler.cpp:329-340). */
int ktj_set_window(ktj_engine* e, int64_t start_ns, int64_t end_ns);

/* Raw record submission: the bulk equivalent of the per-record handleActivity /
 * handleGenericActivity calls (output_json.cpp:837-971) and of the profiler's per-row handlers
 * (RocmActivityProfiler.cpp:150-213).  `packed` is host memory; the caller may free it when the
 * call returns (the copy to the device is ordered in front of the next pass, not necessarily
 * finished: submissions of up to 64 KiB wait in a page-locked ring and are moved by one kernel
 * launch for many of them; ordinary memory of 16 MiB and more is copied into page-locked chunks by
 * several threads while the copy engine empties others; memory from ktj_host_alloc is copied from
 * directly).  Arrival order is: all generic records, then all runtime rows, then all device
 * rows, each in submission order. */
int ktj_submit_records(ktj_engine* e, int rec_class, const void* packed, size_t n_records);

/* Page-locked host memory for record arrays (no counterpart in the reference, whose rows are heap
 * objects: libkineto/src/RocprofLogger.h:84).  A producer that fills such a buffer and passes it to
 * ktj_submit_records has its records copied to the GPU by DMA straight from the buffer; from ordinary
 * memory the HIP runtime copies through a staging buffer of its own, at about half the rate.  The
 * buffer belongs to the caller until ktj_host_free; it may be reused as soon as ktj_submit_records
 * has returned. */
int ktj_host_alloc(ktj_engine* e, size_t n_bytes, void** host_ptr);
int ktj_host_free(ktj_engine* e, void* host_ptr);

/* Same, for records that already live in device memory of the engine's GPU (zero copy; the
 * buffer must stay valid until ktj_finalize / ktj_process returns). */
int ktj_submit_records_device(ktj_engine* e, int rec_class, const void* device_ptr,
                              size_t n_records);

/* handleDeviceInfo / handleResourceInfo / handleOverheadInfo / handleTraceSpan
 * (output_json.cpp:507-658).  Strings are copied.  ChromeTraceLogger writes each of these events
 * where the call arrives, and libkineto calls arrive in two orders: the buffering logger's replay
 * issues device and resource infos before the activities and spans after them
 * (src/output_membuf.h:91-107), the profiler itself issues resource infos, device infos, GPU spans
 * and overhead infos after the activities (src/GenericActivityProfiler.cpp:178-224, 655-740).  The
 * engine keeps the activities in one sorted section and the other events on either side of it, in
 * call order: what is submitted before the first activity goes in front of the section, what is
 * submitted after it goes behind. */
int ktj_submit_info(ktj_engine* e, int info_kind, const void* info);

/* Tells the engine that the first activity has arrived (see ktj_submit_info).  Every record
 * submission of an activity class does so by itself; a caller that batches its records and
 * submits them later (like the ActivityLogger shim) calls this when it receives the first one. */
int ktj_begin_activities(ktj_engine* e);

/* Runs decode → convert → join → sort → size → scan → emit on the GPU and leaves the finished
 * document in a device buffer.  end_time_ns is finalizeTrace's endTime.  Idempotent inputs: may
 * be called again after more ktj_submit_* calls (everything is re-processed). */
int ktj_process(ktj_engine* e, int64_t end_time_ns);

/* ktj_process for callers that cannot allocate device memory while they run: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same pass and same document as ktj_process, but
 *   - every working buffer is a piece of a static array in device memory that the library holds
 *     once per GPU (KTJ_NOALLOC_SCRATCH_BYTES, until the process ends) instead of an allocation;
 *   - the document is written to out_device, a buffer of out_capacity bytes in device memory of the
 *     engine's GPU, 16-byte aligned, which must hold the document plus 64 bytes;
 *   - the call makes no hipMalloc, hipFree, hipHostMalloc or other allocating HIP call.
 * Records, strings, schemas and infos are submitted before, as for ktj_process (those calls may
 * allocate; ktj_submit_records_device does not).  *n_bytes receives the document's length.
 * KTJ_ERR_LIMIT: the trace needs more working memory than the scratch array holds (roughly
 * 100 000 records; ktj_last_error says how much was asked for), or the output buffer is too small
 * (*n_bytes then holds the document's length), or the trace has user-domain correlation records
 * (KTJ_REC_USERCORR), which this entry point does not take.  All engines on one GPU share that
 * GPU's array and it keeps the last call's contents (the pass clears what it needs cleared):
 * calls that overlap in time on one GPU race and must be serialised by the caller. */
#define KTJ_NOALLOC_SCRATCH_BYTES (64u << 20)
int ktj_process_noalloc(ktj_engine* e, int64_t end_time_ns, void* out_device, uint64_t out_capacity,
                        uint64_t* n_bytes);

/* Device / host views of the finished document (valid until the next ktj_process/destroy). */
int ktj_output_device(ktj_engine* e, const void** device_ptr, uint64_t* n_bytes);
int ktj_output_host(ktj_engine* e, const char** host_ptr, uint64_t* n_bytes); /* pinned; D2H on first call */

/* ChromeTraceLogger::finalizeTrace (output_json.cpp:1023-1028, 1066-1108): ktj_process if not
 * done, D2H, write "<path>.tmp", remove + rename. */
int ktj_finalize(ktj_engine* e, int64_t end_time_ns, uint64_t* bytes_written);

int ktj_get_stats(ktj_engine* e, ktj_stats* out);

/* Library identification; does not touch the GPU. */
const char* ktj_version(void);

#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* KTJ_H_ */
