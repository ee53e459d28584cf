"""ctypes mirror of include/ktj.h and include/ktj_stream.h, and loaders for the in-tree libraries.

Only plain C structs and function prototypes live here; no computation.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")

KTJ_NONE = 0xFFFFFFFF
KTJ_OK, KTJ_ERR_ARG, KTJ_ERR_STATE, KTJ_ERR_HIP, KTJ_ERR_IO, KTJ_ERR_NOMEM, KTJ_ERR_LIMIT = 0, -1, -2, -3, -4, -5, -6
KTJ_CREATE_NO_FILE = 0x1
KTJ_CREATE_TILE_EMIT = 0x2
KTJ_CREATE_HASH_JOIN = 0x4
KTJ_CREATE_PAIR_SORT = 0x8
KTJ_CREATE_DISPLAY_NS = 0x10
KTJ_CREATE_CUDA12_ARGS = 0x20
KTJ_CREATE_NO_STAGE_TIMES = 0x40
KTJ_GF_WIDE_DEVICE = 0x04

REC_GENERIC, REC_RUNTIME, REC_DEVICE, REC_EXTCORR, REC_USERCORR = 0, 1, 2, 3, 4
INFO_DEVICE, INFO_RESOURCE, INFO_OVERHEAD, INFO_SPAN = 0, 1, 2, 3
F_I64, F_U64, F_F64, F_BOOL, F_STR, F_RAW, F_I64_ARRAY, F_COLLECTIVE, F_STR_ARRAY, F_DICT_BEGIN, F_DICT_END, F_SHAPES, F_UNSUPPORTED = range(13)
SHAPE_LIST = 1 << 32
N_STAGES = 12
STAGE_NAMES = ["dict", "decode", "convert", "join", "sort", "size", "scan", "emit", "d2h", "file",
               "total_gpu", "reserved"]


class GenericRec(C.Structure):
    _fields_ = [("start_ns", C.c_int64), ("end_ns", C.c_int64), ("resource", C.c_int64),
                ("flow_id", C.c_int64), ("args_off", C.c_uint64), ("id", C.c_int32),
                ("device", C.c_int32), ("name_id", C.c_uint32),
                ("linked_id", C.c_int32), ("schema_id", C.c_uint32), ("type", C.c_uint8),
                ("flow_type", C.c_uint8), ("flags", C.c_uint8), ("pad0", C.c_uint8)]


class _RtKernel(C.Structure):
    _fields_ = [("grid", C.c_uint32 * 3), ("workgroup", C.c_uint32 * 3),
                ("group_segment_size", C.c_uint64), ("stream", C.c_uint64),
                ("kernel_name_id", C.c_uint32), ("pad", C.c_uint32)]


class _RtCopy(C.Structure):
    _fields_ = [("src", C.c_uint64), ("dst", C.c_uint64), ("size", C.c_uint64),
                ("stream", C.c_uint64), ("copy_kind", C.c_uint32), ("pad", C.c_uint32)]


class _RtMalloc(C.Structure):
    _fields_ = [("ptr", C.c_uint64), ("size", C.c_uint64)]


class _RtUnion(C.Union):
    _fields_ = [("kernel", _RtKernel), ("copy", _RtCopy), ("malloc_", _RtMalloc),
                ("raw", C.c_uint64 * 7)]


class RuntimeRec(C.Structure):
    _fields_ = [("id", C.c_uint64), ("begin", C.c_uint64), ("end", C.c_uint64),
                ("cid", C.c_uint32), ("pid", C.c_uint32), ("tid", C.c_uint32), ("kind", C.c_uint32),
                ("u", _RtUnion)]


class DeviceRec(C.Structure):
    _fields_ = [("id", C.c_uint64), ("begin", C.c_uint64), ("end", C.c_uint64),
                ("domain", C.c_uint32), ("op", C.c_uint32), ("device", C.c_int32),
                ("name_id", C.c_uint32), ("queue", C.c_uint64), ("stream", C.c_uint64),
                ("bytes", C.c_uint64)]


class MemsetRec(C.Structure):
    """ktj_memset_rec: the KTJ_DOM_MEMSET view of a device row."""
    _fields_ = [("id", C.c_uint64), ("begin", C.c_uint64), ("end", C.c_uint64),
                ("domain", C.c_uint16), ("channel_type", C.c_uint8), ("memory_kind", C.c_uint8),
                ("graph_node_lo", C.c_uint32), ("device", C.c_int32), ("graph_node_hi", C.c_uint32),
                ("context", C.c_uint32), ("channel_id", C.c_uint32), ("stream", C.c_uint32),
                ("graph_id", C.c_uint32), ("bytes", C.c_uint64)]


KTJ_DOM_MEMSET = 2
KTJ_MEMKIND_DEVICE = 3


class ExtCorrRec(C.Structure):
    _fields_ = [("correlation", C.c_uint64), ("external_id", C.c_uint64)]


class Field(C.Structure):
    _fields_ = [("key_id", C.c_uint32), ("type", C.c_uint16), ("count", C.c_uint16)]


class SchemaDesc(C.Structure):
    _fields_ = [("first_field", C.c_uint32), ("n_fields", C.c_uint32)]


class DeviceInfo(C.Structure):
    _fields_ = [("id", C.c_int64), ("sort_index", C.c_int64), ("name", C.c_char_p),
                ("label", C.c_char_p), ("time_ns", C.c_int64)]


class ResourceInfo(C.Structure):
    _fields_ = [("id", C.c_int64), ("sort_index", C.c_int64), ("device_id", C.c_int64),
                ("name", C.c_char_p), ("host_thread", C.c_int32), ("pad", C.c_int32),
                ("time_ns", C.c_int64)]


class OverheadInfo(C.Structure):
    _fields_ = [("name", C.c_char_p), ("time_ns", C.c_int64)]


class TraceSpan(C.Structure):
    _fields_ = [("start_ns", C.c_int64), ("end_ns", C.c_int64), ("op_count", C.c_int32),
                ("iteration", C.c_int32), ("name", C.c_char_p), ("prefix", C.c_char_p)]


COLLECTIVE_KEYS = ("collective_name", "in_msg_nelems", "out_msg_nelems", "group_size", "dtype", "in_tensors_start",
                   "out_tensors_start", "in_split", "out_split", "pg_name", "pg_desc", "group_ranks", "dst_rank",
                   "src_rank", "seq", "comms_id", "rank")


class CollectiveMeta(C.Structure):
    _fields_ = [(k, C.c_char_p) for k in COLLECTIVE_KEYS]


class ClockModel(C.Structure):
    _fields_ = [("t0_approx", C.c_uint64), ("t0", C.c_int64), ("scale", C.c_double),
                ("async_offset", C.c_int64), ("runtime_mode", C.c_uint32),
                ("device_mode", C.c_uint32)]


class Stats(C.Structure):
    _fields_ = [("n_generic", C.c_uint64), ("n_runtime", C.c_uint64), ("n_device", C.c_uint64),
                ("n_extcorr", C.c_uint64), ("n_emitted", C.c_uint64),
                ("out_of_range_events", C.c_uint64), ("gpu_and_cpu_op_out_of_order", C.c_uint64),
                ("n_flow_events", C.c_uint64), ("n_linked", C.c_uint64),
                ("n_blank_names", C.c_uint64), ("output_bytes", C.c_uint64),
                ("activity_bytes", C.c_uint64), ("stage_ms", C.c_float * N_STAGES),
                ("stage_bytes", C.c_uint64 * N_STAGES)]


class Stream(C.Structure):
    _fields_ = [("base_time_ns", C.c_int64), ("trace_name", C.c_char_p),
                ("device_properties", C.c_char_p), ("meta_kv", C.POINTER(C.c_char_p)),
                ("n_meta", C.c_uint64),
                ("str_blob", C.c_void_p), ("str_off", C.POINTER(C.c_uint64)), ("n_strings", C.c_uint64),
                ("fields", C.POINTER(Field)), ("n_fields", C.c_uint64),
                ("schemas", C.POINTER(SchemaDesc)), ("n_schemas", C.c_uint64),
                ("args", C.POINTER(C.c_uint64)), ("n_args", C.c_uint64),
                ("cid_name_ids", C.POINTER(C.c_uint32)), ("n_cids", C.c_uint64),
                ("flow_start_cids", C.POINTER(C.c_uint32)), ("n_flow_start", C.c_uint64),
                ("malloc_cid", C.c_uint32), ("create_flags", C.c_uint32),
                ("clock", ClockModel), ("window_start_ns", C.c_int64), ("window_end_ns", C.c_int64),
                ("end_time_ns", C.c_int64),
                ("generic", C.POINTER(GenericRec)), ("n_generic", C.c_uint64),
                ("runtime", C.POINTER(RuntimeRec)), ("n_runtime", C.c_uint64),
                ("device", C.POINTER(DeviceRec)), ("n_device", C.c_uint64),
                ("extcorr", C.POINTER(ExtCorrRec)), ("n_extcorr", C.c_uint64),
                ("device_infos", C.POINTER(DeviceInfo)), ("n_device_infos", C.c_uint64),
                ("resource_infos", C.POINTER(ResourceInfo)), ("n_resource_infos", C.c_uint64),
                ("overhead_infos", C.POINTER(OverheadInfo)), ("n_overhead_infos", C.c_uint64),
                ("spans", C.POINTER(TraceSpan)), ("n_spans", C.c_uint64),
                ("collectives", C.POINTER(CollectiveMeta)), ("n_collectives", C.c_uint64),
                ("usercorr", C.POINTER(ExtCorrRec)), ("n_usercorr", C.c_uint64)]


class SynthParams(C.Structure):
    _fields_ = [("config", C.c_uint32), ("pad", C.c_uint32), ("n_device", C.c_uint64),
                ("base_time_ns", C.c_int64), ("host_name", C.c_char_p), ("trace_name", C.c_char_p)]


assert C.sizeof(GenericRec) == 64
assert C.sizeof(RuntimeRec) == 96
assert C.sizeof(DeviceRec) == 64
assert C.sizeof(ExtCorrRec) == 16
assert C.sizeof(Field) == 8

DEFAULT_BASE_TIME_NS = 1790857026000000000

_synth = None
_engine = None


def load_synth():
    """libktj_synth.so: the synthetic stream generator (host C, no GPU)."""
    global _synth
    if _synth is None:
        path = os.path.join(LIB_DIR, "libktj_synth.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        lib = C.CDLL(path)
        lib.ktj_synth_generate.restype = C.POINTER(Stream)
        lib.ktj_synth_generate.argtypes = [C.POINTER(SynthParams)]
        lib.ktj_synth_free.restype = None
        lib.ktj_synth_free.argtypes = [C.POINTER(Stream)]
        _synth = lib
    return _synth


ENGINE_SYMBOLS = [
    "ktj_create", "ktj_destroy", "ktj_last_error", "ktj_trace_start", "ktj_intern_strings",
    "ktj_register_schema", "ktj_add_collective", "ktj_submit_args", "ktj_set_api_table", "ktj_set_clock_model",
    "ktj_set_window", "ktj_submit_records", "ktj_submit_records_device", "ktj_host_alloc", "ktj_host_free", "ktj_submit_info", "ktj_begin_activities",
    "ktj_process", "ktj_process_noalloc", "ktj_output_device", "ktj_output_host", "ktj_finalize", "ktj_get_stats",
    "ktj_version",
    # include/ktj_rocprofiler.h
    "ktj_set_sdk_agents", "ktj_set_sdk_kernel_names", "ktj_submit_sdk_buffer", "ktj_submit_sdk_api_record", "ktj_flush",
]


def load_engine():
    """libktj.so: the HIP engine behind the C ABI of include/ktj.h.  Raises if it is not built."""
    global _engine
    if _engine is None:
        path = os.path.join(LIB_DIR, "libktj.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        lib = C.CDLL(path)
        vp = C.c_void_p
        lib.ktj_create.restype = C.c_int
        lib.ktj_create.argtypes = [C.POINTER(vp), C.c_char_p, C.c_int64, C.c_int, C.c_uint32]
        lib.ktj_destroy.restype = None
        lib.ktj_destroy.argtypes = [vp]
        lib.ktj_last_error.restype = C.c_char_p
        lib.ktj_last_error.argtypes = [vp]
        lib.ktj_trace_start.restype = C.c_int
        lib.ktj_trace_start.argtypes = [vp, C.POINTER(C.c_char_p), C.c_size_t, C.c_char_p]
        lib.ktj_intern_strings.restype = C.c_int
        lib.ktj_intern_strings.argtypes = [vp, C.c_void_p, C.POINTER(C.c_uint64), C.c_size_t,
                                           C.POINTER(C.c_uint32)]
        lib.ktj_add_collective.restype = C.c_int
        lib.ktj_add_collective.argtypes = [vp, C.POINTER(CollectiveMeta), C.POINTER(C.c_uint32)]
        lib.ktj_register_schema.restype = C.c_int
        lib.ktj_register_schema.argtypes = [vp, C.POINTER(Field), C.c_size_t, C.POINTER(C.c_uint32)]
        lib.ktj_submit_args.restype = C.c_int
        lib.ktj_submit_args.argtypes = [vp, C.POINTER(C.c_uint64), C.c_size_t, C.POINTER(C.c_uint64)]
        lib.ktj_set_api_table.restype = C.c_int
        lib.ktj_set_api_table.argtypes = [vp, C.POINTER(C.c_uint32), C.c_size_t,
                                          C.POINTER(C.c_uint32), C.c_size_t, C.c_uint32]
        lib.ktj_set_clock_model.restype = C.c_int
        lib.ktj_set_clock_model.argtypes = [vp, C.POINTER(ClockModel)]
        lib.ktj_set_window.restype = C.c_int
        lib.ktj_set_window.argtypes = [vp, C.c_int64, C.c_int64]
        lib.ktj_submit_records.restype = C.c_int
        lib.ktj_submit_records.argtypes = [vp, C.c_int, C.c_void_p, C.c_size_t]
        lib.ktj_submit_records_device.restype = C.c_int
        lib.ktj_submit_records_device.argtypes = [vp, C.c_int, C.c_void_p, C.c_size_t]
        lib.ktj_begin_activities.restype = C.c_int
        lib.ktj_begin_activities.argtypes = [vp]
        lib.ktj_submit_info.restype = C.c_int
        lib.ktj_submit_info.argtypes = [vp, C.c_int, C.c_void_p]
        lib.ktj_set_sdk_agents.restype = C.c_int
        lib.ktj_set_sdk_agents.argtypes = [vp, C.POINTER(C.c_uint64), C.POINTER(C.c_int32), C.c_size_t]
        lib.ktj_set_sdk_kernel_names.restype = C.c_int
        lib.ktj_set_sdk_kernel_names.argtypes = [vp, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32), C.c_size_t, C.c_uint32]
        lib.ktj_submit_sdk_buffer.restype = C.c_int
        lib.ktj_submit_sdk_buffer.argtypes = [vp, C.POINTER(C.c_void_p), C.c_size_t, C.POINTER(C.c_uint64)]
        lib.ktj_host_alloc.restype = C.c_int
        lib.ktj_host_alloc.argtypes = [vp, C.c_size_t, C.POINTER(C.c_void_p)]
        lib.ktj_host_free.restype = C.c_int
        lib.ktj_host_free.argtypes = [vp, C.c_void_p]
        lib.ktj_flush.restype = C.c_int
        lib.ktj_flush.argtypes = [vp]
        lib.ktj_submit_sdk_api_record.restype = C.c_int
        lib.ktj_submit_sdk_api_record.argtypes = [vp, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint32, C.c_uint32,
                                                  C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        lib.ktj_process.restype = C.c_int
        lib.ktj_process.argtypes = [vp, C.c_int64]
        lib.ktj_process_noalloc.restype = C.c_int
        lib.ktj_process_noalloc.argtypes = [vp, C.c_int64, C.c_void_p, C.c_uint64, C.POINTER(C.c_uint64)]
        lib.ktj_output_device.restype = C.c_int
        lib.ktj_output_device.argtypes = [vp, C.POINTER(C.c_void_p), C.POINTER(C.c_uint64)]
        lib.ktj_output_host.restype = C.c_int
        lib.ktj_output_host.argtypes = [vp, C.POINTER(C.c_void_p), C.POINTER(C.c_uint64)]
        lib.ktj_finalize.restype = C.c_int
        lib.ktj_finalize.argtypes = [vp, C.c_int64, C.POINTER(C.c_uint64)]
        lib.ktj_get_stats.restype = C.c_int
        lib.ktj_get_stats.argtypes = [vp, C.POINTER(Stats)]
        lib.ktj_version.restype = C.c_char_p
        lib.ktj_version.argtypes = []
        lib.ktj_debug_fetch.restype = C.c_int
        lib.ktj_debug_fetch.argtypes = [vp, C.c_int, C.c_void_p, C.c_uint64, C.POINTER(C.c_uint64)]
        lib.ktj_debug_force_sort_passes.restype = None
        lib.ktj_debug_force_sort_passes.argtypes = [C.c_int]
        lib.ktj_debug_copy_reference.restype = C.c_int
        lib.ktj_debug_copy_reference.argtypes = [vp, C.c_uint64, C.POINTER(C.c_float)]
        _engine = lib
    return _engine


def synth_stream(config, n_device=0, base_time_ns=DEFAULT_BASE_TIME_NS, host_name=None,
                 trace_name=None):
    """Generates one synthetic stream.  Returns (POINTER(Stream), release callable)."""
    lib = load_synth()
    p = SynthParams()
    p.config = config
    p.n_device = n_device
    p.base_time_ns = base_time_ns
    p.host_name = host_name.encode() if host_name is not None else None
    p.trace_name = trace_name.encode() if trace_name is not None else None
    s = lib.ktj_synth_generate(C.byref(p))
    if not s:
        raise RuntimeError("ktj_synth_generate failed")
    return s, (lambda: lib.ktj_synth_free(s))
