"""Python face of the HIP engine: thin ctypes calls into libktj.so (include/ktj.h).

Mirrors how libkineto drives an ActivityLogger: trace start, infos, activities, finalize.  All
work happens in the library; this module only moves pointers.  If libktj.so is missing the
constructor raises.
"""
import ctypes as C

import numpy as np

from . import abi

DBG = dict(ts=0, dur=1, dev=2, res=3, meta=4, ext=5, perm=6, len=7, offs=8, mat=9, sort_keys=10,
           name_view=11, name_off=12, arg_view=13, arg_off=14)
_DBG_DTYPE = dict(ts=np.int64, dur=np.int64, dev=np.int64, res=np.int64, meta=np.uint32, ext=np.int32,
                  perm=np.uint32, len=np.uint32, offs=np.uint64, mat=np.uint8, sort_keys=np.uint64,
                  name_view=np.uint8, name_off=np.uint64, arg_view=np.uint8, arg_off=np.uint64)


class EngineError(RuntimeError):
    pass


class TraceEngine:
    def __init__(self, out_path, base_time_ns=abi.DEFAULT_BASE_TIME_NS, device=0, no_file=True, tile_emit=False, hash_join=False, pair_sort=False, display_ns=False, cuda12_args=False, no_stage_times=False):
        self.lib = abi.load_engine()
        self.h = C.c_void_p()
        flags = (abi.KTJ_CREATE_NO_FILE if no_file else 0) | (abi.KTJ_CREATE_TILE_EMIT if tile_emit else 0) | (abi.KTJ_CREATE_HASH_JOIN if hash_join else 0) | (abi.KTJ_CREATE_PAIR_SORT if pair_sort else 0) | (abi.KTJ_CREATE_DISPLAY_NS if display_ns else 0) | (abi.KTJ_CREATE_CUDA12_ARGS if cuda12_args else 0) | (abi.KTJ_CREATE_NO_STAGE_TIMES if no_stage_times else 0)
        rc = self.lib.ktj_create(C.byref(self.h), out_path.encode(), base_time_ns, device, flags)
        if rc != 0:
            msg = self.lib.ktj_last_error(self.h).decode() if self.h else "allocation failed"
            if self.h:
                self.lib.ktj_destroy(self.h)
                self.h = C.c_void_p()
            raise EngineError(f"ktj_create rc={rc}: {msg}")

    def _chk(self, rc, what):
        if rc != 0:
            raise EngineError(f"{what} rc={rc}: {self.lib.ktj_last_error(self.h).decode()}")

    def submit_stream(self, sp):
        """Feeds one ktj_stream through the C ABI, call by call."""
        s = sp.contents
        lib, h = self.lib, self.h
        self._chk(lib.ktj_trace_start(h, s.meta_kv, s.n_meta, s.device_properties), "ktj_trace_start")
        first = C.c_uint32()
        self._chk(lib.ktj_intern_strings(h, s.str_blob, s.str_off, s.n_strings, C.byref(first)), "ktj_intern_strings")
        for i in range(s.n_schemas):
            d = s.schemas[i]
            sid = C.c_uint32()
            fptr = C.cast(C.addressof(s.fields.contents) + d.first_field * C.sizeof(abi.Field), C.POINTER(abi.Field))
            self._chk(lib.ktj_register_schema(h, fptr, d.n_fields, C.byref(sid)), "ktj_register_schema")
        for i in range(s.n_collectives):
            self._chk(lib.ktj_add_collective(h, C.byref(s.collectives[i]), None), "ktj_add_collective")
        slot0 = C.c_uint64()
        self._chk(lib.ktj_submit_args(h, s.args, s.n_args, C.byref(slot0)), "ktj_submit_args")
        self._chk(lib.ktj_set_api_table(h, s.cid_name_ids, s.n_cids, s.flow_start_cids, s.n_flow_start, s.malloc_cid),
                  "ktj_set_api_table")
        self._chk(lib.ktj_set_clock_model(h, C.byref(s.clock)), "ktj_set_clock_model")
        self._chk(lib.ktj_set_window(h, s.window_start_ns, s.window_end_ns), "ktj_set_window")
        # call order of the buffering logger's replay (libkineto/src/output_membuf.h:91-107): device
        # and resource infos, the activities, then the spans
        for kind, ptr, n in ((abi.INFO_DEVICE, s.device_infos, s.n_device_infos),
                             (abi.INFO_RESOURCE, s.resource_infos, s.n_resource_infos),
                             (abi.INFO_OVERHEAD, s.overhead_infos, s.n_overhead_infos)):
            for i in range(n):
                self._chk(lib.ktj_submit_info(h, kind, C.byref(ptr[i])), "ktj_submit_info")
        self._chk(lib.ktj_begin_activities(h), "ktj_begin_activities")
        for cls, ptr, n in ((abi.REC_GENERIC, s.generic, s.n_generic), (abi.REC_RUNTIME, s.runtime, s.n_runtime),
                            (abi.REC_DEVICE, s.device, s.n_device), (abi.REC_EXTCORR, s.extcorr, s.n_extcorr),
                            (abi.REC_USERCORR, s.usercorr, s.n_usercorr)):
            if n:
                self._chk(lib.ktj_submit_records(h, cls, C.cast(ptr, C.c_void_p), n), "ktj_submit_records")
        for i in range(s.n_spans):
            self._chk(lib.ktj_submit_info(h, abi.INFO_SPAN, C.byref(s.spans[i])), "ktj_submit_info")
        self.end_time_ns = s.end_time_ns

    def process(self, end_time_ns=None):
        self._chk(self.lib.ktj_process(self.h, self.end_time_ns if end_time_ns is None else end_time_ns), "ktj_process")

    def finalize(self, end_time_ns=None):
        n = C.c_uint64()
        rc = self.lib.ktj_finalize(self.h, self.end_time_ns if end_time_ns is None else end_time_ns, C.byref(n))
        self._chk(rc, "ktj_finalize")
        return n.value

    def output(self):
        p, n = C.c_void_p(), C.c_uint64()
        self._chk(self.lib.ktj_output_host(self.h, C.byref(p), C.byref(n)), "ktj_output_host")
        return C.string_at(p, n.value)

    def output_view(self):
        """The finished document as a uint8 numpy view of the engine's pinned host copy (no copy;
        valid until the next process() or close(); works beyond 2 GiB)."""
        p, n = C.c_void_p(), C.c_uint64()
        self._chk(self.lib.ktj_output_host(self.h, C.byref(p), C.byref(n)), "ktj_output_host")
        if n.value == 0:
            return np.zeros(0, dtype=np.uint8)
        return np.ctypeslib.as_array((C.c_ubyte * n.value).from_address(p.value))

    def output_size(self):
        p, n = C.c_void_p(), C.c_uint64()
        self._chk(self.lib.ktj_output_device(self.h, C.byref(p), C.byref(n)), "ktj_output_device")
        return n.value

    def stats(self):
        st = abi.Stats()
        self._chk(self.lib.ktj_get_stats(self.h, C.byref(st)), "ktj_get_stats")
        return st

    def debug(self, what):
        n = C.c_uint64()
        self._chk(self.lib.ktj_debug_fetch(self.h, DBG[what], None, 0, C.byref(n)), "ktj_debug_fetch")
        buf = np.empty(max(n.value, 1), dtype=np.uint8)
        self._chk(self.lib.ktj_debug_fetch(self.h, DBG[what], buf.ctypes.data_as(C.c_void_p), n.value, C.byref(n)),
                  "ktj_debug_fetch")
        return buf[:n.value].view(_DBG_DTYPE[what])

    def close(self):
        if self.h:
            self.lib.ktj_destroy(self.h)
            self.h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()
