"""Test-only glue: loads the CPU checker (oracle/libktj_oracle.so) and, when it has been built,
the reference's own logger (oracle/_ref/libktj_ref.so).  Product code never imports this."""
import ctypes as C
import os
import socket
import tempfile

from kineto_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_SO = os.path.join(ROOT, "oracle", "libktj_oracle.so")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libktj_ref.so")
SHIM_SO = os.path.join(ROOT, "oracle", "_ref", "libktj_shim_test.so")


class MatActivity(C.Structure):
    _fields_ = [("ts", C.c_int64), ("dur", C.c_int64), ("device", C.c_int64), ("resource", C.c_int64),
                ("corr", C.c_int64), ("flow_id", C.c_int64), ("linked_corr", C.c_int64),
                ("arrival", C.c_uint64), ("slots", C.POINTER(C.c_uint64)),
                ("fields", C.POINTER(abi.Field)), ("n_fields", C.c_uint32), ("name_id", C.c_uint32),
                ("type", C.c_int32), ("flow_type", C.c_int32), ("flow_start", C.c_int32),
                ("has_linked", C.c_int32), ("collective", C.c_uint32), ("pad", C.c_uint32)]


_oracle = None
_ref = None
_shim = None


def load_oracle():
    global _oracle
    if _oracle is None:
        lib = C.CDLL(ORACLE_SO)
        vp = C.c_void_p
        lib.ktj_oracle_run.restype = vp
        lib.ktj_oracle_run.argtypes = [C.POINTER(abi.Stream)]
        lib.ktj_oracle_free.restype = None
        lib.ktj_oracle_free.argtypes = [vp]
        lib.ktj_oracle_output.restype = None
        lib.ktj_oracle_output.argtypes = [vp, C.POINTER(C.c_void_p), C.POINTER(C.c_uint64)]
        lib.ktj_oracle_activities.restype = None
        lib.ktj_oracle_activities.argtypes = [vp, C.POINTER(C.POINTER(MatActivity)), C.POINTER(C.c_uint64)]
        lib.ktj_oracle_order.restype = None
        lib.ktj_oracle_order.argtypes = [vp, C.POINTER(C.POINTER(C.c_uint64)), C.POINTER(C.c_uint64)]
        lib.ktj_oracle_string.restype = None
        lib.ktj_oracle_string.argtypes = [vp, C.c_uint32, C.POINTER(C.c_void_p), C.POINTER(C.c_uint64)]
        lib.ktj_oracle_n_strings.restype = C.c_uint64
        lib.ktj_oracle_n_strings.argtypes = [vp]
        lib.ktj_oracle_counters.restype = None
        lib.ktj_oracle_counters.argtypes = [vp] + [C.POINTER(C.c_uint64)] * 5
        lib.ktj_oracle_timings.restype = None
        lib.ktj_oracle_timings.argtypes = [vp, C.POINTER(C.c_double)]
        lib.ktj_oracle_fmt_double.restype = C.c_size_t
        lib.ktj_oracle_fmt_double.argtypes = [C.c_double, C.c_char_p]
        lib.ktj_oracle_fmt_ts.restype = C.c_size_t
        lib.ktj_oracle_fmt_ts.argtypes = [C.c_int64, C.c_char_p]
        lib.ktj_oracle_convert_ts.restype = C.c_int64
        lib.ktj_oracle_convert_ts.argtypes = [C.POINTER(abi.ClockModel), C.c_uint64]
        lib.ktj_oracle_sanitize_name.restype = C.c_size_t
        lib.ktj_oracle_sanitize_name.argtypes = [C.c_char_p, C.c_size_t, C.c_char_p]
        lib.ktj_oracle_sanitize_str.restype = C.c_size_t
        lib.ktj_oracle_sanitize_str.argtypes = [C.c_char_p, C.c_size_t, C.c_char_p]
        lib.ktj_oracle_type_name.restype = C.c_char_p
        lib.ktj_oracle_type_name.argtypes = [C.c_int]
        _oracle = lib
    return _oracle


def have_ref():
    return os.path.exists(REF_SO)


def load_ref():
    global _ref
    if _ref is None:
        lib = C.CDLL(REF_SO)
        lib.ktj_ref_base_time.restype = C.c_int64
        lib.ktj_ref_render.restype = C.c_int
        lib.ktj_ref_render.argtypes = [C.POINTER(abi.Stream), C.POINTER(MatActivity), C.c_uint64,
                                       C.c_void_p, C.c_void_p, C.c_char_p, C.c_int, C.c_int]
        lib.ktj_ref_fmt_double.restype = C.c_size_t
        lib.ktj_ref_fmt_double.argtypes = [C.c_double, C.c_char_p]
        lib.ktj_ref_metadata_order.restype = C.c_size_t
        lib.ktj_ref_metadata_order.argtypes = [C.POINTER(C.c_char_p), C.c_uint64, C.c_char_p, C.c_size_t]
        lib.ktj_ref_generic_metadata.restype = C.c_size_t
        lib.ktj_ref_generic_metadata.argtypes = [C.c_int, C.POINTER(C.c_char_p), C.POINTER(C.c_int),
                                                 C.POINTER(C.c_int64), C.POINTER(C.c_double),
                                                 C.POINTER(C.c_char_p), C.c_char_p, C.c_size_t]
        _ref = lib
    return _ref


def have_shim():
    return os.path.exists(SHIM_SO)


def load_shim():
    """The ActivityLogger shim (kineto_amd/shim) built against the reference's headers, plus its
    replay driver.  Links the engine library, so it is only loaded where a GPU is present."""
    global _shim
    if _shim is None:
        abi.load_engine()
        lib = C.CDLL(SHIM_SO)
        lib.ktj_shim_base_time.restype = C.c_int64
        lib.ktj_shim_render.restype = C.c_int
        lib.ktj_shim_render.argtypes = [C.POINTER(abi.Stream), C.POINTER(MatActivity), C.c_uint64,
                                        C.c_void_p, C.c_void_p, C.c_char_p, C.c_int, C.POINTER(C.c_uint64), C.c_int, C.c_int, C.c_int]
        _shim = lib
    return _shim


class OracleRun:
    """Runs the oracle on a stream; exposes output bytes, activities and counters."""

    def __init__(self, stream_ptr):
        self.lib = load_oracle()
        self.h = self.lib.ktj_oracle_run(stream_ptr)
        if not self.h:
            raise MemoryError("oracle failed")

    def output(self):
        p, n = C.c_void_p(), C.c_uint64()
        self.lib.ktj_oracle_output(self.h, C.byref(p), C.byref(n))
        return C.string_at(p, n.value)

    def output_view(self):
        """uint8 numpy view of the oracle's document (no copy; works beyond 2 GiB)."""
        import numpy as np
        p, n = C.c_void_p(), C.c_uint64()
        self.lib.ktj_oracle_output(self.h, C.byref(p), C.byref(n))
        if n.value == 0:
            return np.zeros(0, dtype=np.uint8)
        return np.ctypeslib.as_array((C.c_ubyte * n.value).from_address(p.value))

    def activities(self):
        p, n = C.POINTER(MatActivity)(), C.c_uint64()
        self.lib.ktj_oracle_activities(self.h, C.byref(p), C.byref(n))
        return p, n.value

    def order(self):
        p, n = C.POINTER(C.c_uint64)(), C.c_uint64()
        self.lib.ktj_oracle_order(self.h, C.byref(p), C.byref(n))
        return [p[i] for i in range(n.value)]

    def string(self, sid):
        p, n = C.c_void_p(), C.c_uint64()
        self.lib.ktj_oracle_string(self.h, sid, C.byref(p), C.byref(n))
        return C.string_at(p, n.value)

    def counters(self):
        v = [C.c_uint64() for _ in range(5)]
        self.lib.ktj_oracle_counters(self.h, *[C.byref(x) for x in v])
        keys = ["out_of_range", "out_of_order", "n_flow_events", "n_linked", "n_blank_names"]
        return dict(zip(keys, [x.value for x in v]))

    def timings(self):
        t = (C.c_double * 3)()
        self.lib.ktj_oracle_timings(self.h, t)
        return list(t)

    def close(self):
        if self.h:
            self.lib.ktj_oracle_free(self.h)
            self.h = None


def ref_render(stream_ptr, oracle_run, skip_arrival_mod=0, call_order=0, wide_device_mod=0):
    """Renders the stream with the reference's own ChromeTraceLogger, fed with the activities the
    oracle's join stage produced (arrival order; the driver sorts them itself).  skip_arrival_mod >
    0 leaves out every activity whose arrival index is 1 modulo it.  call_order 1: infos and spans
    arrive after the activities, as GenericActivityProfiler issues them (see replay_stream in
    oracle/ref_driver/mat_activity.h).  wide_device_mod > 0: every activity whose arrival index is
    1 modulo it reports a deviceId of 2^40."""
    ref = load_ref()
    acts, n = oracle_run.activities()
    if skip_arrival_mod > 0:
        keep = [i for i in range(n) if acts[i].arrival % skip_arrival_mod != 1]
        kept = (MatActivity * max(len(keep), 1))()
        for j, i in enumerate(keep):
            C.memmove(C.byref(kept, j * C.sizeof(MatActivity)), C.byref(acts[i]), C.sizeof(MatActivity))
        acts, n = kept, len(keep)
    fn = C.cast(load_oracle().ktj_oracle_string, C.c_void_p)
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, stream_ptr.contents.trace_name.decode())
        rc = ref.ktj_ref_render(stream_ptr, acts, n, fn, oracle_run.h, path.encode(), call_order, wide_device_mod)
        if rc != 0:
            raise RuntimeError(f"ktj_ref_render rc={rc}")
        with open(path, "rb") as f:
            data = f.read()
    # The real logger prints the path it was given as "traceName"; the stream carries the bare name.
    return data.replace(path.encode(), stream_ptr.contents.trace_name)


def shim_render(stream_ptr, oracle_run, protocol="gpujson", directory=None, bulk_threads=0, huge_device_mod=0, call_order=0):
    """Renders the stream through the GpuChromeTraceLogger shim obtained from a logger factory by
    URL, fed with the same activities as ref_render, one handleActivity() call each or, with
    bulk_threads > 0, in one handleActivities() call.  huge_device_mod > 0: every activity whose
    arrival index is 1 modulo it reports a deviceId of 2^40.
    Returns (status, bytes or None, dropped)."""
    shim = load_shim()
    acts, n = oracle_run.activities()
    fn = C.cast(load_oracle().ktj_oracle_string, C.c_void_p)
    dropped = C.c_uint64()
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(directory or d, stream_ptr.contents.trace_name.decode())
        url = f"{protocol}://{path}"
        rc = shim.ktj_shim_render(stream_ptr, acts, n, fn, oracle_run.h, url.encode(), 0, C.byref(dropped), bulk_threads, huge_device_mod, call_order)
        data = None
        if rc == 0:
            with open(path, "rb") as f:
                data = f.read()
            assert not os.path.exists(path + ".tmp")
            data = data.replace(path.encode(), stream_ptr.contents.trace_name)
    return rc, data, dropped.value


def ref_stream_args():
    """Stream parameters that make a synthetic stream comparable with the real logger: its base
    time comes from the wall clock and its header carries the machine's host name."""
    return dict(base_time_ns=load_ref().ktj_ref_base_time(), host_name=socket.gethostname())
