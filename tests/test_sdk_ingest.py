"""rocprofiler-sdk buffer records as device rows (include/ktj_rocprofiler.h).

The record structs come from the SDK's own header (tests/host_sim/sdk_records.cpp builds them).
CPU: the checker's restatement of RocprofLogger::buffer_callback (oracle/sdk_rows.c) against the
reference's own function (libkineto/src/RocprofLogger.cpp:681-749, compiled where it lies into
oracle/_ref/sdk_ref_driver and run on the same records) and against hand-written expectations.
GPU: ktj_submit_sdk_buffer against the checker, end to end."""
import ctypes as C
import os
import struct
import subprocess

import pytest

import oracle_glue as og
from kineto_amd import abi
from stream_builder import B, StreamBuilder

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
AGENT_BASE, KERNEL_BASE = 0xA0000, 0x5000


def _sim():
    lib = C.CDLL(os.path.join(ROOT, "tests", "host_sim", "libktjsim.so"))
    lib.ktjsim_sdk_buffer_create.restype = C.c_void_p
    lib.ktjsim_sdk_buffer_create.argtypes = [C.POINTER(abi.DeviceRec), C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint32, C.c_int]
    lib.ktjsim_sdk_buffer_headers.restype = C.POINTER(C.c_void_p)
    lib.ktjsim_sdk_buffer_headers.argtypes = [C.c_void_p]
    lib.ktjsim_sdk_buffer_count.restype = C.c_uint64
    lib.ktjsim_sdk_buffer_count.argtypes = [C.c_void_p]
    lib.ktjsim_sdk_buffer_free.argtypes = [C.c_void_p]
    return lib


def _oracle_rows(headers, n_headers, agents, kernels, unknown):
    lib = og.load_oracle()
    lib.ktj_oracle_sdk_rows.restype = C.c_uint64
    lib.ktj_oracle_sdk_rows.argtypes = [C.POINTER(C.c_void_p), C.c_uint64, C.POINTER(C.c_uint64), C.POINTER(C.c_int32), C.c_uint64,
                                        C.POINTER(C.c_uint64), C.POINTER(C.c_uint32), C.c_uint64, C.c_uint32, C.POINTER(abi.DeviceRec)]
    ah = (C.c_uint64 * max(len(agents), 1))(*[a for a, _ in agents])
    ad = (C.c_int32 * max(len(agents), 1))(*[d for _, d in agents])
    ki = (C.c_uint64 * max(len(kernels), 1))(*[k for k, _ in kernels])
    kn = (C.c_uint32 * max(len(kernels), 1))(*[v for _, v in kernels])
    out = (abi.DeviceRec * max(n_headers, 1))()
    n = lib.ktj_oracle_sdk_rows(headers, n_headers, ah, ad, len(agents), ki, kn, len(kernels), unknown, out)
    return out, n


def _tables(rows, unknown):
    """Agent and kernel-name tables for rows built by ktjsim_sdk_buffer_create: devices >= 0 are
    listed (device -1 stands for an agent the logger does not know), every name but `unknown` too."""
    agents = sorted({(AGENT_BASE + r.device + 1, r.device) for r in rows if r.device >= 0})
    kernels = sorted({(KERNEL_BASE + r.name_id, r.name_id) for r in rows if r.domain == 0 and r.name_id != unknown})
    return agents, kernels


def _row(**kw):
    r = abi.DeviceRec()
    for k, v in kw.items():
        setattr(r, k, v)
    return r


def test_checker_restatement_on_hand_written_records():
    sim = _sim()
    unknown = 900
    rows = [_row(id=11, begin=1000, end=2000, domain=0, op=1, device=0, name_id=5, queue=77),
            _row(id=12, begin=3000, end=3500, domain=1, op=2, device=1, name_id=123, queue=99, stream=7, bytes=4096),
            _row(id=(1 << 40) + 3, begin=5000, end=5001, domain=0, op=1, device=-1, name_id=unknown, queue=(1 << 63) + 2),
            _row(id=14, begin=0, end=0, domain=1, op=4, device=-1)]
    arr = (abi.DeviceRec * len(rows))(*rows)
    buf = sim.ktjsim_sdk_buffer_create(arr, len(rows), AGENT_BASE, KERNEL_BASE, unknown, 1)
    n_headers = sim.ktjsim_sdk_buffer_count(buf)
    assert n_headers > len(rows)  # records of other kinds and categories are mixed in
    agents, kernels = _tables(rows, unknown)
    out, n = _oracle_rows(sim.ktjsim_sdk_buffer_headers(buf), n_headers, agents, kernels, unknown)
    sim.ktjsim_sdk_buffer_free(buf)
    assert n == 4
    got = [(r.id, r.begin, r.end, r.domain, r.op, r.device, r.name_id, r.queue, r.stream, r.bytes) for r in out[:n]]
    assert got == [
        (11, 1000, 2000, 0, 1, 0, 5, 77, 0, 0),                       # kernel: every field of the dispatch record
        (12, 3000, 3500, 1, 2, 1, abi.KTJ_NONE, 0, 0, 0),             # copy: no name, queue 0, destination agent, no byte count
        ((1 << 40) + 3, 5000, 5001, 0, 1, -1, unknown, (1 << 63) + 2, 0, 0),  # unknown agent and kernel
        (14, 0, 0, 1, 4, -1, abi.KTJ_NONE, 0, 0, 0),
    ]


SDK_REF_DRIVER = os.path.join(ROOT, "oracle", "_ref", "sdk_ref_driver")


def _reference_rows(rows, agents, kernels, unknown, noise):
    """The rocprofAsyncRow objects the reference's buffer_callback makes of the SDK records that
    tests/host_sim/sdk_records.cpp builds from `rows`, as DeviceRec-shaped tuples."""
    req = struct.pack("<IQ", 1, len(rows)) + b"".join(bytes(r) for r in rows)
    req += struct.pack("<QQIIQ", AGENT_BASE, KERNEL_BASE, unknown, noise, len(agents))
    req += b"".join(struct.pack("<Qq", a, d) for a, d in agents)
    req += struct.pack("<Q", len(kernels)) + b"".join(struct.pack("<QQ", k, v) for k, v in kernels)
    out = subprocess.run([SDK_REF_DRIVER], input=req, stdout=subprocess.PIPE, check=True, timeout=120).stdout.decode("latin1")
    lines = out.split("\n")
    kinds = dict(kv.split("=") for kv in lines[0].split()[1:])
    domain_of = {int(kinds["dispatch"]): 0, int(kinds["copy"]): 1}
    got = []
    for line in lines[1:]:
        if not line:
            continue
        head, name = line.split(" name=", 1)
        kind, *kv = head.split()
        assert kind == "async", line
        f = dict(x.split("=") for x in kv)
        if name == "":
            name_id = abi.KTJ_NONE
        elif name == "<unknown kernel>":
            name_id = unknown
        else:
            assert name.startswith("name#"), line
            name_id = int(name[5:])
        assert f["kind"] == f["op"]     # "shared op" placeholder, RocprofLogger.cpp:716-720
        got.append((int(f["id"]), int(f["begin"]), int(f["end"]), domain_of[int(f["domain"])], int(f["op"]), int(f["device"]),
                    name_id, int(f["queue"]), int(f["stream"])))
    return got


@pytest.mark.skipif(not os.path.exists(SDK_REF_DRIVER), reason="oracle/_ref/sdk_ref_driver is not built (needs the reference's sources)")
@pytest.mark.parametrize("case", ["hand", 1, 2, 3, 4])
def test_checker_restatement_matches_the_reference_buffer_callback(case):
    """Pins ktj_oracle_sdk_rows: same SDK records through the reference's RocprofLogger::buffer_callback
    and through the checker's restatement give the same rows, field by field, in the same order;
    records of other kinds and categories are skipped by both."""
    sim = _sim()
    if case == "hand":
        unknown = 900
        rows = [_row(id=11, begin=1000, end=2000, domain=0, op=1, device=0, name_id=5, queue=77),
                _row(id=12, begin=3000, end=3500, domain=1, op=2, device=1, name_id=123, queue=99, stream=7, bytes=4096),
                _row(id=(1 << 40) + 3, begin=5000, end=5001, domain=0, op=1, device=-1, name_id=unknown, queue=(1 << 63) + 2),
                _row(id=(1 << 64) - 1, begin=(1 << 64) - 1, end=0, domain=0, op=0xFFFFFFFF, device=7, name_id=0, queue=(1 << 64) - 1),
                _row(id=14, begin=0, end=0, domain=1, op=4, device=-1),
                _row(id=0, begin=9, end=8, domain=1, op=0, device=3)]
        release = None
    else:
        sp, release, rows, unknown = _sdk_case(case, 4000)
    try:
        arr = (abi.DeviceRec * max(len(rows), 1))(*rows)
        agents, kernels = _tables(rows, unknown)
        for noise in (0, 1):
            want = _reference_rows(rows, agents, kernels, unknown, noise)
            buf = sim.ktjsim_sdk_buffer_create(arr, len(rows), AGENT_BASE, KERNEL_BASE, unknown, noise)
            n_headers = sim.ktjsim_sdk_buffer_count(buf)
            out, n = _oracle_rows(sim.ktjsim_sdk_buffer_headers(buf), n_headers, agents, kernels, unknown)
            got = [(r.id, r.begin, r.end, r.domain, r.op, r.device, r.name_id, r.queue, r.stream) for r in out[:n]]
            sim.ktjsim_sdk_buffer_free(buf)
            assert n == len(rows) == len(want)
            assert got == want
    finally:
        if release:
            release()


def _golden_api_rows():
    """tests/golden/sdk_api_rows.txt (written by tests/golden/make_sdk_api_golden.py from the
    reference's api_callback): per operation id the row line and, for rows that read arguments, the
    SDK's rendering of the call's arguments."""
    lines = open(os.path.join(ROOT, "tests", "golden", "sdk_api_rows.txt")).read().split("\n")
    domain = int(lines[0].split("=")[1])
    rows, k = [], 1
    while k < len(lines) and lines[k]:
        args = None
        if k + 1 < len(lines) and lines[k + 1].startswith("args"):
            args = dict(kv.strip().split("=", 1) for kv in lines[k + 1][4:].split(";") if "=" in kv and "{" not in kv)
            rows.append((lines[k], args))
            k += 2
        else:
            rows.append((lines[k], None))
            k += 1
    return domain, rows


def test_api_callback_rows_match_the_reference_for_every_hip_operation():
    """ktj_submit_sdk_api_record's conversion (kineto_amd/csrc/sdk_api_rows.h) against the rows the
    reference's RocprofLogger::api_callback makes of the same calls: one call of every HIP runtime
    API operation of this SDK, arguments filled with a fixed pattern.  Row class, operation,
    correlation id and every argument the reference keeps must agree; dst, src and ptr, of which the
    reference only keeps a text, must read as that text."""
    import sdk_api_pattern as pat
    domain, golden = _golden_api_rows()
    assert len(golden) == pat.n_ops() > 400
    kinds = {"kernel": 0, "copy": 0, "malloc": 0, "default": 0}
    for op, (want, args) in enumerate(golden):
        got, r = pat.engine_line(op, domain)
        assert got == want, op
        kinds[want.split()[0]] += 1
        if want.startswith("copy"):
            assert ("dst" in args) == (r.u.copy.dst != 0) and ("src" in args) == (r.u.copy.src != 0), op
            for name, value in (("dst", r.u.copy.dst), ("src", r.u.copy.src)):
                if name in args:
                    assert args[name] == hex(value), (op, name)
        if want.startswith("malloc") and "ptr" in args:
            assert args["ptr"] == hex(r.u.malloc_.ptr), op
    assert kinds["kernel"] == 12 and kinds["copy"] == 29 and kinds["malloc"] == 2   # RocprofLogger.cpp:165-245


@pytest.mark.skipif(not os.path.exists(SDK_REF_DRIVER), reason="oracle/_ref/sdk_ref_driver is not built (needs the reference's sources)")
def test_api_callback_golden_file_is_what_the_reference_produces():
    import sdk_api_pattern as pat
    want = open(os.path.join(ROOT, "tests", "golden", "sdk_api_rows.txt")).read().split("\n")
    assert pat.reference_lines() == [line for line in want if line]


def _sdk_case(cfg, n):
    """A synthetic stream whose kernel and copy rows went through SDK records: returns the stream
    with its device rows replaced by the checker's reading of those records, and what the engine
    needs to submit them."""
    sp, release = abi.synth_stream(cfg, n, host_name="box")
    s = sp.contents
    unknown = s.n_strings  # one more string: "<unknown kernel>"
    rows = [s.device[i] for i in range(s.n_device) if s.device[i].domain != 2]
    for k, r in enumerate(rows):
        if k % 11 == 3:
            r.device = -1
        if k % 13 == 5 and r.domain == 0:
            r.name_id = unknown
    return sp, release, rows, unknown


def _with_extra_string(sp, text, keep):
    s = sp.contents
    blob = C.string_at(s.str_blob, s.str_off[s.n_strings]) + text
    offs = (C.c_uint64 * (s.n_strings + 2))(*([s.str_off[i] for i in range(s.n_strings + 1)] + [len(blob)]))
    bb = C.create_string_buffer(blob, len(blob))
    keep += [bb, offs]
    s.str_blob = C.cast(bb, C.c_void_p)
    s.str_off = offs
    s.n_strings += 1


@pytest.mark.gpu
@pytest.mark.parametrize("cfg,n", [(1, 3000), (2, 5000), (3, 20000), (4, 8000)])
def test_sdk_buffer_ingestion_matches_checker(cfg, n):
    from kineto_amd.engine import TraceEngine
    sim = _sim()
    sp, release, rows, unknown = _sdk_case(cfg, n)
    keep = []
    try:
        s = sp.contents
        _with_extra_string(sp, b"<unknown kernel>", keep)
        arr = (abi.DeviceRec * max(len(rows), 1))(*rows)
        buf = sim.ktjsim_sdk_buffer_create(arr, len(rows), AGENT_BASE, KERNEL_BASE, unknown, 1)
        headers, n_headers = sim.ktjsim_sdk_buffer_headers(buf), sim.ktjsim_sdk_buffer_count(buf)
        agents, kernels = _tables(rows, unknown)
        expect_rows, n_rows = _oracle_rows(headers, n_headers, agents, kernels, unknown)
        assert n_rows == len(rows)
        # the checker renders the stream with exactly these device rows
        s.device, s.n_device = C.cast(expect_rows, C.POINTER(abi.DeviceRec)), n_rows
        ora = og.OracleRun(sp)
        want = ora.output()
        ora.close()
        # the engine gets the same stream, but its device rows arrive as SDK buffers (three calls)
        with TraceEngine(s.trace_name.decode(), device=0) as eng:
            s.n_device = 0
            eng.submit_stream(sp)
            s.n_device = n_rows
            lib, h = eng.lib, eng.h
            ah = (C.c_uint64 * max(len(agents), 1))(*[a for a, _ in agents])
            ad = (C.c_int32 * max(len(agents), 1))(*[d for _, d in agents])
            ki = (C.c_uint64 * max(len(kernels), 1))(*[k for k, _ in kernels])
            kn = (C.c_uint32 * max(len(kernels), 1))(*[v for _, v in kernels])
            assert lib.ktj_set_sdk_agents(h, ah, ad, len(agents)) == 0
            assert lib.ktj_set_sdk_kernel_names(h, ki, kn, len(kernels), unknown) == 0
            taken_total, cut = 0, [0, n_headers // 3, n_headers // 2, n_headers]
            for lo, hi in zip(cut, cut[1:]):
                taken = C.c_uint64()
                part = C.cast(C.addressof(headers.contents) + 8 * lo, C.POINTER(C.c_void_p))
                assert lib.ktj_submit_sdk_buffer(h, part, hi - lo, C.byref(taken)) == 0
                taken_total += taken.value
            assert taken_total == n_rows
            eng.process()
            got = eng.output()
        sim.ktjsim_sdk_buffer_free(buf)
        assert got == want
        assert b"<unknown kernel>" in want and b'"pid": -1,' in want
    finally:
        release()


@pytest.mark.gpu
def test_sdk_api_records_end_to_end():
    """HIP runtime API callback records through ktj_submit_sdk_api_record give the document of the
    same calls submitted as packed runtime rows and external-correlation pairs (and the checker's)."""
    import sdk_api_pattern as pat
    from kineto_amd.engine import TraceEngine
    sim = pat.sim()
    golden_domain, golden = _golden_api_rows()
    by_class = {}
    for op, (line, _) in enumerate(golden):
        by_class.setdefault(line.split()[0], []).append(op)
    ops = by_class["kernel"] + by_class["copy"][:8] + by_class["malloc"] + by_class["default"][:5]
    calls = [(ops[k % len(ops)], 1000 + k, B + 1000 * k, B + 1000 * k + 300 + k, 77, 100 + k % 3) for k in range(5 * len(ops))]

    def base_stream():
        b = StreamBuilder()
        b.api(["op%d" % c for c in range(pat.n_ops())], flow_start=by_class["kernel"][:3] + by_class["copy"][:2], malloc_cid=by_class["malloc"][0])
        for k in range(4):
            b.add_generic("cpu_op", 0, B + 10 * k, B + 10 * k + 5, 77, 100, id=500 + k)
        return b

    # the calls as packed rows
    b = base_stream()
    for op, corr, t0, t1, pid, tid in calls:
        r = abi.RuntimeRec()
        sim.ktjsim_sdk_api_row(op, corr, pat.args_bytes(op), t0, t1, pid, tid, C.byref(r))
        r.id = corr
        b.runtime.append(r)
        if corr % 2 == 0:
            b.add_extcorr(corr, 500 + corr % 4)
    sp = b.build()
    ora = og.OracleRun(sp)
    want = ora.output()
    ora.close()
    with TraceEngine(sp.contents.trace_name.decode(), device=0) as eng:
        eng.submit_stream(sp)
        eng.process()
        rows_doc = eng.output()
    assert rows_doc == want
    # the same calls as SDK callback records
    sp2 = base_stream().build()
    with TraceEngine(sp2.contents.trace_name.decode(), device=0) as eng:
        eng.submit_stream(sp2)
        other = sim.ktjsim_sdk_api_record_create(sim.ktjsim_sdk_api_kind_hip_runtime() + 1, 5, 1, pat.args_bytes(5))
        assert eng.lib.ktj_submit_sdk_api_record(eng.h, other, 1, 2, 3, 4, None, None) == 0   # not a HIP runtime API record: ignored
        sim.ktjsim_sdk_api_record_free(other)
        for op, corr, t0, t1, pid, tid in calls:
            rec = sim.ktjsim_sdk_api_record_create(sim.ktjsim_sdk_api_kind_hip_runtime(), op, corr, pat.args_bytes(op))
            ext = C.c_uint64(500 + corr % 4)
            assert eng.lib.ktj_submit_sdk_api_record(eng.h, rec, t0, t1, pid, tid, C.byref(ext) if corr % 2 == 0 else None, None) == 0
            sim.ktjsim_sdk_api_record_free(rec)
        eng.process()
        got = eng.output()
    assert got == want
    assert got.count(b'"cat": "cuda_runtime"') == len(calls)
    # The first half as SDK callback records, the second half as packed rows: the buffered rows reach
    # the device before the packed ones are appended, so arrival order is call order.  The last few
    # calls come as SDK records again and stay buffered: ktj_flush sends them without processing,
    # after which the pass that allocates nothing takes the trace too.
    import torch
    half, tail = len(calls) // 2, len(calls) - 7
    sp3 = base_stream().build()
    with TraceEngine(sp3.contents.trace_name.decode(), device=0) as eng:
        eng.submit_stream(sp3)

        def as_sdk_record(call):
            op, corr, t0, t1, pid, tid = call
            rec = sim.ktjsim_sdk_api_record_create(sim.ktjsim_sdk_api_kind_hip_runtime(), op, corr, pat.args_bytes(op))
            ext = C.c_uint64(500 + corr % 4)
            assert eng.lib.ktj_submit_sdk_api_record(eng.h, rec, t0, t1, pid, tid, C.byref(ext) if corr % 2 == 0 else None, None) == 0
            sim.ktjsim_sdk_api_record_free(rec)

        for call in calls[:half]:
            as_sdk_record(call)
        rows = (abi.RuntimeRec * (tail - half))()
        pairs = []
        for k, (op, corr, t0, t1, pid, tid) in enumerate(calls[half:tail]):
            sim.ktjsim_sdk_api_row(op, corr, pat.args_bytes(op), t0, t1, pid, tid, C.byref(rows[k]))
            rows[k].id = corr
            if corr % 2 == 0:
                pairs.append(abi.ExtCorrRec(corr, 500 + corr % 4))
        assert eng.lib.ktj_submit_records(eng.h, abi.REC_RUNTIME, rows, len(rows)) == 0
        ext_arr = (abi.ExtCorrRec * len(pairs))(*pairs)
        assert eng.lib.ktj_submit_records(eng.h, abi.REC_EXTCORR, ext_arr, len(pairs)) == 0
        for call in calls[tail:]:
            as_sdk_record(call)
        out = torch.zeros(len(want) + 4096, dtype=torch.uint8, device="cuda:0")
        n = C.c_uint64()
        KTJ_ERR_STATE = -2
        assert eng.lib.ktj_process_noalloc(eng.h, eng.end_time_ns, out.data_ptr(), out.numel(), C.byref(n)) == KTJ_ERR_STATE
        assert b"ktj_flush" in eng.lib.ktj_last_error(eng.h)
        assert eng.lib.ktj_flush(eng.h) == 0
        assert eng.lib.ktj_process_noalloc(eng.h, eng.end_time_ns, out.data_ptr(), out.numel(), C.byref(n)) == 0, eng.lib.ktj_last_error(eng.h)
        assert bytes(out[:n.value].cpu().numpy()) == want
        eng.process()
        assert eng.output() == want
