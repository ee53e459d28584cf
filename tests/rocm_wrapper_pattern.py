"""Test-only: a fixed set of ROCm runtime and device rows, what the reference's own activity wrappers
(RuntimeActivity<T>, GpuActivity; libkineto/src/RocprofActivity.h, RocprofActivity_inl.h) report for
them through oracle/_ref/sdk_ref_driver, and the same rows as a stream for the checker and the
engine."""
import os
import re
import struct
import subprocess

from kineto_amd import abi
import sdk_api_pattern as sp
from stream_builder import B, StreamBuilder

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rocm_wrapper_rows.txt")
WIDE = 1 << 32   # two ids this far apart are one key of the reference's int-keyed hand-over maps


def op(name):
    lib = sp.sim()
    lib.ktjsim_sdk_api_op_id.restype = abi.C.c_int64
    lib.ktjsim_sdk_api_op_id.argtypes = [abi.C.c_char_p]
    v = lib.ktjsim_sdk_api_op_id(name.encode())
    assert v >= 0, name
    return v


def rows():
    """(runtime rows, device rows, device names): every row kind, every copy direction, ids shared by
    several runtime rows (the last one hands over), a copy and a launch with one id (size wins over
    grid), ids that coincide after narrowing to int, device rows without a stream or without a
    runtime row, zero-length copies (no bandwidth).  No runtime row carries a stream: the stream
    back-fill (RocmStreamQueue.h), which precedes the wrappers in the profiler and renumbers the
    streams of the device rows, then leaves the device rows' streams as they are."""
    launch, memcpy_async, malloc, free = op("hipLaunchKernel"), op("hipMemcpyAsync"), op("hipMalloc"), op("hipFree")
    sync, graph = op("hipDeviceSynchronize"), op("hipGraphLaunch")
    t = B + 1000
    rt = [
        # (id, begin, end, cid, pid, tid, kind, fields)
        (101, t + 10, t + 20, launch, 4242, 77, 1, dict(grid=(7, 2, 1), workgroup=(256, 1, 1), lds=4096, stream=0)),
        (102, t + 30, t + 45, memcpy_async, 4242, 77, 2, dict(src=0x7000a000, dst=0x7000b000, size=65536, copy_kind=1, stream=0)),
        (103, t + 50, t + 55, malloc, 4242, 78, 3, dict(ptr=0x7000c000, size=1 << 20)),
        (104, t + 60, t + 61, free, 4242, 78, 3, dict(ptr=0x7000c000, size=0)),
        (105, t + 70, t + 90, sync, 4242, 77, 0, {}),
        (106, t + 100, t + 110, launch, 4242, 77, 1, dict(grid=(1, 1, 1), workgroup=(64, 1, 1), lds=0, stream=0)),
        (106, t + 111, t + 120, launch, 4242, 79, 1, dict(grid=(9, 9, 9), workgroup=(32, 2, 2), lds=128, stream=0)),
        (107, t + 130, t + 140, launch, 4242, 77, 1, dict(grid=(3, 1, 1), workgroup=(128, 1, 1), lds=0, stream=0)),
        (107, t + 141, t + 150, memcpy_async, 4242, 77, 2, dict(src=0x10, dst=0x20, size=4096, copy_kind=3, stream=0)),
        (108 + WIDE, t + 160, t + 170, launch, 4242, 77, 1, dict(grid=(5, 5, 1), workgroup=(16, 16, 1), lds=0, stream=0)),
        (109, t + 180, t + 190, graph, 4242, 77, 0, {}),
        (110, t + 200, t + 210, memcpy_async, 4242, 80, 2, dict(src=0, dst=0xffffffffffff, size=0, copy_kind=4, stream=0)),
    ]
    names = ["void gemm<float>(float*, int)", "vector_add", ""]
    dv = [
        # (id, begin, end, domain, op, device, name_id, queue, stream)
        (101, t + 500, t + 700, 0, 0, 0, 0, 11, 3),          # kernel with its launch: grid and block
        (102, t + 710, t + 910, 1, 2, 1, 2, 12, 3),          # HtoD with its copy: bytes and bandwidth
        (106, t + 920, t + 930, 0, 0, 0, 1, 11, 0),          # two launches share the id; stream 0: the queue is the row
        (107, t + 940, t + 960, 1, 4, 0, 2, 12, 5),          # a launch and a copy share the id: bytes, no grid
        (108, t + 970, t + 980, 0, 0, 2, 1, 13, 7),          # the launch's id differs by 2^32: same int key
        (555, t + 990, t + 995, 0, 0, 0, 0, 11, 3),          # no runtime row
        (110, t + 1000, t + 1000, 1, 3, 0, 2, 12, 3),        # begin == end: no bandwidth
        (103, t + 1010, t + 1020, 1, 1, 0, 2, 12, 3),        # HtoH after a malloc of the same id: bytes handed over
        (556, t + 1030, t + 1040, 1, 9, 0, 2, 12, 3),        # unknown copy direction
    ]
    return rt, dv, names


def _runtime_rec(r):
    rid, begin, end, cid, pid, tid, kind, f = r
    x = abi.RuntimeRec()
    x.id, x.begin, x.end, x.cid, x.pid, x.tid, x.kind = rid, begin, end, cid, pid, tid, kind
    if kind == 1:
        for i in range(3):
            x.u.kernel.grid[i] = f["grid"][i]
            x.u.kernel.workgroup[i] = f["workgroup"][i]
        x.u.kernel.group_segment_size, x.u.kernel.stream, x.u.kernel.kernel_name_id = f["lds"], f["stream"], abi.KTJ_NONE
    elif kind == 2:
        x.u.copy.src, x.u.copy.dst, x.u.copy.size = f["src"], f["dst"], f["size"]
        x.u.copy.copy_kind, x.u.copy.stream = f["copy_kind"], f["stream"]
    elif kind == 3:
        x.u.malloc_.ptr, x.u.malloc_.size = f["ptr"], f["size"]
    return x


def _device_rec(d):
    rid, begin, end, domain, opn, device, name_id, queue, stream = d
    x = abi.DeviceRec()
    x.id, x.begin, x.end, x.domain, x.op, x.device, x.name_id, x.queue, x.stream = rid, begin, end, domain, opn, device, name_id, queue, stream
    return x


def random_rows(seed):
    """Seeded rows for the stream back-fill (RocmStreamQueue.h:42-136): runtime rows with and without
    a stream, ids shared between them, device rows with and without a stream on several devices and
    queues (one queue used by two streams: ambiguous), device rows with neither stream nor queue."""
    import random
    rng = random.Random(seed)
    launch, memcpy_async, malloc, sync = op("hipLaunchKernel"), op("hipMemcpyAsync"), op("hipMalloc"), op("hipDeviceSynchronize")
    streams = [0, 0, 0x7f10, 0x7f20, 0x7f30, 0x7f40]
    t = B + 5000
    rt, dv = [], []
    for i in range(80):
        rid = rng.randrange(1, 60)
        kind = rng.choice([0, 1, 1, 1, 2, 2, 3])
        begin = t + 10 * i
        if kind == 1:
            f = dict(grid=(rng.randrange(1, 9), 1, 1), workgroup=(64, 1, 1), lds=0, stream=rng.choice(streams))
            cid = launch
        elif kind == 2:
            f = dict(src=0x1000, dst=0x2000, size=rng.randrange(0, 1 << 20), copy_kind=rng.randrange(0, 5), stream=rng.choice(streams))
            cid = memcpy_async
        elif kind == 3:
            f = dict(ptr=0x3000, size=rng.randrange(0, 1 << 16))
            cid = malloc
        else:
            f, cid = {}, sync
        rt.append((rid, begin, begin + rng.randrange(1, 9), cid, 4242, 70 + rng.randrange(3), kind, f))
    for i in range(160):
        rid = rng.randrange(1, 75)   # some ids have no runtime row
        domain = rng.choice([0, 0, 1])
        begin = t + 2000 + 10 * i
        dv.append((rid, begin, begin + rng.randrange(0, 9), domain, rng.randrange(1, 5) if domain else 0, rng.randrange(3),
                   rng.randrange(2), rng.choice([0, 11, 12, 13, 14, 15]), rng.choice([0, 0, 0, 0x7f10, 0x7f50])))
    return rt, dv, ["kernel_a", "kernel_b"]


def driver_lines(all_rows=None, mode=3):
    rt, dv, names = all_rows or rows()
    req = struct.pack("<IQ", mode, len(rt)) + b"".join(bytes(_runtime_rec(r)) for r in rt)
    req += struct.pack("<Q", len(dv)) + b"".join(bytes(_device_rec(d)) for d in dv)
    req += struct.pack("<Q", len(names)) + b"".join(struct.pack("<I", len(n)) + n.encode() for n in names)
    out = subprocess.run([sp.SDK_REF_DRIVER], input=req, stdout=subprocess.PIPE, check=True, timeout=120).stdout.decode("latin1")
    return [line for line in out.split("\n") if line]


def reference_lines():
    if os.path.exists(sp.SDK_REF_DRIVER):
        return driver_lines()
    return [line for line in open(GOLDEN).read().split("\n") if line]


_LINE = re.compile(r"^(runtime|device) idx=(\d+) corr=(-?\d+) type=(\d+) dev=(-?\d+) res=(-?\d+) ts=(-?\d+) dur=(-?\d+) "
                   r"flowstart=(\d) flowid=(-?\d+) flowtype=(\d+) name=(.*?) json=(.*)$")


def parse(line):
    m = _LINE.match(line)
    assert m, line
    what, idx, corr, typ, dev, res, ts, dur, fs, fid, ft, name, js = m.groups()
    return dict(what=what, idx=int(idx), corr=int(corr), type=int(typ), dev=int(dev), res=int(res), ts=int(ts), dur=int(dur),
                flowstart=int(fs), flowid=int(fid), flowtype=int(ft), name=name, json=js)


def stream(ref, all_rows=None):
    """The same rows as a ktj_stream (no clock conversion, wide window).  The API names and the
    flow-start set are what a caller of the engine provides: the names come from the reference's
    lines, the flow-start operations from kineto_amd/csrc/sdk_api_rows.h."""
    rt, dv, names = all_rows or rows()
    b = StreamBuilder(host_name="wrap")
    n_cids = max(r[3] for r in rt) + 1
    api_names = [None] * n_cids
    for r, line in zip(rt, ref):
        api_names[r[3]] = parse(line)["name"]
    flow = [c for c in range(n_cids) if sp.sim().ktjsim_sdk_api_is_flow_start(c)]
    b.api(api_names, flow_start=flow, malloc_cid=op("hipMalloc"))
    for rid, begin, end, cid, pid, tid, kind, f in rt:
        kw = dict(f)
        if kind == 1:
            kw["kernel_name"] = None
        b.add_runtime(rid, begin, end, cid, pid, tid, kind=kind, **kw)
    for rid, begin, end, domain, opn, device, name_id, queue, stream_ in dv:
        b.add_device(rid, begin, end, domain=domain, op=opn, device=device, name=names[name_id] if names[name_id] else None,
                     queue=queue, stream=stream_)
    return b


_EVENT = re.compile(r'"ph": "X",\n    "cat": "([^"]*)",\n    "name": "(.*)",\n    "pid": (-?\d+),\n    "tid": (-?\d+),\n'
                    r'    "ts": ([0-9.]+),\n    "dur": ([0-9.]+)\n    (?:,\n    "args": \{\n      (.*)\n    \}\n  \},|\n  \},)')


def events(document):
    """(cat, name, pid, tid, ts, dur, args text or None) of every complete event, in document order."""
    return [m.groups() for m in _EVENT.finditer(document.decode("latin1"))]


# ---- the reference's whole post-processing loop (oracle/_ref/profiler_ref_driver) ----
PROFILER_REF_DRIVER = os.path.join(sp.ROOT, "oracle", "_ref", "profiler_ref_driver")


MARKER_ID = 99999   # the first device row: inside the window, its id used by no other row


def profiler_case(seed):
    """CPU ops, external-correlation pairs of both domains, runtime rows and device rows for the
    reference's processTraceInternal: ids linked to existing and to missing CPU ops, rows before,
    across and after the capture window, device rows that start before their launch, ids shared by
    several rows, ids beyond 32 bits.  Times are milliseconds apart and rows keep 5 ms from the
    window's edges (or lie 5 ms and more outside): the reference shifts device rows by a clock
    offset it samples while it runs, known only to within a millisecond beforehand."""
    import random
    rng = random.Random(1000 + seed)
    ms = 1_000_000
    t0 = B + 100 * ms
    window = (t0, t0 + 1000 * ms)
    launch, memcpy_async, malloc, sync = op("hipLaunchKernel"), op("hipMemcpyAsync"), op("hipMalloc"), op("hipDeviceSynchronize")
    names = ["aten::mm", "aten::add", "annotation_a", "gemm_kernel", "copy_kernel", ""]

    def when():   # a start time: mostly inside the window, sometimes well before or after it
        r = rng.random()
        if r < 0.08:
            return t0 - rng.randrange(5 * ms, 50 * ms)
        if r < 0.16:
            return t0 + 1000 * ms + rng.randrange(5 * ms, 50 * ms)
        return t0 + rng.randrange(5 * ms, 900 * ms)

    def length(start):   # rows that start inside end inside, or stick out by 5 ms and more
        if rng.random() < 0.06:
            return (t0 + 1000 * ms - start) + rng.randrange(5 * ms, 20 * ms) if start < t0 + 1000 * ms else 3 * ms
        return rng.randrange(0, 40 * ms)

    cpu_ops, ext, user, rt, dv = [], [], [], [], []
    for i in range(12):
        start = t0 + 6 * ms + 70 * ms * i
        cpu_ops.append(dict(name_id=rng.randrange(2), start=start, end=start + rng.randrange(1 * ms, 60 * ms), id=10 + i, device=4242,
                            resource=77 + (i % 2), type=0))
    for i in range(3):
        start = t0 + 8 * ms + 300 * ms * i
        cpu_ops.append(dict(name_id=2, start=start, end=start + 250 * ms, id=40 + i, device=4242, resource=77, type=1))  # user annotations
    for i in range(70):
        rid = rng.choice([rng.randrange(100, 140), rng.randrange(100, 140) + WIDE * rng.randrange(2)])
        begin = when()
        kind = rng.choice([0, 1, 1, 1, 2, 2, 3])
        if kind == 1:
            f, cid = dict(grid=(rng.randrange(1, 9), 1, 1), workgroup=(64, 1, 1), lds=0, stream=rng.choice([0, 0x7f10, 0x7f20])), launch
        elif kind == 2:
            f, cid = dict(src=0x1000, dst=0x2000, size=rng.randrange(0, 1 << 20), copy_kind=rng.randrange(0, 5), stream=rng.choice([0, 0x7f10])), memcpy_async
        elif kind == 3:
            f, cid = dict(ptr=0x3000, size=rng.randrange(0, 1 << 16)), malloc
        else:
            f, cid = {}, sync
        end = min(begin + length(begin), begin + 30 * ms) if begin >= t0 and begin + 30 * ms < t0 + 995 * ms else begin + length(begin)
        rt.append((rid, begin, end, cid, 4242, 77 + rng.randrange(2), kind, f))
        if rng.random() < 0.7:
            ext.append((rid, rng.choice([10 + rng.randrange(12), 10 + rng.randrange(12), 500 + rng.randrange(5)])))
        if rng.random() < 0.4:
            user.append((rid, 40 + rng.randrange(4)))
    dv.append((MARKER_ID, t0 + 500 * ms, t0 + 501 * ms, 0, 0, 0, 3, 11, 0x7f10))
    for i in range(110):
        rid = rng.randrange(100, 150)
        domain = rng.choice([0, 0, 1])
        begin = when()
        dv.append((rid, begin, begin + length(begin), domain, rng.randrange(1, 5) if domain else 0, rng.randrange(2),
                   3 + rng.randrange(2), rng.choice([0, 11, 12, 13]), rng.choice([0, 0, 0x7f10, 0x7f50])))
    return dict(window=window, cpu_ops=cpu_ops, ext=ext, user=user, rows=(rt, dv, names))


def _generic_rec(o):
    g = abi.GenericRec()
    g.start_ns, g.end_ns, g.resource, g.id, g.device = o["start"], o["end"], o["resource"], o["id"], o["device"]
    g.name_id, g.type, g.schema_id = o["name_id"], o["type"], abi.KTJ_NONE
    return g


def run_reference_profiler(case, path):
    """Runs oracle/_ref/profiler_ref_driver on the case; returns (info dict, trace bytes)."""
    rt, dv, names = case["rows"]
    req = struct.pack("<qq", *case["window"])
    req += struct.pack("<Q", len(case["cpu_ops"])) + b"".join(bytes(_generic_rec(o)) for o in case["cpu_ops"])
    for pairs in (case["ext"], case["user"]):
        req += struct.pack("<Q", len(pairs)) + b"".join(struct.pack("<QQ", c, e) for c, e in pairs)
    req += struct.pack("<Q", len(rt)) + b"".join(bytes(_runtime_rec(r)) for r in rt)
    req += struct.pack("<Q", len(dv)) + b"".join(bytes(_device_rec(d)) for d in dv)
    req += struct.pack("<Q", len(names)) + b"".join(struct.pack("<I", len(n)) + n.encode() for n in names)
    out = subprocess.run([PROFILER_REF_DRIVER, path], input=req, stdout=subprocess.PIPE, stderr=subprocess.PIPE, check=True, timeout=120)
    info = dict(line.split("=", 1) for line in out.stdout.decode().split("\n") if "=" in line)
    return {k: int(v) for k, v in info.items()}, open(path, "rb").read()


_FLOW = re.compile(r'"ph": "([sf])",\n    "id": (-?\d+),\n    "pid": (-?\d+),\n    "tid": (-?\d+),\n    "ts": ([0-9.]+),\n'
                   r'    "cat": "([^"]*)",\n    "name": "([^"]*)"\n    (\n  \},|, "bp": "e"\n  \},)')


def flow_events(document):
    return [m.groups() for m in _FLOW.finditer(document.decode("latin1"))]


def profiler_stream(case, base_time, device_offset, reference_events):
    """The case as a ktj_stream for the checker and the engine: the reference's base time, device
    rows shifted by device_offset (what the reference's clock sampling left over), API names as
    the reference printed them."""
    rt, dv, names = case["rows"]
    b = StreamBuilder(base=base_time, host_name="prof", window=case["window"], end_time=case["window"][1])
    n_cids = max(r[3] for r in rt) + 1
    api_names = [None] * n_cids
    for cat, name, pid, tid, ts, dur, args in reference_events:
        m = re.match(r'"cid": (\d+),', args or "") or re.search(r', "cid": (\d+),', args or "")
        if cat == "cuda_runtime" and m:
            api_names[int(m.group(1))] = name
    for r in rt:   # operations whose rows were all outside the window are not in the trace: any name will do
        if api_names[r[3]] is None:
            api_names[r[3]] = "op%d" % r[3]
    flow = [c for c in range(n_cids) if sp.sim().ktjsim_sdk_api_is_flow_start(c)]
    b.api(api_names, flow_start=flow, malloc_cid=op("hipMalloc"))
    b.clock = abi.ClockModel(0, 0, 1.0, device_offset, 0, 2)   # runtime rows as they are, device rows + offset
    for o in case["cpu_ops"]:
        b.add_generic(names[o["name_id"]], o["type"], o["start"], o["end"], o["device"], o["resource"], id=o["id"])
    for c, e in case["ext"]:
        b.add_extcorr(c, e)
    for c, e in case["user"]:
        b.add_usercorr(c, e)
    for rid, begin, end, cid, pid, tid, kind, f in rt:
        kw = dict(f)
        if kind == 1:
            kw["kernel_name"] = None
        b.add_runtime(rid, begin, end, cid, pid, tid, kind=kind, **kw)
    for rid, begin, end, domain, opn, device, name_id, queue, stream_ in dv:
        b.add_device(rid, begin, end, domain=domain, op=opn, device=device, name=names[name_id] if names[name_id] else None,
                     queue=queue, stream=stream_)
    return b
