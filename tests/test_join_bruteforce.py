"""CPU: the oracle's join stage against a literal, sequential Python statement of what the
reference's ROCm post-processing does row by row (dicts in arrival order):
  external correlation   RocmActivityProfiler.cpp:135-148, GenericActivityProfiler.cpp:262, 397-408
  stream back-fill       RocmStreamQueue.h:42-136
  grid/block/bytes       RocprofActivity_inl.h:28-30, 147-180, 208-277 (thread_local maps keyed by int)
  window filter / order  GenericActivityProfiler.cpp:329-340, 363-395
  GPU user annotations   GenericActivityProfiler.cpp:277-327, 423-433 (spans compared as a set: their
                         relative order is the iteration order of the profiler's own maps)
on small synthetic streams and on hand-made streams with duplicate ids, ids that collide after
narrowing, ambiguous queues and out-of-window launch rows."""
import ctypes as C
import struct

import pytest

import oracle_glue as og
from kineto_amd import abi
from stream_builder import B, StreamBuilder


def to_i32(v):
    v &= 0xFFFFFFFF
    return v - (1 << 32) if v >= (1 << 31) else v


def to_i64(v):
    v &= 0xFFFFFFFFFFFFFFFF
    return v - (1 << 64) if v >= (1 << 63) else v


def convert(m, t):
    """x87 expression via ctypes longdouble is not available in Python; reuse exact arithmetic."""
    from fractions import Fraction
    t_ = to_i64(t)
    t0a = to_i64(m.t0_approx)
    if t_ <= t0a:
        return 0
    p = Fraction(float(t_ - t0a)) * Fraction(m.scale)
    if p == 0:
        return m.t0
    e = p.numerator.bit_length() - p.denominator.bit_length()
    if Fraction(2) ** e > p:
        e -= 1
    q = p / Fraction(2) ** (e - 63)
    fl = q.numerator // q.denominator
    rem = q - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return int(Fraction(fl) * Fraction(2) ** (e - 63)) + m.t0


def brute(sp):
    s = sp.contents
    clk = s.clock
    acts = []          # dicts in arrival order, filtered
    counters = dict(out_of_range=0, out_of_order=0)
    activity_map = {}  # int64(int32 id) -> generic index
    for i in range(s.n_generic):
        g = s.generic[i]
        device = g.device
        if g.flags & abi.KTJ_GF_WIDE_DEVICE:  # the slot before the record's values, read as a signed 64-bit value
            device = C.c_int64(s.args[g.args_off - 1]).value
        acts.append(dict(arrival=i, ts=g.start_ns, dur=g.end_ns - g.start_ns, device=device, resource=g.resource,
                         type=g.type, linked=(g.linked_id if g.flags & 2 else None), extra={}))
        activity_map[g.id] = i
    cpu_corr = {}
    for i in range(s.n_extcorr):
        cpu_corr[s.extcorr[i].correlation] = s.extcorr[i].external_id

    def linked(idv):
        ext = cpu_corr.get(to_i32(idv) & 0xFFFFFFFFFFFFFFFF)
        if ext is None:
            return None
        gi = activity_map.get(to_i64(ext))
        return None if gi is None else s.generic[gi].id

    def conv(mode, b, e):
        if mode == 1:
            return convert(clk, b) & 0xFFFFFFFFFFFFFFFF, convert(clk, e) & 0xFFFFFFFFFFFFFFFF
        if mode == 2:
            return (b + clk.async_offset) & 0xFFFFFFFFFFFFFFFF, (e + clk.async_offset) & 0xFFFFFFFFFFFFFFFF
        return b, e

    def oor(ts, dur):
        r = ts < s.window_start_ns or ts + dur > s.window_end_ns
        if r:
            counters["out_of_range"] += 1
        return r

    seen = {}

    def check_order(corr, is_rt, ts):
        if corr not in seen:
            seen[corr] = (is_rt, ts)
            return
        a1, a2 = (is_rt, ts), seen[corr]
        if a2[0]:
            a1, a2 = a2, a1
        if a2[1] == 0:
            return
        if a1[1] > a2[1]:
            counters["out_of_order"] += 1

    # stream back-fill
    stream_by_corr = {}
    for i in range(s.n_runtime):
        r = s.runtime[i]
        sid = r.u.kernel.stream if r.kind == 1 else (r.u.copy.stream if r.kind == 2 else 0)
        if sid:
            stream_by_corr[r.id] = sid
    dstream = [s.device[i].stream for i in range(s.n_device)]
    is_async = [(s.device[i].domain & 0xFFFF) != 2 for i in range(s.n_device)]
    if stream_by_corr:
        for i in range(s.n_device):
            if is_async[i] and dstream[i] == 0 and s.device[i].id in stream_by_corr:
                dstream[i] = stream_by_corr[s.device[i].id]
        by_queue, ambiguous = {}, set()
        for i in range(s.n_device):
            d = s.device[i]
            if not is_async[i] or dstream[i] == 0 or d.queue == 0 or d.queue in ambiguous:
                continue
            if d.queue not in by_queue:
                by_queue[d.queue] = dstream[i]
            elif by_queue[d.queue] != dstream[i]:
                del by_queue[d.queue]
                ambiguous.add(d.queue)
        for i in range(s.n_device):
            d = s.device[i]
            if is_async[i] and dstream[i] == 0 and d.queue in by_queue:
                dstream[i] = by_queue[d.queue]
        idx = {}
        for i in range(s.n_device):
            d = s.device[i]
            if not is_async[i]:
                continue
            if dstream[i]:
                key = dstream[i]
            elif d.queue:
                key = d.queue | (1 << 63)
            else:
                continue
            m = idx.setdefault(d.device, {})
            if key not in m:
                m[key] = len(m) + 1
            dstream[i] = m[key]

    user_corr = {}
    for i in range(s.n_usercorr):
        user_corr[to_i64(s.usercorr[i].correlation)] = to_i64(s.usercorr[i].external_id)
    spans = {}  # (device, resource, annotation id) -> [start, end, generic index], insertion-ordered

    to_grid, to_size = {}, {}
    for i in range(s.n_runtime):
        r = s.runtime[i]
        b, e = conv(clk.runtime_mode, r.begin, r.end)
        ts, dur = to_i64(b), to_i64(e - b)
        lk = linked(r.id)
        check_order(to_i64(r.id), True, ts)
        if oor(ts, dur):
            continue
        extra = {}
        key = to_i32(r.id)
        if r.kind == 1:
            to_grid[key] = (tuple(r.u.kernel.grid), tuple(r.u.kernel.workgroup))
        elif r.kind == 2:
            to_size[key] = r.u.copy.size
        elif r.kind == 3:
            to_size[key] = r.u.malloc_.size
        acts.append(dict(arrival=s.n_generic + i, ts=ts, dur=dur, device=r.pid, resource=r.tid, type=7, linked=lk, extra=extra))
    for i in range(s.n_device):
        d = s.device[i]
        b, e = conv(clk.device_mode, d.begin, d.end)
        dom = d.domain & 0xFFFF                       # the kind of the row; a memset row keeps more in the upper half
        if dom == 2:
            ts, dur, res = to_i64(b), to_i64(e) - to_i64(b), d.stream & 0xFFFFFFFF
        else:
            ts, dur = to_i64(b + 1), to_i64(e - (b + 1))
            res = to_i64(dstream[i] if dstream[i] else d.queue)
        lk = linked(d.id)
        if oor(ts, dur):
            continue
        check_order(to_i64(d.id), False, ts)
        extra = {}
        key = to_i32(d.id)
        if dom != 2:
            if key in to_size:
                extra["bytes"] = to_size[key]
                if (e - b) & 0xFFFFFFFFFFFFFFFF:
                    extra["bw"] = to_size[key] / float((e - b) & 0xFFFFFFFFFFFFFFFF)
            elif key in to_grid:
                extra["grid"], extra["block"] = to_grid[key]
        else:
            extra["bytes"] = d.bytes
            if dur != 0:
                extra["bw"] = d.bytes / float(dur)
        typ = 4 if dom == 2 else (3 if dom == 1 else 5)
        acts.append(dict(arrival=s.n_generic + s.n_runtime + i, ts=ts, dur=dur, device=d.device, resource=res, type=typ,
                         linked=lk, extra=extra))
        ext = user_corr.get(to_i64(d.id)) if s.n_usercorr else None
        gi = activity_map.get(ext) if ext is not None else None
        if gi is not None:
            key = (d.device, res, s.generic[gi].id)
            if key not in spans:
                spans[key] = [ts, ts + dur, gi]
            sp = spans[key]
            if ts < sp[0] or sp[0] == 0:
                sp[0] = ts
            sp[1] = max(sp[1], ts + dur)
    span_acts = [dict(ts=v[0], dur=v[1] - v[0], device=k[0], resource=k[1], type=2, linked=None, corr=k[2],
                      name=s.generic[v[2]].name_id) for k, v in spans.items()]
    return acts, counters, span_acts


def oracle_extra(o, a):
    """bytes / bandwidth / grid / block as the oracle's typed metadata lists them (device rows)."""
    extra = {}
    slot = 0
    for f in range(a.n_fields):
        fd = a.fields[f]
        key = o.string(fd.key_id).decode()
        vals = [a.slots[slot + k] for k in range(fd.count)]
        slot += fd.count
        if a.type in (3, 4, 5):
            if key == "bytes":
                extra["bytes"] = vals[0]
            elif key == "memory bandwidth (GB/s)":
                extra["bw"] = struct.unpack("<d", struct.pack("<Q", vals[0]))[0]
            elif key in ("grid", "block"):
                extra[key] = tuple(vals)
    return extra


def compare(sp):
    want, counters, want_spans = brute(sp)
    o = og.OracleRun(sp)
    acts, n_all = o.activities()
    n = len(want)
    assert n_all == n + len(want_spans)
    # the synthesised spans follow every other activity; compared as a set
    def stream_string(sid):
        s = sp.contents
        return b"" if sid == abi.KTJ_NONE else C.string_at(s.str_blob + s.str_off[sid], s.str_off[sid + 1] - s.str_off[sid])
    got_spans = sorted((acts[i].device, acts[i].resource, acts[i].corr, acts[i].ts, acts[i].dur, acts[i].type,
                        o.string(acts[i].name_id), acts[i].has_linked) for i in range(n, n_all))
    assert got_spans == sorted((w["device"], w["resource"], w["corr"], w["ts"], w["dur"], 2, stream_string(w["name"]), 0)
                               for w in want_spans)
    assert [acts[i].arrival for i in range(n, n_all)] == [sp.contents.n_generic + sp.contents.n_runtime + sp.contents.n_device + k
                                                          for k in range(n_all - n)]
    for i in range(n):
        a, w = acts[i], want[i]
        got = dict(arrival=a.arrival, ts=a.ts, dur=a.dur, device=a.device, resource=a.resource, type=a.type,
                   linked=(a.linked_corr if a.has_linked else None))
        for k, v in got.items():
            assert v == w[k], (i, k, v, w[k])
        if a.type in (3, 4, 5) and a.arrival >= sp.contents.n_generic:
            assert oracle_extra(o, a) == w["extra"], (i, oracle_extra(o, a), w["extra"])
    c = o.counters()
    assert c["out_of_range"] == counters["out_of_range"]
    assert c["out_of_order"] == counters["out_of_order"]
    # canonical order: stable sort by (device, resource, ts)
    order = o.order()
    keys = [(w["device"], w["resource"], w["ts"]) for w in want] + [(acts[i].device, acts[i].resource, acts[i].ts) for i in range(n, n_all)]
    exp = sorted(range(n_all), key=lambda i: keys[i])
    assert order == exp
    o.close()


@pytest.mark.parametrize("cfg,n", [(1, 400), (2, 600), (3, 5000), (4, 1500)])
def test_join_on_small_synthetic_streams(cfg, n):
    sp, release = abi.synth_stream(cfg, n)
    compare(sp)
    release()


@pytest.mark.parametrize("seed", range(16))
def test_join_on_random_streams(seed):
    import random_streams
    compare(random_streams.random_stream(seed, wide_ids=seed % 2 == 1, unique_runtime_ids=seed % 3 == 2).build())


def test_user_annotation_spans():
    import kat_cases
    for case in (kat_cases.case_gpu_user_annotation_reference_test, kat_cases.case_gpu_user_annotations):
        compare(case()[0].build())


def join_edge_case_builder():
    """The hand-made stream of join edge cases (shared with the GPU parity suite)."""
    b = StreamBuilder(window=(B + 100, B + 10**9))
    b.api(["hipLaunchKernel", "hipMemcpyAsync", "hipMalloc", "hipGraphLaunch"], flow_start=[0, 1, 2, 3], malloc_cid=2)
    pid, tid = 10, 11
    b.add_generic("op", 0, B + 200, B + 900, pid, tid, id=5)
    b.add_generic("op", 0, B + 300, B + 400, pid, tid, id=-2)                      # negative id
    b.add_generic("op", 0, B + 300, B + 400, pid, tid, id=5)                       # duplicate id: last wins
    s1, s2 = 0x7000, 0x8000
    b.add_runtime(1, B + 500, B + 600, 0, pid, tid, kind=1, grid=(1, 2, 3), workgroup=(4, 5, 6), stream=s1)
    b.add_runtime(1, B + 700, B + 800, 0, pid, tid, kind=1, grid=(7, 8, 9), workgroup=(1, 1, 1), stream=s2)   # duplicate id
    b.add_runtime(2, B + 10, B + 20, 0, pid, tid, kind=1, grid=(9, 9, 9), workgroup=(9, 9, 9), stream=s1)     # out of window
    b.add_runtime((1 << 32) + 3, B + 510, B + 520, 1, pid, tid, kind=2, size=4096, stream=s2)                    # id beyond 32 bits
    b.add_runtime(4, B + 530, B + 540, 2, pid, tid, kind=3, ptr=0x1000, size=777)                                # malloc writes a size
    b.add_runtime(6, B + 550, B + 560, 3, pid, tid, kind=0)                                                      # graph launch
    b.add_runtime(0xFFFFFFFFFFFFFFFF, B + 570, B + 580, 0, pid, tid, kind=1, grid=(2, 2, 2), workgroup=(3, 3, 3), stream=s1)
    b.add_extcorr(1, 5); b.add_extcorr(3, 5); b.add_extcorr(4, 12345); b.add_extcorr(6, 0xFFFFFFFFFFFFFFFE)
    b.add_extcorr(1, 5); b.add_extcorr(0xFFFFFFFFFFFFFFFF, 5)
    b.add_device(1, B + 900, B + 950, domain=0, name="k", queue=1)                    # stream from last runtime row with id 1
    b.add_device(2, B + 960, B + 970, domain=0, name="k", queue=1)                    # launch row was out of window: no grid
    b.add_device(3, B + 980, B + 990, domain=1, op=2, queue=2)                        # narrowed id 3 matches the copy row
    b.add_device((1 << 32) + 3, B + 1000, B + 1010, domain=1, op=3, queue=2)
    b.add_device(4, B + 1020, B + 1020, domain=0, name="k", queue=3)                  # malloc size, zero raw duration
    b.add_device(6, B + 1030, B + 1040, domain=0, name="k", queue=7)                  # graph kernel, queue fallback
    b.add_device(6, B + 1035, B + 1045, domain=0, name="k", queue=7)
    b.add_device(77, B + 1050, B + 1060, domain=0, name="k", queue=1)                 # queue 1 saw two streams: ambiguous
    b.add_device(78, B + 1070, B + 1080, domain=0, name="k", queue=0)                 # neither stream nor queue
    b.add_device(79, B + 50, B + 60, domain=0, name="k", queue=9)                     # out of window
    b.add_device(80, B + 1090, B + 1100, domain=2, queue=1, stream=5, nbytes=1000)    # memset
    b.add_device(0xFFFFFFFFFFFFFFFF, B + 1110, B + 1120, domain=0, name="k", queue=4, device=1)
    b.add_device(81, 0, B + 1130, domain=0, name="k", queue=4, device=1)              # begin 0
    return b


def test_join_edge_cases():
    compare(join_edge_case_builder().build())


def test_join_without_any_runtime_stream():
    """No runtime row carries a stream: the back-fill returns early and the raw queue is the resource."""
    import kat_cases
    b, _ = kat_cases.case_rocm_sync_trace()
    compare(b.build())


def test_empty_stream():
    b = StreamBuilder()
    compare(b.build())
