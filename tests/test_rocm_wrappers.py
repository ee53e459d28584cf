"""The ROCm wrapper layer (RuntimeActivity<T>, GpuActivity: libkineto/src/RocprofActivity.h:37-162,
RocprofActivity_inl.h:98-299) pinned against the reference's own wrapper code: what those classes
report for a fixed set of rows (oracle/_ref/sdk_ref_driver, mode 3; kept in
tests/golden/rocm_wrapper_rows.txt for machines without the reference) against the checker's
activities and document, and, on the GPU, the engine's document."""
import os

import pytest

import oracle_glue as og
import rocm_wrapper_pattern as rw
import sdk_api_pattern as sp

HAVE_DRIVER = os.path.exists(sp.SDK_REF_DRIVER)


def _flow_start_ops(lines):
    last = [line for line in lines if line.startswith("flowstart_ops=")]
    assert len(last) == 1
    return [int(x) for x in last[0].split("=", 1)[1].split()]


def _all_lines():
    if HAVE_DRIVER:
        import golden.make_rocm_wrapper_golden as mk
        return mk.lines()
    return [line for line in open(rw.GOLDEN).read().split("\n") if line]


def _compare_checker_with_reference(lines, all_rows):
    ref = [rw.parse(line) for line in lines]
    rt, dv, names = all_rows
    assert len(ref) == len(rt) + len(dv)
    sp_ = rw.stream(lines, all_rows).build()
    ora = og.OracleRun(sp_)
    acts, n = ora.activities()
    order = ora.order()
    doc = ora.output()
    assert n == len(ref), "every row is inside the window"
    by_arrival = {int(acts[i].arrival): i for i in range(n)}
    ev = rw.events(doc)
    assert len(ev) == n
    for k, r in enumerate(ref):
        a = acts[by_arrival[k]]
        what = f"{r['what']} row {r['idx']}"
        assert (a.ts, a.dur, a.device, a.resource) == (r["ts"], r["dur"], r["dev"], r["res"]), what
        assert a.type == r["type"] and a.flow_id == r["flowid"] and a.flow_type == r["flowtype"], what
        assert bool(a.flow_start) == bool(r["flowstart"]), what
    # the document: events come in canonical order; position p holds activity order[p]
    for p, e in enumerate(ev):
        a = acts[order[p]]
        r = ref[int(a.arrival)]
        cat, name, pid, tid, ts, dur, args = e
        what = f"{r['what']} row {r['idx']}"
        assert name == r["name"], what
        assert args == r["json"], what
        assert int(pid) == r["dev"] and int(tid) == r["res"], what
    ora.close()


def test_checker_matches_the_reference_wrappers():
    lines = [line for line in _all_lines() if not line.startswith("flowstart_ops=")]
    _compare_checker_with_reference(lines, rw.rows())


@pytest.mark.skipif(not HAVE_DRIVER, reason="oracle/_ref/sdk_ref_driver is built only where the reference's sources are")
@pytest.mark.parametrize("seed", range(12))
def test_stream_backfill_matches_the_reference(seed):
    """The reference's own detail::backfillAsyncStreams (RocmStreamQueue.h:42-136) over seeded rows,
    then its wrappers: the device rows' resourceId and "stream" against the checker's."""
    all_rows = rw.random_rows(seed)
    _compare_checker_with_reference(rw.driver_lines(all_rows, mode=4), all_rows)


def test_flow_start_operations_are_the_references():
    """kineto_amd/csrc/sdk_api_rows.h:is_flow_start against RuntimeActivity<T>::flowStart for every HIP
    runtime operation of the SDK."""
    want = _flow_start_ops(_all_lines())
    got = [op for op in range(sp.n_ops()) if sp.sim().ktjsim_sdk_api_is_flow_start(op)]
    assert got == want and len(got) == 12


@pytest.mark.skipif(not HAVE_DRIVER, reason="oracle/_ref/sdk_ref_driver is built only where the reference's sources are")
def test_wrapper_golden_file_is_what_the_reference_produces():
    import golden.make_rocm_wrapper_golden as mk
    assert mk.lines() == [line for line in open(rw.GOLDEN).read().split("\n") if line]


@pytest.mark.gpu
def test_engine_matches_the_reference_wrappers():
    import test_gpu_parity as tp
    lines = [line for line in _all_lines() if not line.startswith("flowstart_ops=")]
    got = tp._engine_vs_oracle(rw.stream(lines).build())
    ev = rw.events(got)
    ref = [rw.parse(line) for line in lines]
    assert sorted(e[6] or "" for e in ev) == sorted(r["json"] for r in ref)


HAVE_PROFILER_DRIVER = os.path.exists(rw.PROFILER_REF_DRIVER)


def _reference_profiler_run(seed, tmp_path):
    """Runs the reference's processTraceInternal on the seeded case; returns the case, the reference's
    complete and flow events, its counters, and the stream that gives the checker the same input."""
    case = rw.profiler_case(seed)
    info, doc = rw.run_reference_profiler(case, str(tmp_path / "ref_trace.json"))
    ev, fl = rw.events(doc), rw.flow_events(doc)
    marker = [e for e in ev if e[6] and '"correlation": %d,' % rw.MARKER_ID in e[6]]
    assert len(marker) == 1
    marker_begin = case["rows"][1][0][1]
    whole, frac = marker[0][4].split(".")
    shown_ns = int(whole) * 1000 + int(frac)                       # "ts" is microseconds with three decimals
    offset = info["base_time"] + shown_ns - (marker_begin + 1)     # device rows start one nanosecond late
    assert abs(offset) < 4_000_000, "the rows keep 5 ms from the window's edges"
    return case, ev, fl, info, rw.profiler_stream(case, info["base_time"], offset, ev)


@pytest.mark.skipif(not HAVE_PROFILER_DRIVER, reason="oracle/_ref/profiler_ref_driver is built only where the reference's sources are")
@pytest.mark.parametrize("seed", range(8))
def test_checker_matches_the_reference_profiler_loop(seed, tmp_path):
    """The reference's own GenericActivityProfiler::processTraceInternal (with RocmActivityProfiler's
    handlers, RocprofActivityApi::processActivities and the real ChromeTraceLogger) on seeded CPU
    ops, external-correlation pairs, runtime rows and device rows: every complete event and flow
    event it writes, as text, and its two counters against the checker's.  The reference writes in
    call order, the checker in canonical order: the events are compared as sorted lists."""
    case, ev, fl, info, b = _reference_profiler_run(seed, tmp_path)
    ora = og.OracleRun(b.build())
    doc = ora.output()
    cnt = ora.counters()
    ora.close()
    mine_ev, mine_fl = rw.events(doc), rw.flow_events(doc)
    assert sorted(mine_ev) == sorted(ev)
    assert sorted(mine_fl) == sorted(fl)
    assert len(ev) > 150 and len(fl) > 100
    assert cnt["out_of_range"] == info["out_of_range"]
    assert cnt["out_of_order"] == info["out_of_order"]


@pytest.mark.parametrize("seed", (0, 1))
def test_checker_matches_the_committed_profiler_loop_output(seed):
    """The same comparison against tests/golden/profiler_loop_seed<k>.json (written by
    tests/golden/make_profiler_loop_golden.py where the reference is present), for machines without it."""
    import json
    import golden.make_profiler_loop_golden as mk
    g = json.load(open(mk.golden_path(seed)))
    ev, fl = [tuple(e) for e in g["events"]], [tuple(f) for f in g["flows"]]
    b = rw.profiler_stream(rw.profiler_case(seed), g["base_time"], g["device_offset"], ev)
    ora = og.OracleRun(b.build())
    doc = ora.output()
    cnt = ora.counters()
    ora.close()
    assert sorted(rw.events(doc)) == sorted(ev) and sorted(rw.flow_events(doc)) == sorted(fl)
    assert (cnt["out_of_range"], cnt["out_of_order"]) == (g["out_of_range"], g["out_of_order"])


@pytest.mark.gpu
@pytest.mark.parametrize("seed", (0, 1))
def test_engine_matches_the_reference_profiler_loop(seed):
    """The engine's document on the seeded cases: the same events as the reference's own profiler loop
    wrote (committed fixture), the reference's counters, and the checker's bytes."""
    import json
    import golden.make_profiler_loop_golden as mk
    import test_gpu_parity as tp
    from kineto_amd.engine import TraceEngine
    g = json.load(open(mk.golden_path(seed)))
    ev, fl = [tuple(e) for e in g["events"]], [tuple(f) for f in g["flows"]]
    sp_ = rw.profiler_stream(rw.profiler_case(seed), g["base_time"], g["device_offset"], ev).build()
    got = tp._engine_vs_oracle(sp_, base_time_ns=g["base_time"])
    assert sorted(rw.events(got)) == sorted(ev) and sorted(rw.flow_events(got)) == sorted(fl)
    with TraceEngine("t.json", base_time_ns=g["base_time"], device=0) as eng:
        eng.submit_stream(sp_)
        eng.process()
        st = eng.stats()
    assert (st.out_of_range_events, st.gpu_and_cpu_op_out_of_order) == (g["out_of_range"], g["out_of_order"])
