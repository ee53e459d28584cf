"""GPU parity: the HIP engine, called through the C ABI, must produce the same bytes as the CPU
checker on the same seeded streams; intermediate stages are compared too so that a failure names
the stage."""
import ctypes as C

import numpy as np
import pytest

from kineto_amd import abi

pytestmark = pytest.mark.gpu

# (1, 10922) and (1, 10923): 32766 and 32769 rows, either side of the single-workgroup scan's limit
CASES = [(1, 10000), (2, 20000), (3, 30000), (4, 30000), (5, 5000), (1, 1), (3, 4097), (5, 3), (1, 10922), (1, 10923)]


def _first_diff(a, b):
    n = min(len(a), len(b))
    x = np.frombuffer(a, dtype=np.uint8, count=n)
    y = np.frombuffer(b, dtype=np.uint8, count=n)
    d = np.nonzero(x != y)[0]
    return int(d[0]) if len(d) else n


def run_case(cfg, n, check_stages=True):
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    sp, release = abi.synth_stream(cfg, n, host_name="gpubox")
    ora = og.OracleRun(sp)
    want = ora.output()
    acts, n_acts = ora.activities()
    order = ora.order()
    with TraceEngine(sp.contents.trace_name.decode(), device=0) as eng:
        eng.submit_stream(sp)
        eng.process()
        st = eng.stats()
        if check_stages:
            arrival = np.array([acts[i].arrival for i in range(n_acts)], dtype=np.int64)
            meta = eng.debug("meta")
            valid = (meta >> 9) & 1
            assert int(valid.sum()) == n_acts, "window filter: number of surviving rows"
            assert np.array_equal(np.nonzero(valid)[0], arrival), "window filter: which rows survive"
            for col, field in (("ts", "ts"), ("dur", "dur"), ("dev", "device"), ("res", "resource")):
                got = eng.debug(col)[arrival]
                exp = np.array([getattr(acts[i], field) for i in range(n_acts)], dtype=np.int64)
                bad = np.nonzero(got != exp)[0]
                assert len(bad) == 0, f"column {col}: first mismatch at activity {bad[:5]} got {got[bad[:5]]} want {exp[bad[:5]]}"
            perm = eng.debug("perm")[:n_acts].astype(np.int64)
            exp_perm = arrival[np.array(order, dtype=np.int64)] if n_acts else np.zeros(0, dtype=np.int64)
            bad = np.nonzero(perm != exp_perm)[0]
            assert len(bad) == 0, f"sort: first mismatch at position {bad[:5]}: got {perm[bad[:5]]} want {exp_perm[bad[:5]]}"
            cnt = ora.counters()
            assert st.out_of_range_events == cnt["out_of_range"]
            assert st.gpu_and_cpu_op_out_of_order == cnt["out_of_order"]
            assert st.n_flow_events == cnt["n_flow_events"]
            assert st.n_linked == cnt["n_linked"]
        got = eng.output()
    # the output-partitioned emit kernel and hash-mode join tables must produce the same document
    with TraceEngine(sp.contents.trace_name.decode(), device=0, tile_emit=True, hash_join=True, pair_sort=True) as eng:
        eng.submit_stream(sp)
        eng.process()
        st_hash = eng.stats()
        got_tile = eng.output()
        if check_stages:
            assert np.array_equal(eng.debug("perm")[:n_acts].astype(np.int64), perm), "pair sort and word sort disagree"
    if check_stages:  # hash-mode join tables: same counters as the direct-addressed ones
        assert st_hash.gpu_and_cpu_op_out_of_order == st.gpu_and_cpu_op_out_of_order and st_hash.n_linked == st.n_linked
    ora.close()
    release()
    if got_tile != want:
        i = _first_diff(got_tile, want)
        raise AssertionError(f"tile emit + hash join: byte {i} of {len(want)}: got {got_tile[max(0, i - 60):i + 60]!r} want {want[max(0, i - 60):i + 60]!r}")
    if got != want:
        i = _first_diff(got, want)
        raise AssertionError(f"config {cfg} n={n}: bytes differ at {i} (got {len(got)} bytes, want {len(want)}):\n"
                             f"GOT : {got[max(0, i - 200):i + 120]!r}\nWANT: {want[max(0, i - 200):i + 120]!r}")
    return st


@pytest.mark.parametrize("cfg,n", CASES)
def test_engine_matches_oracle(cfg, n):
    print(f"case config={cfg} n={n}", flush=True)
    run_case(cfg, n)


def _engine_vs_oracle(sp, check_substrings=(), **engine_options):
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    ora = og.OracleRun(sp)
    want = ora.output()
    # the create flags that change the document travel with the stream (the checker reads them there)
    engine_options.setdefault("cuda12_args", bool(sp.contents.create_flags & abi.KTJ_CREATE_CUDA12_ARGS))
    with TraceEngine(sp.contents.trace_name.decode(), device=0, **engine_options) as eng:
        eng.submit_stream(sp)
        eng.process()
        got = eng.output()
        st = eng.stats()
    cnt = ora.counters()
    ora.close()
    if got != want:
        i = _first_diff(got, want)
        raise AssertionError(f"bytes differ at {i}:\nGOT : {got[max(0, i - 200):i + 120]!r}\nWANT: {want[max(0, i - 200):i + 120]!r}")
    for sub in check_substrings:
        assert sub.encode("latin1") in got
    assert st.out_of_range_events == cnt["out_of_range"]
    assert st.gpu_and_cpu_op_out_of_order == cnt["out_of_order"]
    return got


def test_known_answer_cases_on_gpu():
    import kat_cases
    for case in kat_cases.SUBSTRING_CASES:
        print("case", case.__name__, flush=True)
        b, expect = case()
        _engine_vs_oracle(b.build(), expect)
    b, counts = kat_cases.case_rocm_sync_trace()
    got = _engine_vs_oracle(b.build()).decode("latin1")
    for k, v in counts.items():
        assert got.count(k) == v


@pytest.mark.parametrize("seed", range(24))
def test_random_streams_on_gpu(seed):
    """Every record class, activity type and edge value, mixed at random (tests/random_streams.py),
    with direct-addressed and with hash-mode join tables and both emit kernels."""
    import random_streams
    print(f"random stream seed={seed}", flush=True)
    sp = random_streams.random_stream(seed, wide_ids=seed % 2 == 1, unique_runtime_ids=seed % 3 == 2).build()
    _engine_vs_oracle(sp)
    _engine_vs_oracle(sp, hash_join=True, tile_emit=True, pair_sort=True)


@pytest.mark.parametrize("cfg,n", [(3, 20000), (4, 6000), (2, 9000)])
def test_user_annotation_spans_at_scale(cfg, n):
    """Thousands of GPU user-annotation spans: every external-correlation record of a synthetic stream
    is also submitted in the user domain, so each (stream, CPU op) pair with kernels gets a span."""
    print(f"user annotation spans cfg={cfg} n={n}", flush=True)
    sp, release = abi.synth_stream(cfg, n, host_name="box")
    try:
        s = sp.contents
        s.usercorr, s.n_usercorr = s.extcorr, s.n_extcorr
        _engine_vs_oracle(sp, check_substrings=('"cat": "gpu_user_annotation"',))
        _engine_vs_oracle(sp, hash_join=True)
    finally:
        release()


def test_join_edge_cases_on_gpu():
    import test_join_bruteforce as tj
    got = _engine_vs_oracle(tj.join_edge_case_builder().build())
    assert got.count(b'"ph": "X"') == 20   # every in-window row of the hand-made stream printed


KTJ_MAX_STREAM_PAIRS, KTJ_MAX_QUEUES, KTJ_MAX_SYNC_ROWS = 4096, 32768, 32768   # include/ktj.h


def _many_ids_builder(n_resources, n_devices, n_streams=0, n_queues=0, n_sync_rows=0):
    """CPU ops on n_resources distinct threads of n_devices distinct processes (ids spread over the
    whole signed 64-bit / 32-bit range, arrival order scrambled), plus optional device rows on
    n_streams distinct streams or n_queues distinct queues, plus n_sync_rows Stream Sync events on
    distinct rows."""
    from stream_builder import StreamBuilder, B
    b = StreamBuilder(host_name="many")
    b.api(["hipLaunchKernel"], flow_start=[0])
    n = max(n_resources, n_devices)
    for i in range(n):
        j = (i * 7919) % n
        res = ((j % n_resources) * 0x9E3779B97F4A7C15 + 12345) % (1 << 64) - (1 << 63)
        dev = (((j % n_devices) * 0x45D9F3B + 77) % (1 << 32)) - (1 << 31)
        b.add_generic("op%d" % (i % 5), 0, B + 1000 + 13 * ((i * 31) % n), B + 1500 + 13 * ((i * 31) % n), dev, res, id=i + 1)
    for i in range(max(n_streams, n_queues)):
        b.add_runtime(10**6 + i, B + 5000 + i, B + 5400 + i, 0, 1, 1, kind=1, stream=(0x7000 + 8 * i) if n_streams else 0)
        b.add_device(10**6 + i, B + 6000 + i, B + 6300 + i, domain=0,
                     device=i % 3, name="k%d" % (i % 4), queue=0x100 + i)
    for i in range(n_sync_rows):
        b.add_generic("Stream Sync", 15, B + 9000 + i, B + 9100 + i, 0, 1000 + i, id=2 * 10**6 + i)
    return b


def _queue_limit_builder(n_queues):
    """Device rows on n_queues distinct hardware queues in a trace where the queue -> stream table is
    used: one runtime row carries a stream, one device row has neither a stream nor a runtime row."""
    from stream_builder import StreamBuilder, B
    b = StreamBuilder(host_name="queues")
    b.api(["hipLaunchKernel"], flow_start=[0])
    b.add_runtime(1, B + 5000, B + 5400, 0, 1, 1, kind=1, stream=0x7000)
    b.add_device(1, B + 6000, B + 6300, domain=0, device=0, name="k", queue=0x100)
    b.add_device(5, B + 6400, B + 6500, domain=0, device=0, name="k", queue=0x100)      # takes its queue's stream
    for i in range(1, n_queues):
        b.add_device(10**6 + i, B + 7000 + i, B + 7300 + i, domain=i % 2, op=2 * (i % 2), device=0, name="k%d" % (i % 4),
                     queue=0x100 + i, stream=0x7000 + 8 * (i % 5))
    return b


def test_more_distinct_ids_than_the_rank_sets_hold():
    """Above 4096 distinct resourceId or deviceId values the sort works on the raw values: same bytes
    as the checker, no error."""
    for n_res, n_dev in ((5000, 3), (300, 4200), (20000, 4500)):
        print(f"distinct ids: {n_res} resources, {n_dev} devices", flush=True)
        _engine_vs_oracle(_many_ids_builder(n_res, n_dev).build())


def test_limits_end_in_a_named_error():
    """A trace beyond one of the engine's documented limits is refused with KTJ_ERR_LIMIT and a text
    that names the limit (include/ktj.h: KTJ_MAX_*)."""
    from kineto_amd.engine import TraceEngine, EngineError
    for make, limit, name in ((lambda n: _many_ids_builder(10, 1, n_streams=n), KTJ_MAX_STREAM_PAIRS, "KTJ_MAX_STREAM_PAIRS"),
                              (_queue_limit_builder, KTJ_MAX_QUEUES, "KTJ_MAX_QUEUES"),
                              (lambda n: _many_ids_builder(10, 1, n_sync_rows=n), KTJ_MAX_SYNC_ROWS, "KTJ_MAX_SYNC_ROWS")):
        # the limits are counts of distinct keys: one key more is refused, however the keys hash
        for n in (limit + 1, limit + 200):
            print("limit", name, n, flush=True)
            sp = make(n).build()
            with TraceEngine("t.json", device=0) as eng:
                eng.submit_stream(sp)
                with pytest.raises(EngineError) as ei:
                    eng.process()
                assert "rc=%d" % abi.KTJ_ERR_LIMIT in str(ei.value) and name in str(ei.value)
                assert eng.lib.ktj_process(eng.h, eng.end_time_ns) == abi.KTJ_ERR_LIMIT   # and again: every kernel ended normally
        # exactly at the limit: accepted and identical to the checker
        print("at the limit", name, flush=True)
        _engine_vs_oracle(make(limit).build())


def test_header_text_beyond_the_pinned_staging_buffer():
    """Thousands of resource infos make the text around the activities larger than the engine's
    256 KiB pinned staging buffer: the buffer grows and the text still lands byte for byte
    (both pieces, whatever the alignment of the place after the activities)."""
    from stream_builder import StreamBuilder, B
    for extra in (0, 1, 7, 9):  # shifts the suffix to different positions modulo 16
        print(f"large header, name length +{extra}", flush=True)
        b = StreamBuilder(host_name="big" + "x" * extra)
        b.api(["hipLaunchKernel"], flow_start=[0])
        for k in range(4000):
            b.add_resource_info(100 + k, 100 + k, 7, "worker thread %d" % k, host_thread=(k % 2 == 0))
        for k in range(50):
            b.add_generic("op%d" % (k % 3), 0, B + 1000 + 10 * k, B + 1005 + 10 * k, 7, 100 + k, id=k + 1)
        b.add_span(B, B + 10**6, 50, 0, "PyTorch Profiler")
        _engine_vs_oracle(b.build())


def test_document_longer_than_the_first_guess_of_its_buffer():
    """An engine's first pass allocates the document's buffer from a guess (rows times the fixed text
    of an event plus one string of average length) before the lengths are known.  Here every device
    row carries the one long name of a dictionary of short strings, so the document is several times
    the guess and the buffer has to be allocated again; a second pass on the same engine then finds
    the buffer large enough.  Both documents must be the oracle's."""
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    from stream_builder import StreamBuilder, B
    b = StreamBuilder(host_name="guess")
    ids, plain_s = {}, b.s
    b.s = lambda text: ids[text] if text in ids else ids.setdefault(text, plain_s(text))  # one dictionary entry per text
    b.api(["hipLaunchKernel"], flow_start=[0])
    long_name = "void long_kernel<" + ", ".join("T%d" % k for k in range(400)) + ">(int)"
    assert len(long_name) > 2000
    for k in range(3000):  # many short strings: the average stays small
        b.add_generic("op%d" % k, 0, B + 1000 + 10 * k, B + 1005 + 10 * k, 7, 100 + (k % 4), id=k + 1)
    for k in range(6000):
        b.add_runtime(10 + k, B + 2000 + 20 * k, B + 2010 + 20 * k, 0, 7, 100 + (k % 4), kind=1, stream=1 + k % 3)
        b.add_device(10 + k, B + 2020 + 20 * k, B + 2030 + 20 * k, domain=0, device=0, name=long_name, queue=1 + k % 3, stream=0)
    b.add_span(B, B + 10**6, 50, 0, "PyTorch Profiler")
    sp = b.build()
    ora = og.OracleRun(sp)
    want = ora.output()
    ora.close()
    assert len(want) > 6000 * 2000
    with TraceEngine(sp.contents.trace_name.decode(), device=0) as eng:
        eng.submit_stream(sp)
        for attempt in range(2):
            print(f"document of {len(want)} bytes, pass {attempt}", flush=True)
            eng.process()
            got = eng.output()
            assert got == want, f"pass {attempt}: bytes differ at {_first_diff(got, want)}"


def test_golden_digests_on_gpu():
    """The engine's document against the committed digests (tests/golden/digests.json, written where
    the checker's output had just been compared byte for byte with the reference logger's): no
    checker takes part in this comparison."""
    import hashlib
    import json
    import os
    from kineto_amd.engine import TraceEngine
    here = os.path.dirname(os.path.abspath(__file__))
    gold = json.load(open(os.path.join(here, "golden", "digests.json")))
    assert len(gold) == 5
    for key, g in sorted(gold.items()):
        cfg, n = (int(x) for x in key.split(":"))
        print("golden", key, flush=True)
        sp, release = abi.synth_stream(cfg, n, host_name="golden", trace_name="golden.json")
        for opts in ({}, {"tile_emit": True, "hash_join": True, "pair_sort": True}):
            with TraceEngine(sp.contents.trace_name.decode(), device=0, **opts) as eng:
                eng.submit_stream(sp)
                eng.process()
                got = eng.output()
            assert len(got) == g["output_bytes"], key
            assert hashlib.sha256(got).hexdigest() == g["output_sha256"], key
        release()


def test_display_unit_switch():
    """KTJ_CREATE_DISPLAY_NS is the reference's DISPLAY_TRACE_IN_NS build switch (output_json.cpp:451-454):
    one word of the header changes."""
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    sp, release = abi.synth_stream(1, 300, host_name="unit")
    ora = og.OracleRun(sp)
    want = ora.output()
    ora.close()
    with TraceEngine(sp.contents.trace_name.decode(), device=0, display_ns=True) as eng:
        eng.submit_stream(sp)
        eng.process()
        got = eng.output()
    release()
    assert want.count(b'"displayTimeUnit": "ms"') == 1
    assert got == want.replace(b'"displayTimeUnit": "ms"', b'"displayTimeUnit": "ns"')


def test_empty_and_tiny_streams_on_gpu():
    from stream_builder import StreamBuilder, B
    _engine_vs_oracle(StreamBuilder().build())
    b = StreamBuilder()
    b.add_generic(None, 0, B, B, 0, 0)          # no name, zero everything
    _engine_vs_oracle(b.build())
    b = StreamBuilder(window=(B + 10, B + 20))
    b.api(["hipLaunchKernel"], flow_start=[0])
    b.add_runtime(1, B, B + 5, 0, 1, 1, kind=1)  # everything filtered out by the window
    b.add_device(1, B + 100, B + 200, name="k", queue=1)
    _engine_vs_oracle(b.build())


def test_small_traces_through_the_passes_of_a_large_one():
    """A trace of up to 4096 rows is sorted by one launch of one workgroup; with that switched off it
    takes the key and scatter launches of a large trace.  Both forms, on the smallest cases, the
    known-answer cases, a tile that is exactly full and one row more, and seeded
    random streams: same permutation, same document."""
    import kat_cases
    import random_streams
    lib = abi.load_engine()
    sizes = [(1, 1), (5, 3), (1, 1365), (1, 1366), (3, 1300), (4, 1000), (2, 900)]   # (1, 1365): 4095 rows; (1, 1366): 4098
    try:
        for forced in (1, 0):
            lib.ktj_debug_force_sort_passes(forced)
            for cfg, n in sizes:
                print(f"forced={forced} config={cfg} n={n}", flush=True)
                run_case(cfg, n)
            for case in kat_cases.SUBSTRING_CASES:
                print(f"forced={forced} case {case.__name__}", flush=True)
                b, expect = case()
                _engine_vs_oracle(b.build(), expect)
            for seed in (3, 11, 14):
                sp = random_streams.random_stream(seed, wide_ids=seed % 2 == 1, unique_runtime_ids=seed % 3 == 2).build()
                _engine_vs_oracle(sp)
    finally:
        lib.ktj_debug_force_sort_passes(0)


def test_process_is_repeatable_and_file_output(tmp_path):
    import hashlib
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    path = str(tmp_path / "trace.json")
    sp, release = abi.synth_stream(2, 5000, host_name="gpubox", trace_name=path)
    ora = og.OracleRun(sp)
    want = ora.output()
    ora.close()
    with TraceEngine(path, device=0, no_file=False) as eng:
        eng.submit_stream(sp)
        eng.process()
        a = eng.output()
        eng.process()
        b = eng.output()
        assert a == b == want
        import os
        assert os.path.exists(path + ".tmp") and not os.path.exists(path)
        n = eng.finalize()
        assert n == len(want)
        assert not os.path.exists(path + ".tmp")
        assert open(path, "rb").read() == want
    release()


def test_file_output_of_a_document_of_several_staging_chunks(tmp_path):
    """The file sink streams the document through pinned staging buffers, one chunk being copied
    while the previous one is written: a document of several chunks (and a ragged last one) must
    reach the file byte for byte, and a second trace through the same engine settings too."""
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    for n_dev in (60000, 17000):
        path = str(tmp_path / f"trace_{n_dev}.json")
        sp, release = abi.synth_stream(3, n_dev, host_name="gpubox", trace_name=path)
        ora = og.OracleRun(sp)
        want = ora.output()
        ora.close()
        with TraceEngine(path, device=0, no_file=False) as eng:
            eng.submit_stream(sp)
            n = eng.finalize()
        release()
        assert n == len(want)
        if n_dev == 60000:
            assert n > 3 * (16 << 20)
        with open(path, "rb") as f:
            assert f.read() == want


def test_unwritable_sink_is_a_silent_noop():
    """ChromeTraceLogger with a file it cannot open: every handler returns silently and only
    finalizeTrace reports (output_json.cpp:485-505, 1067-1070)."""
    from kineto_amd.engine import TraceEngine, EngineError
    sp, release = abi.synth_stream(1, 100)
    eng = TraceEngine("/nonexistent-dir/sub/trace.json", device=0, no_file=False)
    eng.submit_stream(sp)        # no error
    eng.process()                # no error, nothing done
    with pytest.raises(EngineError) as ei:
        eng.finalize()
    assert "rc=-4" in str(ei.value)
    eng.close()
    release()


def test_device_resident_submission():
    """Records handed over as device pointers (zero copy) give the same document."""
    import torch
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    sp, release = abi.synth_stream(3, 20000, host_name="gpubox")
    s = sp.contents
    ora = og.OracleRun(sp)
    want = ora.output()
    ora.close()
    keep = []

    def to_dev(ptr, n, size):
        raw = C.string_at(C.cast(ptr, C.c_void_p), n * size)
        t = torch.frombuffer(bytearray(raw), dtype=torch.uint8).cuda()
        keep.append(t)
        return t.data_ptr()

    devptrs = {abi.REC_GENERIC: (to_dev(s.generic, s.n_generic, 64), s.n_generic),
               abi.REC_RUNTIME: (to_dev(s.runtime, s.n_runtime, 96), s.n_runtime),
               abi.REC_DEVICE: (to_dev(s.device, s.n_device, 64), s.n_device),
               abi.REC_EXTCORR: (to_dev(s.extcorr, s.n_extcorr, 16), s.n_extcorr)}
    torch.cuda.synchronize()
    counts = (s.n_generic, s.n_runtime, s.n_device, s.n_extcorr)
    s.n_generic = s.n_runtime = s.n_device = s.n_extcorr = 0   # submit_stream then sends no records
    with TraceEngine(s.trace_name.decode(), device=0) as eng:
        eng.submit_stream(sp)
        for cls, (p, n) in devptrs.items():
            assert eng.lib.ktj_submit_records_device(eng.h, cls, p, n) == 0
        eng.process()
        got = eng.output()
    s.n_generic, s.n_runtime, s.n_device, s.n_extcorr = counts
    release()
    assert got == want


def test_records_submitted_in_many_pieces():
    """The same stream handed over a few records at a time (small submissions wait in a page-locked
    ring and are moved by one kernel launch per sixteen pieces; the arrays they go to grow and move
    in between), by two engines that are alive at the same time and by one created after both were
    destroyed (it starts from what they left behind): every document equals the checker's."""
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    sp, release = abi.synth_stream(3, 20000, host_name="gpubox")
    s = sp.contents
    ora = og.OracleRun(sp)
    want = ora.output()
    ora.close()
    sets = ((abi.REC_GENERIC, s.generic, s.n_generic, 64), (abi.REC_RUNTIME, s.runtime, s.n_runtime, 96),
            (abi.REC_DEVICE, s.device, s.n_device, 64), (abi.REC_EXTCORR, s.extcorr, s.n_extcorr, 16))
    counts = (s.n_generic, s.n_runtime, s.n_device, s.n_extcorr)

    def feed(eng, step):
        s.n_generic = s.n_runtime = s.n_device = s.n_extcorr = 0   # submit_stream then sends no records
        try:
            eng.submit_stream(sp)
        finally:
            s.n_generic, s.n_runtime, s.n_device, s.n_extcorr = counts
        for cls, ptr, n, size in sets:
            base = C.cast(ptr, C.c_void_p).value
            k = 0
            while k < n:
                m = min(step + (k % 7), n - k)   # ragged piece sizes
                assert eng.lib.ktj_submit_records(eng.h, cls, C.c_void_p(base + k * size), m) == 0
                k += m

    a = TraceEngine(s.trace_name.decode(), device=0)
    b = TraceEngine(s.trace_name.decode(), device=0)
    feed(a, 37)
    feed(b, 611)      # pieces just below the ring's limit per submission
    b.process()
    a.process()
    got_a, got_b = a.output(), b.output()
    a.close()
    b.close()
    with TraceEngine(s.trace_name.decode(), device=0) as c:
        feed(c, 5)
        c.process()
        got_c = c.output()
    release()
    assert got_a == want
    assert got_b == want
    assert got_c == want


def test_engines_on_several_threads():
    """Four threads create, feed, run and destroy engines at the same time (a profiler finishes traces
    on background threads): the stream, events and buffers that a destroyed engine leaves for the next
    one change hands between the threads; every document equals the checker's."""
    import threading
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    cases = [(1, 300), (3, 2000), (4, 900), (5, 200), (2, 3000), (3, 40000)]
    streams, want = {}, {}
    for key in cases:
        sp, release = abi.synth_stream(*key, host_name="gpubox")
        ora = og.OracleRun(sp)
        want[key] = ora.output()
        ora.close()
        streams[key] = (sp, release)
    bad = []

    def work(tid):
        try:
            for it in range(12):
                key = cases[(tid + it) % len(cases)]
                sp = streams[key][0]
                with TraceEngine(sp.contents.trace_name.decode(), device=0, no_stage_times=it % 2 == 0) as eng:
                    eng.submit_stream(sp)
                    eng.process()
                    if eng.output() != want[key]:
                        bad.append((tid, it, key))
        except Exception as ex:   # noqa: BLE001 - reported by the assertion below
            bad.append((tid, repr(ex)))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for sp, release in streams.values():
        release()
    assert not bad, bad


@pytest.mark.parametrize("cfg", [3, 2, 4, 5])
def test_full_size_config_digest(cfg):
    """Configurations 2 to 5 at their full sizes (1 is at its full size among the cases above): the
    engine's document and the CPU checker's must have the same length and the same BLAKE2 digest
    (hashed in place, chunk by chunk)."""
    import hashlib
    import oracle_glue as og
    from kineto_amd.engine import TraceEngine
    sp, release = abi.synth_stream(cfg, 0, host_name="gpubox")
    with TraceEngine(sp.contents.trace_name.decode(), device=0) as eng:
        eng.submit_stream(sp)
        eng.process()
        p, n = C.c_void_p(), C.c_uint64()
        assert eng.lib.ktj_output_host(eng.h, C.byref(p), C.byref(n)) == 0
        h1 = hashlib.blake2b()
        view = (C.c_char * n.value).from_address(p.value)
        mv = memoryview(view)
        for off in range(0, n.value, 1 << 26):
            h1.update(mv[off:off + (1 << 26)])
        got_n = n.value
    print("engine done", got_n, flush=True)
    ora = og.OracleRun(sp)
    p, n = C.c_void_p(), C.c_uint64()
    ora.lib.ktj_oracle_output(ora.h, C.byref(p), C.byref(n))
    h2 = hashlib.blake2b()
    mv = memoryview((C.c_char * n.value).from_address(p.value))
    for off in range(0, n.value, 1 << 26):
        h2.update(mv[off:off + (1 << 26)])
    want_n = n.value
    ora.close()
    release()
    assert got_n == want_n
    assert h1.hexdigest() == h2.hexdigest()
