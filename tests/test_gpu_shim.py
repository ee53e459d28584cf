"""GPU: the libkineto ActivityLogger shim (kineto_amd/shim/GpuChromeTraceLogger) against the
reference's own ChromeTraceLogger.  Both loggers are fed the same libkineto::ITraceActivity objects
through the same calls (handleTraceStart, handle*Info, handleActivity, handleTraceSpan,
finalizeTrace); the shim is obtained from an ActivityLoggerFactory by URL.  The two files must be
byte-identical.  Needs oracle/_ref (built where the reference sources are available)."""
import pytest

import kat_cases
import oracle_glue as og
from kineto_amd import abi

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not (og.have_ref() and og.have_shim()), reason="oracle/_ref not built")]


def _first_diff(a, b):
    n = min(len(a), len(b))
    for i in range(0, n, 4096):
        if a[i:i + 4096] != b[i:i + 4096]:
            for k in range(i, min(i + 4096, n)):
                if a[k] != b[k]:
                    return k
    return n


def _compare(sp, bulk_threads=3):
    o = og.OracleRun(sp)
    try:
        theirs = og.ref_render(sp, o)
        rc, mine, dropped = og.shim_render(sp, o)
        mixed_case_rc, mixed, _ = og.shim_render(sp, o, protocol="GPUJSON")
        bulk_rc, bulk, bulk_dropped = og.shim_render(sp, o, bulk_threads=bulk_threads)
    finally:
        o.close()
    assert rc == 0 and dropped == 0
    if mine != theirs:
        i = _first_diff(mine, theirs)
        raise AssertionError(f"byte {i} of {len(theirs)}: shim {mine[max(0, i - 80):i + 80]!r} "
                             f"reference {theirs[max(0, i - 80):i + 80]!r}")
    assert mixed_case_rc == 0 and mixed == theirs  # protocol lookup is case-insensitive
    # all activities in one handleActivities() call, packed by several workers
    assert bulk_rc == 0 and bulk_dropped == 0
    if bulk != theirs:
        i = _first_diff(bulk, theirs)
        raise AssertionError(f"bulk: byte {i} of {len(theirs)}: shim {bulk[max(0, i - 80):i + 80]!r} "
                             f"reference {theirs[max(0, i - 80):i + 80]!r}")


@pytest.mark.parametrize("cfg,n", [(1, 10000), (2, 20000), (3, 30000), (4, 30000), (5, 4000), (1, 1), (2, 7)])
def test_shim_matches_reference_logger(cfg, n):
    sp, release = abi.synth_stream(cfg, n, **og.ref_stream_args())
    try:
        _compare(sp)
    finally:
        release()


@pytest.mark.parametrize("case", kat_cases.SUBSTRING_CASES + [kat_cases.case_rocm_sync_trace], ids=lambda c: c.__name__)
def test_shim_hand_made_cases(case):
    sp = kat_cases.build_for_real_logger(case, og.ref_stream_args())
    _compare(sp)


@pytest.mark.parametrize("seed", range(12))
def test_shim_random_streams(seed):
    import random_streams
    sp = kat_cases.build_for_real_logger(lambda: (random_streams.random_stream(seed, wide_ids=seed % 2 == 1), None),
                                         og.ref_stream_args())
    _compare(sp)


@pytest.mark.parametrize("case", [(1, 3000), (2, 6000), (3, 20000), (4, 9000), (5, 800), "random3", "random8", "kat"])
def test_shim_in_the_profilers_call_order(case):
    """GenericActivityProfiler drives a logger in another order than the buffering logger's replay
    (src/GenericActivityProfiler.cpp:178-224, 655-740): CPU-side activities, the CPU buffer's span,
    GPU-side activities, then resource infos, device infos, GPU spans and overhead infos.  The
    reference logger writes every event where its call arrives; fed those calls, the shim must write
    the reference's file for the same calls with the activity segment sorted."""
    import random_streams
    if case == "kat":
        sp, release = kat_cases.build_for_real_logger(kat_cases.case_rocm_sync_trace, og.ref_stream_args()), None
    elif isinstance(case, str):
        seed = int(case[6:])
        sp, release = kat_cases.build_for_real_logger(lambda: (random_streams.random_stream(seed), None), og.ref_stream_args()), None
    else:
        sp, release = abi.synth_stream(case[0], case[1], **og.ref_stream_args())
    o = og.OracleRun(sp)
    try:
        theirs = og.ref_render(sp, o, call_order=1)
        if sp.contents.n_device_infos or sp.contents.n_resource_infos:
            assert theirs != og.ref_render(sp, o)          # the two orders give different files
        for threads in (0, 4):
            rc, mine, dropped = og.shim_render(sp, o, bulk_threads=threads, call_order=2)
            assert rc == 0 and dropped == 0
            if mine != theirs:
                i = _first_diff(mine, theirs)
                raise AssertionError(f"threads={threads}: byte {i} of {len(theirs)}: shim {mine[max(0, i - 80):i + 80]!r} "
                                     f"reference {theirs[max(0, i - 80):i + 80]!r}")
    finally:
        o.close()
        if release:
            release()


def test_shim_bulk_packing_is_independent_of_the_worker_count():
    """handleActivities() with 1, 2, 5 and 16 workers writes the same file as the reference."""
    sp, release = abi.synth_stream(3, 40000, **og.ref_stream_args())
    o = og.OracleRun(sp)
    try:
        theirs = og.ref_render(sp, o)
        for threads in (1, 2, 5, 16):
            rc, mine, dropped = og.shim_render(sp, o, bulk_threads=threads)
            assert rc == 0 and dropped == 0
            assert mine == theirs, threads
    finally:
        o.close()
        release()


def test_shim_keeps_activities_whose_device_id_does_not_fit_32_bits():
    """A deviceId beyond 32 bits has no place in the packed record's device field: it travels in the
    slot before the record's values (KTJ_GF_WIDE_DEVICE).  The file is the one the reference logger
    writes from the same activities, whether they come one by one or inside one handleActivities()
    call, and nothing is dropped."""
    sp, release = abi.synth_stream(3, 20000, **og.ref_stream_args())
    o = og.OracleRun(sp)
    try:
        for mod in (5, 1000):
            theirs = og.ref_render(sp, o, wide_device_mod=mod)
            assert b'"pid": 1099511627776' in theirs
            for threads in (0, 1, 6):
                rc, mine, dropped = og.shim_render(sp, o, bulk_threads=threads, huge_device_mod=mod)
                assert rc == 0 and dropped == 0, (mod, threads, dropped)
                assert mine == theirs, (mod, threads)
    finally:
        o.close()
        release()


def test_shim_unknown_protocol_and_bad_sink():
    sp, release = abi.synth_stream(1, 50, **og.ref_stream_args())
    o = og.OracleRun(sp)
    try:
        rc, data, _ = og.shim_render(sp, o, protocol="nosuch")
        assert rc == -3 and data is None          # factory: no logger for that prefix
        rc, data, _ = og.shim_render(sp, o, directory="/nonexistent-dir/sub")
        assert rc == abi.KTJ_ERR_IO and data is None  # bad sink: handlers are no-ops, finalize reports
    finally:
        o.close()
        release()
