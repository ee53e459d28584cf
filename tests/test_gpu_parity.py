"""GPU parity: the HIP engine, called through the C ABI, must produce the same bytes as the CPU
checker on the same seeded streams; intermediate stages are compared too so that a failure names
the stage."""
import ctypes as C

import numpy as np
import pytest

from kineto_amd import abi

pytestmark = pytest.mark.gpu

CASES = [(1, 10000), (2, 20000), (3, 30000), (4, 30000), (5, 5000), (1, 1), (3, 4097), (5, 3)]


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
    ora.close()
    release()
    if got != want:
        i = _first_diff(got, want)
        raise AssertionError(f"config {cfg} n={n}: bytes differ at {i} (got {len(got)} bytes, want {len(want)}):\n"
                             f"GOT : {got[max(0, i - 200):i + 120]!r}\nWANT: {want[max(0, i - 200):i + 120]!r}")
    return st


@pytest.mark.parametrize("cfg,n", CASES)
def test_engine_matches_oracle(cfg, n):
    print(f"case config={cfg} n={n}", flush=True)
    run_case(cfg, n)
