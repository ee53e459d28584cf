"""Writes tests/golden/profiler_loop_seed<k>.json: what the reference's own post-processing loop
(GenericActivityProfiler::processTraceInternal with the ROCm handlers and the real ChromeTraceLogger,
run by oracle/_ref/profiler_ref_driver) writes for the seeded cases of
tests/rocm_wrapper_pattern.py:profiler_case — its complete and flow events as text, its counters,
its base time and the clock offset it applied to the device rows.  Run from the repository root
where the reference is present:
  python3 tests/golden/make_profiler_loop_golden.py"""
import json
import os
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import rocm_wrapper_pattern as rw     # noqa: E402

SEEDS = (0, 1)


def golden_path(seed):
    return os.path.join(HERE, "profiler_loop_seed%d.json" % seed)


def reference_run(seed, directory):
    case = rw.profiler_case(seed)
    info, doc = rw.run_reference_profiler(case, os.path.join(directory, "ref_trace.json"))
    ev, fl = rw.events(doc), rw.flow_events(doc)
    marker = [e for e in ev if e[6] and '"correlation": %d,' % rw.MARKER_ID in e[6]]
    assert len(marker) == 1
    whole, frac = marker[0][4].split(".")
    offset = info["base_time"] + int(whole) * 1000 + int(frac) - (case["rows"][1][0][1] + 1)
    return dict(seed=seed, base_time=info["base_time"], device_offset=offset, out_of_range=info["out_of_range"],
                out_of_order=info["out_of_order"], events=[list(e) for e in ev], flows=[list(f) for f in fl])


if __name__ == "__main__":
    with tempfile.TemporaryDirectory() as d:
        for seed in SEEDS:
            with open(golden_path(seed), "w") as f:
                json.dump(reference_run(seed, d), f, indent=0)
            print("wrote", golden_path(seed))
