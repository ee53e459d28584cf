"""Memset device rows (ktj_memset_rec, CUDA-shaped) pinned against the reference's own wrapper,
GpuActivity<CUpti_ActivityMemsetType> (libkineto/src/CuptiActivity.h:682-719; the graph and channel keys
:424-458), compiled with HAS_CUPTI against CUDA 12.8 headers: what it reports for a fixed set of rows
(oracle/_ref/cupti_ref_driver; kept in tests/golden/cuda_memset_rows.txt for machines without the
reference) against the checker's activities and document and, on the GPU, the engine's document.
With KTJ_CREATE_CUDA12_ARGS every key is compared; without it the document must hold the same text up
to the first of the four keys that the reference compiles in for CUDA >= 12 only."""
import os

import pytest

import cuda_memset_pattern as cm
import oracle_glue as og
import rocm_wrapper_pattern as rw

HAVE_DRIVER = os.path.exists(cm.CUPTI_REF_DRIVER)


def _split(lines):
    assert lines[0].startswith("cuda_version ")
    assert int(lines[0].split()[1]) >= 12000, "the driver prints the CUDA >= 12 key set"
    return [cm.parse(line) for line in lines[1:]]


def _compare_checker_with_reference(ref, all_rows, cuda12):
    assert len(ref) == len(all_rows)
    ora = og.OracleRun(cm.stream(all_rows, cuda12=cuda12).build())
    acts, n = ora.activities()
    order = ora.order()
    doc = ora.output()
    assert n == len(ref), "every row is inside the window"
    by_arrival = {int(acts[i].arrival): i for i in range(n)}
    ev = rw.events(doc)
    assert len(ev) == n
    for k, r in enumerate(ref):
        a = acts[by_arrival[k]]
        what = f"memset row {r['idx']}"
        assert (a.ts, a.dur, a.device, a.resource) == (r["ts"], r["dur"], r["dev"], r["res"]), what
        assert a.type == r["type"] == 4 and a.flow_id == r["flowid"] and a.flow_type == r["flowtype"], what
        assert bool(a.flow_start) == bool(r["flowstart"]), what
    for p, e in enumerate(ev):
        a = acts[order[p]]
        r = ref[int(a.arrival)]
        cat, name, pid, tid, ts, dur, args = e
        what = f"memset row {r['idx']}"
        assert cat == "gpu_memset" and name == r["name"], what
        assert args == (r["json"] if cuda12 else cm.cuda_lt12_json(r["json"])), what
        assert int(pid) == r["dev"] and int(tid) == r["res"], what
    ora.close()


@pytest.mark.parametrize("cuda12", (True, False))
def test_checker_matches_the_reference_memset_wrapper(cuda12):
    _compare_checker_with_reference(_split(cm.reference_lines()), cm.rows(), cuda12)


@pytest.mark.skipif(not HAVE_DRIVER, reason="oracle/_ref/cupti_ref_driver is built only where the reference's sources are")
@pytest.mark.parametrize("seed", range(6))
def test_checker_matches_the_reference_memset_wrapper_on_seeded_rows(seed):
    all_rows = cm.random_rows(seed)
    _compare_checker_with_reference(_split(cm.driver_lines(all_rows)), all_rows, True)


@pytest.mark.skipif(not HAVE_DRIVER, reason="oracle/_ref/cupti_ref_driver is built only where the reference's sources are")
def test_memset_golden_file_is_what_the_reference_produces():
    assert cm.driver_lines() == [line for line in open(cm.GOLDEN).read().split("\n") if line]


def test_golden_rows_cover_the_names_and_the_key_sets():
    ref = _split([line for line in open(cm.GOLDEN).read().split("\n") if line])
    names = {r["name"] for r in ref}
    assert {"Memset (Unknown)", "Memset (Pageable)", "Memset (Pinned)", "Memset (Device)", "Memset (Array)", "Memset (Managed)",
            "Memset (Device Static)", "Memset (Managed Static)", "Memset (Unrecognized)"} <= names
    assert any('"memory bandwidth (GB/s)"' not in r["json"] for r in ref)
    assert all(r["json"].startswith('"device": ') and '"channel_type": ' in r["json"] for r in ref)


@pytest.mark.gpu
@pytest.mark.parametrize("cuda12", (True, False))
def test_engine_matches_the_reference_memset_wrapper(cuda12):
    import test_gpu_parity as tp
    ref = _split([line for line in open(cm.GOLDEN).read().split("\n") if line])
    got = tp._engine_vs_oracle(cm.stream(cuda12=cuda12).build())
    ev = rw.events(got)
    want = [(r["name"], r["json"] if cuda12 else cm.cuda_lt12_json(r["json"])) for r in ref]
    assert sorted((e[1], e[6] or "") for e in ev) == sorted(want)


@pytest.mark.gpu
def test_engine_on_seeded_memset_rows():
    import test_gpu_parity as tp
    for seed in range(3):
        print(f"memset rows seed={seed}", flush=True)
        sp = cm.stream(cm.random_rows(seed, n=3000), cuda12=seed != 1).build()
        tp._engine_vs_oracle(sp)
        tp._engine_vs_oracle(sp, hash_join=True, tile_emit=True)


@pytest.mark.gpu
@pytest.mark.skipif(not HAVE_DRIVER, reason="oracle/_ref/cupti_ref_driver is built only where the reference's sources are")
@pytest.mark.parametrize("seed", range(4))
def test_real_cuda_wrappers_through_the_shim(seed, tmp_path):
    """The reference's own CUDA activity wrappers (runtime and driver API calls, overhead,
    synchronization, CUDA events, memcpy, peer-to-peer memcpy, memset; libkineto/src/CuptiActivity.h),
    some linked to CPU ops, logged through the reference's ChromeTraceLogger and through the
    GpuChromeTraceLogger shim by oracle/_ref/cupti_ref_driver: the two files must be identical.
    (Kernel wrappers are left out: their metadata asks the CUDA runtime for device properties.)"""
    import subprocess
    ref, shim = tmp_path / "ref.json", tmp_path / "shim.json"
    print(f"cuda wrappers through the shim, seed={seed}", flush=True)
    out = subprocess.run([cm.CUPTI_REF_DRIVER, "log", str(seed), str(ref), str(shim)], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                         timeout=120)
    assert out.returncode == 0, out.stderr.decode("latin1")[-2000:]
    assert out.stdout.decode().startswith("activities 166")
    a = ref.read_bytes().replace(str(ref).encode(), b"FILE")
    b = shim.read_bytes().replace(str(shim).encode(), b"FILE")
    assert a.count(b'"ph": "X"') == 166
    for cat in (b'"cuda_runtime"', b'"cuda_driver"', b'"overhead"', b'"cuda_sync"', b'"cuda_event"', b'"gpu_memcpy"', b'"gpu_memset"', b'"cpu_op"'):
        assert cat in a, cat
    assert b'"graph node id"' in a and b'"External id"' in a
    if a != b:
        import test_gpu_parity as tp
        i = tp._first_diff(a, b)
        raise AssertionError(f"files differ at byte {i}:\nREF : {a[max(0, i - 300):i + 200]!r}\nSHIM: {b[max(0, i - 300):i + 200]!r}")
