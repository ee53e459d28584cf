"""CPU: host-side pieces of the product — the C-ABI library loads and exports what include/ktj.h
declares, the formatting core (host build) agrees with the oracle, the generator is deterministic."""
import ctypes as C
import hashlib
import json
import os
import re

import pytest

import oracle_glue as og
from kineto_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SIM_SO = os.path.join(ROOT, "tests", "host_sim", "libktjsim.so")


def test_engine_library_exports_every_declared_symbol():
    decl = set()
    for hdr in ("ktj.h", "ktj_debug.h", "ktj_rocprofiler.h"):
        text = open(os.path.join(ROOT, "include", hdr)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        decl |= set(re.findall(r"\b(ktj_[a-z_]+)\s*\(", text))
    decl -= {"ktj_synth_generate", "ktj_synth_free"}
    lib = abi.load_engine()          # no GPU call happens on load
    for name in sorted(decl):
        assert hasattr(lib, name), name
    assert set(abi.ENGINE_SYMBOLS) <= decl
    assert lib.ktj_version().startswith(b"ktj")


def test_record_layouts_match_the_header():
    src = r'''
    #include "ktj_stream.h"
    #include <stdio.h>
    #include <stddef.h>
    int main(void) { printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(ktj_generic_rec), sizeof(ktj_runtime_rec),
      sizeof(ktj_device_rec), sizeof(ktj_extcorr_rec), sizeof(ktj_stream), sizeof(ktj_stats), offsetof(ktj_runtime_rec, u),
      offsetof(ktj_device_rec, queue), sizeof(ktj_clock_model)); return 0; }'''
    import subprocess
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "a.c"), "w").write(src)
        subprocess.run(["gcc", "-I" + os.path.join(ROOT, "include"), os.path.join(d, "a.c"), "-o", os.path.join(d, "a")], check=True)
        out = subprocess.run([os.path.join(d, "a")], check=True, capture_output=True, text=True).stdout.split()
    want = [C.sizeof(abi.GenericRec), C.sizeof(abi.RuntimeRec), C.sizeof(abi.DeviceRec), C.sizeof(abi.ExtCorrRec),
            C.sizeof(abi.Stream), C.sizeof(abi.Stats), abi.RuntimeRec.u.offset, abi.DeviceRec.queue.offset,
            C.sizeof(abi.ClockModel)]
    assert [int(x) for x in out] == want


@pytest.fixture(scope="module")
def sim():
    lib = C.CDLL(SIM_SO)
    lib.ktjsim_render.argtypes = [C.POINTER(abi.Stream), C.c_uint32, C.POINTER(C.c_void_p), C.POINTER(C.c_uint64)]
    lib.ktjsim_free.argtypes = [C.c_void_p]
    lib.ktjsim_fmt_double.argtypes = [C.c_double, C.c_char_p]
    lib.ktjsim_convert_ts.restype = C.c_longlong
    lib.ktjsim_convert_ts.argtypes = [C.c_ulonglong, C.c_ulonglong, C.c_longlong, C.c_double]
    return lib


@pytest.mark.parametrize("cfg,n,tile", [(1, 5000, 16384), (2, 9000, 16384), (3, 12000, 4096), (4, 12000, 16384),
                                        (5, 1500, 16384), (5, 700, 336), (1, 300, 24), (3, 9000, 0), (5, 900, 0), (2, 7000, 0), (4, 9000, 0)])
def test_formatting_core_host_build_matches_oracle(sim, cfg, n, tile):
    sp, release = abi.synth_stream(cfg, n, host_name="box")
    o = og.OracleRun(sp)
    want = o.output()
    p, nb = C.c_void_p(), C.c_uint64()
    rc = sim.ktjsim_render(sp, tile, C.byref(p), C.byref(nb))
    assert rc == 0
    got = C.string_at(p, nb.value)
    sim.ktjsim_free(p)
    o.close()
    release()
    assert got == want


def _sim_vs_oracle(sim, sp, tile):
    o = og.OracleRun(sp)
    want = o.output()
    o.close()
    p, nb = C.c_void_p(), C.c_uint64()
    rc = sim.ktjsim_render(sp, tile, C.byref(p), C.byref(nb))
    assert rc == 0
    got = C.string_at(p, nb.value)
    sim.ktjsim_free(p)
    if got != want:
        i = next((k for k in range(min(len(got), len(want))) if got[k] != want[k]), min(len(got), len(want)))
        raise AssertionError(f"byte {i}: got {got[max(0, i - 80):i + 60]!r} want {want[max(0, i - 80):i + 60]!r}")


def test_hand_made_cases_host_build_matches_oracle(sim):
    import kat_cases
    for case in kat_cases.SUBSTRING_CASES + [kat_cases.case_rocm_sync_trace]:
        b, _ = case()
        sp = b.build()
        for tile in (0, 4096):
            _sim_vs_oracle(sim, sp, tile)


@pytest.mark.parametrize("seed", range(40))
def test_random_streams_host_build_matches_oracle(sim, seed):
    import random_streams
    sp = random_streams.random_stream(seed, wide_ids=seed % 2 == 1).build()
    _sim_vs_oracle(sim, sp, 0 if seed % 3 else 4096)


def test_device_double_and_clock_code_matches_oracle(sim):
    import math
    import random
    import struct
    ora = og.load_oracle()
    rng = random.Random(3)
    b1, b2 = C.create_string_buffer(64), C.create_string_buffer(64)
    for _ in range(200000):
        v = struct.unpack("<d", struct.pack("<Q", rng.getrandbits(64)))[0] if rng.random() < 0.5 else rng.randrange(1, 1 << 40) / rng.randrange(1, 1 << 24)
        if math.isnan(v):
            continue
        n1 = sim.ktjsim_fmt_double(v, b1)
        n2 = ora.ktj_oracle_fmt_double(v, b2)
        assert b1.raw[:n1] == b2.raw[:n2], v
    for _ in range(100000):
        t0a = rng.randrange(0, 1 << 40)
        t = max(0, t0a + rng.choice([rng.randrange(-3, 4), rng.randrange(1, 1 << 30), rng.randrange(1, 1 << 62)]))
        scale = rng.choice([1.0, 1.000001, 0.999999, rng.uniform(1e-3, 1e3)])
        t0 = rng.randrange(-(1 << 40), 1 << 61)
        m = abi.ClockModel(t0a, t0, scale, 0, 1, 1)
        assert sim.ktjsim_convert_ts(t, t0a, t0, scale) == ora.ktj_oracle_convert_ts(C.byref(m), t)


def _stream_digest(sp):
    s = sp.contents
    h = hashlib.sha256()
    h.update(C.string_at(s.str_blob, s.str_off[s.n_strings]))
    for ptr, n, sz in ((s.generic, s.n_generic, 64), (s.runtime, s.n_runtime, 96), (s.device, s.n_device, 64),
                       (s.extcorr, s.n_extcorr, 16), (s.args, s.n_args, 8)):
        if n:
            h.update(C.string_at(C.cast(ptr, C.c_void_p), n * sz))
    return h.hexdigest()


def test_golden_digests():
    """Generator and oracle outputs are pinned: tests/golden/digests.json was written by
    tests/golden/make_golden.py in a container where the oracle's output had just been compared
    byte for byte with the real logger's."""
    gold = json.load(open(os.path.join(ROOT, "tests", "golden", "digests.json")))
    for key, g in gold.items():
        cfg, n = (int(x) for x in key.split(":"))
        sp, release = abi.synth_stream(cfg, n, host_name="golden", trace_name="golden.json")
        assert _stream_digest(sp) == g["stream_sha256"], key
        o = og.OracleRun(sp)
        out = o.output()
        o.close()
        release()
        assert len(out) == g["output_bytes"], key
        assert hashlib.sha256(out).hexdigest() == g["output_sha256"], key


def test_bench_refuses_more_than_one_gpu_and_fails_without_one():
    """bench.py measures one GPU: --gpus above 1 exits with a message that says so; where no GPU is
    visible it fails instead of measuring anything else."""
    import subprocess
    import sys
    import torch
    bench = os.path.join(ROOT, "bench.py")
    r = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""
    if not torch.cuda.is_available():
        r = subprocess.run([sys.executable, bench, "--steps", "1", "--warmup", "0"], capture_output=True, text=True, timeout=300)
        assert r.returncode != 0 and "no GPU" in r.stderr and r.stdout.strip() == ""


def test_product_fails_loudly_without_its_library_or_a_gpu(tmp_path, monkeypatch):
    """There is no CPU fallback: without the built HIP library the loader raises, and where the
    library is there but no GPU is visible the engine cannot be created."""
    import torch
    from kineto_amd import engine
    monkeypatch.setattr(abi, "_engine", None)
    monkeypatch.setattr(abi, "LIB_DIR", str(tmp_path))
    with pytest.raises(RuntimeError, match="not built"):
        abi.load_engine()
    monkeypatch.undo()
    if not torch.cuda.is_available():
        with pytest.raises(engine.EngineError):
            engine.TraceEngine("t.json", device=0)
