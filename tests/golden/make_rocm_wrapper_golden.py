"""Writes tests/golden/rocm_wrapper_rows.txt: what the reference's RuntimeActivity<T> and GpuActivity
wrappers report for the rows of tests/rocm_wrapper_pattern.py, and which HIP runtime operations
RuntimeActivity<T>::flowStart names, both printed by oracle/_ref/sdk_ref_driver (mode 3), which
compiles the reference's own headers.  Run from the repository root where the reference is present:
  python3 tests/golden/make_rocm_wrapper_golden.py"""
import os
import struct
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from kineto_amd import abi            # noqa: E402
import rocm_wrapper_pattern as rw     # noqa: E402
import sdk_api_pattern as sp          # noqa: E402


def flow_start_ops():
    """One plain runtime row per operation through the wrapper: the operations whose flowStart() is true."""
    n = sp.n_ops()
    recs = []
    for op in range(n):
        r = abi.RuntimeRec()
        r.id, r.begin, r.end, r.cid, r.pid, r.tid, r.kind = 1000 + op, 10, 20, op, 1, 1, 0
        recs.append(bytes(r))
    req = struct.pack("<IQ", 3, n) + b"".join(recs) + struct.pack("<QQ", 0, 0)
    out = subprocess.run([sp.SDK_REF_DRIVER], input=req, stdout=subprocess.PIPE, check=True, timeout=120).stdout.decode("latin1")
    rows = [rw.parse(line) for line in out.split("\n") if line]
    assert len(rows) == n
    return [r["idx"] for r in rows if r["flowstart"]]


def lines():
    return rw.driver_lines() + ["flowstart_ops=" + " ".join(str(x) for x in flow_start_ops())]


if __name__ == "__main__":
    with open(rw.GOLDEN, "w") as f:
        f.write("\n".join(lines()) + "\n")
    print("wrote", rw.GOLDEN)
