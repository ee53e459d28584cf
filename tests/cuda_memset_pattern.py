"""Test-only: a fixed set of memset device rows (ktj_memset_rec), what the reference's own
GpuActivity<CUpti_ActivityMemsetType> (libkineto/src/CuptiActivity.h:682-719, compiled against CUDA 12
headers) reports for them through oracle/_ref/cupti_ref_driver, and the same rows as a stream for
the checker and the engine."""
import os
import random
import struct
import subprocess

from kineto_amd import abi
from stream_builder import B, StreamBuilder
import rocm_wrapper_pattern as rw

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CUPTI_REF_DRIVER = os.path.join(ROOT, "oracle", "_ref", "cupti_ref_driver")
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cuda_memset_rows.txt")
# the four keys a reference built against CUDA >= 12 appends (CuptiActivity.h:424-458)
CUDA12_TAIL = ', "graph id": '


def rows():
    """Keyword arguments of StreamBuilder.add_memset: every memory kind (the name), an unknown one,
    zero duration (no bandwidth), a negative duration, ids at the edges of 32 bits, a graph node id
    beyond 32 bits, every channel type, a bandwidth with many digits, a device beyond one digit."""
    t = B + 1000
    out = [
        dict(id=42, begin=t + 1000, end=t + 3000, device=0, context=3, stream=7, nbytes=4096, memory_kind=3),
        dict(id=43, begin=t + 3100, end=t + 3100, device=1, context=1, stream=7, nbytes=1 << 20, memory_kind=3),          # no bandwidth
        dict(id=44, begin=t + 3200, end=t + 3190, device=0, context=2, stream=9, nbytes=777, memory_kind=3),              # negative duration
        dict(id=45, begin=t + 3300, end=t + 3307, device=0, context=0xFFFFFFFF, stream=0xFFFFFFFF, nbytes=1000,
             memory_kind=3, graph_id=0xFFFFFFFF, graph_node_id=0xFFFFFFFFFFFFFFFF, channel_id=0xFFFFFFFF, channel_type=2),
        dict(id=0xFFFFFFFF, begin=t + 3400, end=t + 3403, device=15, context=5, stream=1, nbytes=(1 << 40) + 1, memory_kind=3,
             graph_id=9, graph_node_id=(1 << 32) + 5, channel_id=11, channel_type=1),
        dict(id=0, begin=t + 3500, end=t + 3600, device=0, context=1, stream=2, nbytes=0, memory_kind=3),                 # id 0: no flow event
        dict(id=46, begin=t + 3700, end=t + 3701, device=0, context=1, stream=0, nbytes=3, memory_kind=3, channel_type=3),
    ]
    for kind in (0, 1, 2, 4, 5, 6, 7, 8, 200):
        out.append(dict(id=100 + kind, begin=t + 4000 + 10 * kind, end=t + 4003 + 10 * kind, device=0, context=1, stream=4,
                        nbytes=10 + kind, memory_kind=kind, graph_id=kind, graph_node_id=kind * 3, channel_id=kind % 4,
                        channel_type=kind % 3))
    return out


def random_rows(seed, n=200):
    rng = random.Random(seed)
    t = B + 10000
    out = []
    for i in range(n):
        begin = t + rng.randrange(0, 10**6)
        out.append(dict(id=rng.choice([rng.randrange(1, 1 << 32), rng.randrange(1, 500)]), begin=begin,
                        end=begin + rng.choice([0, 1, 3, 7, 1000, rng.randrange(1, 10**6)]), device=rng.randrange(0, 16),
                        context=rng.choice([1, 2, rng.getrandbits(32)]), stream=rng.choice([0, 7, 13, rng.getrandbits(32)]),
                        nbytes=rng.choice([0, 1, 4096, rng.getrandbits(20), rng.getrandbits(48), rng.getrandbits(64)]),
                        memory_kind=rng.randrange(0, 10), graph_id=rng.choice([0, rng.getrandbits(32)]),
                        graph_node_id=rng.choice([0, rng.getrandbits(20), rng.getrandbits(64)]),
                        channel_id=rng.choice([0, 3, rng.getrandbits(32)]), channel_type=rng.randrange(0, 4)))
    return out


def stream(all_rows=None, cuda12=True):
    """The rows as a ktj_stream (no clock conversion, wide window)."""
    b = StreamBuilder(host_name="memset")
    b.create_flags = abi.KTJ_CREATE_CUDA12_ARGS if cuda12 else 0
    for kw in (all_rows or rows()):
        b.add_memset(**kw)
    return b


def driver_lines(all_rows=None):
    b = stream(all_rows)
    req = struct.pack("<Q", len(b.device)) + b"".join(bytes(d) for d in b.device)
    out = subprocess.run([CUPTI_REF_DRIVER], input=req, stdout=subprocess.PIPE, check=True, timeout=120).stdout.decode("latin1")
    return [line for line in out.split("\n") if line]


def reference_lines():
    """cuda_version line first, then one line per row."""
    if os.path.exists(CUPTI_REF_DRIVER):
        return driver_lines()
    return [line for line in open(GOLDEN).read().split("\n") if line]


def parse(line):
    return rw.parse(line.replace("memset idx=", "device idx=", 1))


def cuda_lt12_json(js):
    """What the same wrapper prints when compiled for CUDA < 12: the text up to the graph keys."""
    i = js.index(CUDA12_TAIL)
    return js[:i]
