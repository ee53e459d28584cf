#!/usr/bin/env python3
"""Writes tests/golden/digests.json: sha256 of the synthetic input records and of the oracle's JSON
for each configuration at test size.  When oracle/_ref (the reference's own logger) is built, the
oracle's bytes are first compared with the real logger's on the same stream (with the real
logger's wall-clock base time and host name), so the digests stand for reference output."""
import hashlib
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle_glue as og  # noqa: E402
from kineto_amd import abi  # noqa: E402
from test_host_side import _stream_digest  # noqa: E402

CASES = [(1, 10000), (2, 30000), (3, 50000), (4, 40000), (5, 6000)]
out = {}
for cfg, n in CASES:
    checked = False
    if og.have_ref():
        sp, release = abi.synth_stream(cfg, n, **og.ref_stream_args())
        o = og.OracleRun(sp)
        assert o.output() == og.ref_render(sp, o), f"oracle differs from the real logger on config {cfg}"
        o.close()
        release()
        checked = True
    sp, release = abi.synth_stream(cfg, n, host_name="golden", trace_name="golden.json")
    o = og.OracleRun(sp)
    data = o.output()
    out[f"{cfg}:{n}"] = {"stream_sha256": _stream_digest(sp), "output_bytes": len(data),
                         "output_sha256": hashlib.sha256(data).hexdigest(), "compared_with_real_logger": checked}
    o.close()
    release()
json.dump(out, open(os.path.join(HERE, "digests.json"), "w"), indent=1, sort_keys=True)
print(json.dumps(out, indent=1))
