#!/usr/bin/env python3
"""Writes tests/golden/sdk_api_rows.txt: the rows the reference's RocprofLogger::api_callback
(libkineto/src/RocprofLogger.cpp:561-679) makes of one call of every HIP runtime API operation the
rocprofiler-sdk of this image knows, with the call's argument union filled by a fixed pattern
(tests/sdk_api_pattern.py).  Needs oracle/_ref/sdk_ref_driver, which compiles the reference's
translation unit where it lies; the file it writes is data (one text line per row, plus the SDK's
own rendering of the call's arguments), not reference source."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import sdk_api_pattern as pat  # noqa: E402

lines = pat.reference_lines()
with open(os.path.join(HERE, "sdk_api_rows.txt"), "w") as f:
    f.write("\n".join(lines) + "\n")
print(len(lines), "lines")
