"""Writes tests/golden/cuda_memset_rows.txt: what the reference's GpuActivity<CUpti_ActivityMemsetType>
(libkineto/src/CuptiActivity.h:682-719) reports for the rows of tests/cuda_memset_pattern.py, printed by
oracle/_ref/cupti_ref_driver, which compiles the reference's own header against the CUDA 12 and CUPTI
headers of this image.  Run from the repository root where the reference is present:
  python3 tests/golden/make_cuda_memset_golden.py"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import cuda_memset_pattern as cm     # noqa: E402


if __name__ == "__main__":
    with open(cm.GOLDEN, "w") as f:
        f.write("\n".join(cm.driver_lines()) + "\n")
    print("wrote", cm.GOLDEN)
