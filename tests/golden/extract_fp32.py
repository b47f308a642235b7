"""Writes tests/golden/dlrm_*_fp32.bin: the first 16 of the 64 samples of the float32 data files the reference
keeps under test/dlrm/data/ (samples are independent of one another; a quarter keeps the fixtures small).
Run where the reference checkout is: python tests/golden/extract_fp32.py /root/reference"""
import os
import sys

import numpy as np

SAMPLES, M, K = 16, 27, 128
WIDTH = K + M * (M - 1) // 2
ROWS = {"input_fp32": M * K, "output_fp32": WIDTH, "input_grad_fp32": WIDTH, "output_input_grad_fp32": M * K,
        "output_mlp_input_grad_fp32": K}

if __name__ == "__main__":
    src = os.path.join(sys.argv[1], "test", "dlrm", "data")
    here = os.path.dirname(os.path.abspath(__file__))
    for name, per_sample in ROWS.items():
        data = np.fromfile(os.path.join(src, name), dtype=np.float32)
        assert data.size == 64 * per_sample, (name, data.size)
        data[: SAMPLES * per_sample].tofile(os.path.join(here, f"dlrm_{name}.bin"))
