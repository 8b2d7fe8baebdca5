"""Writes tests/golden/config1_fprop.npy: the CPU oracle's output for the
CPU-runnable configuration (batch 4, 16 -> 16 planes, 32x32 input, 5x5 kernel,
stride 1, no padding, inputs uniform[-1,1) from seed 1001).

The reference's own CPU convolution cannot be compiled in this image (it needs
thpp, folly and glog), so this vector comes from oracle/refconv.c, which
tests/test_oracle_conv.py pins by other means.  Run from the repo root:
    python tests/golden/make_config1.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from fbcunn_amd import synth  # noqa: E402

x = synth.uniform(1001, (4, 16, 32, 32), stream=0)
w = synth.uniform(1001, (16, 16, 5, 5), stream=1)
out = oracle.cross_correlation_valid(x, w)
np.save(os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1_fprop.npy"), out)
print(out.shape, float(out.min()), float(out.max()))
