"""Writes tests/golden/c1_seed0.npz: the oracle's output for configuration c1
(B2 C8 T32 H4 Dh32, q/k/v ~ N(0,1), seed 0, fp32).

The reference ships no golden vectors and was not executed to make this file: the numbers come
from oracle/mvpa_oracle.py (float64 closed form, stored as float32) once it had passed
tests/test_oracle.py.  The fixture pins the oracle and the input generator against drift and gives
the GPU tests a vector that does not depend on recomputation on the test machine.

    python tests/golden/make_c1_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [os.path.join(ROOT, "multi-variate-parallel-transformer_amd"), ROOT]

from mvpa_hip.synthetic import make_mvpa_inputs  # noqa: E402
from oracle import mvpa_oracle as O  # noqa: E402

inp = make_mvpa_inputs(B=2, C=8, T=32, H=4, Dh=32, seed=0)
out, lse = O.mvpa_direct(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                         return_lse=True)
np.savez_compressed(os.path.join(HERE, "c1_seed0.npz"),
                    out=out.numpy().astype(np.float32), lse=lse.numpy().astype(np.float32),
                    q_probe=inp.q[0, 0, :4].numpy(), k_time_probe=inp.k_time[0, :2].numpy())
print("wrote c1_seed0.npz", out.shape)
