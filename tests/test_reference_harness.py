"""The reference's main() (csrc/ring_attention.cu:750-790) rebuilt on the C ABI as a plain C++
program: its own configuration (dim 64, 2 ranks x 8192 tokens, fp16, the reference's fill)."""
import os
import re
import subprocess

import numpy as np
import pytest

from ringattention_amd import api
from ringattention_amd._build import HARNESS_PATH


def test_harness_is_built():
    assert os.path.exists(HARNESS_PATH), "run __graft_entry__.build() first"


@pytest.mark.gpu
def test_harness_runs_the_reference_configuration(oracle):
    npes, chunk, dim = 2, 8192, 64
    res = subprocess.run([HARNESS_PATH, str(npes), str(chunk), "3"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    lines = res.stdout.strip().splitlines()
    assert lines[:npes] == [f"mype: {i} success" for i in range(npes)]
    assert re.fullmatch(r"elapsedtime=\d+\.\d+", lines[-1])
    corner = np.array([[float(x) for x in ln.split()] for ln in lines[npes:npes + 8]])
    assert corner.shape == (8, 8)
    # the same inputs through the oracle: every rank's block holds the reference's pattern
    lib = api._lib.load()
    blk = np.empty((chunk, dim), dtype=np.uint16)
    assert lib.ringattn_fill_reference_pattern(blk.ctypes.data, 0, chunk, dim) == 0
    x = np.ascontiguousarray(np.tile(blk, (npes, 1))[None, None])
    o_ref, _ = oracle.attention_rows(x, x, x, "fp16", causal=False, rows=np.arange(8))
    ulp = 2.0**-10 * np.abs(o_ref[:, :8]).max()
    assert np.abs(corner - o_ref[:, :8]).max() <= max(1e-2, 2 * ulp)   # printed with 4 decimals, fp16 values
