"""The seeded input generator of the product library (host code) against an independent
numpy implementation and the committed checksums."""
import hashlib
import json
import os

import numpy as np
import pytest

from np_reference import bits_to_float64, np_fill_normal
from ringattention_amd import api
from ringattention_amd.configs import WORKLOADS

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("seed,offset,sigma", [(0, 0, 1.0), (3, 12345, 1.0), (4, 2**33 + 7, 3.0)])
def test_c_generator_equals_numpy(dtype, seed, offset, sigma):
    n = 200_000
    assert np.array_equal(api.fill_normal(n, dtype, seed, offset, sigma), np_fill_normal(n, dtype, seed, offset, sigma))


def test_known_answers():
    kat = json.load(open(os.path.join(GOLD, "generator_kat.json")))
    assert api.fill_normal(8, "fp16", 0).tolist() == kat["fp16_seed0_first8"]
    assert api.fill_normal(8, "bf16", 3, 1000).tolist() == kat["bf16_seed3_offset1000_first8"]
    assert api.fill_normal(8, "fp16", 4, 0, 3.0).tolist() == kat["fp16_seed4_sigma3_first8"]


def test_distribution_moments():
    x = bits_to_float64(api.fill_normal(2_000_000, "fp16", 17, 0, 3.0), "fp16")
    assert abs(x.mean()) < 0.01 and abs(x.std() - 3.0) < 0.01
    z = x / 3.0
    assert abs((z**3).mean()) < 0.02 and abs((z**4).mean() - 3.0) < 0.05
    # counter based: a slice generated on its own equals the slice of the whole
    a = api.fill_normal(1000, "bf16", 9, 0)
    assert np.array_equal(api.fill_normal(100, "bf16", 9, 500), a[500:600])


def test_workload_input_checksums():
    gold = json.load(open(os.path.join(GOLD, "input_checksums.json")))
    sl = gold["slice"]
    for name, w in WORKLOADS.items():
        ent = gold["workloads"][name]
        n = w.batch * w.heads * w.seq * w.dim
        assert ent["n_per_tensor"] == n
        for ti, (tname, sigma) in enumerate((("q", w.sigma_qk), ("k", w.sigma_qk), ("v", w.sigma_v))):
            base = ti * n
            if "full" in ent[tname]:
                assert sha(api.fill_normal(n, w.dtype, w.seed, base, sigma)) == ent[tname]["full"], (name, tname)
            else:
                assert sha(api.fill_normal(sl, w.dtype, w.seed, base, sigma)) == ent[tname]["head"], (name, tname)
                assert sha(api.fill_normal(sl, w.dtype, w.seed, base + n - sl, sigma)) == ent[tname]["tail"], (name, tname)


def test_make_qkv_layout_is_q_then_k_then_v():
    w = WORKLOADS["cfg1"]
    q, k, v = api.make_qkv_bits(w)
    n = q.size
    whole = api.fill_normal(3 * n, w.dtype, w.seed)
    assert np.array_equal(np.concatenate([q.ravel(), k.ravel(), v.ravel()]), whole)
    assert q.shape == (w.batch, w.heads, w.seq, w.dim)
