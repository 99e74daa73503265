"""Writes the committed fixtures under tests/golden/.  Run from the repository root:

    python tests/golden/make_golden.py

The reference repository holds no golden vector, fixture or assertion for this path (its
test/ directory has three unrelated print-only programs), and its only Python file
(csrc/self_attention.py) is a CUDA-device script with unseeded inputs, so nothing is
imported from it.  The fixtures are therefore made from independent restatements only:
inputs by the numpy generator in tests/np_reference.py and expected outputs by torch CPU
float64 library routines (matmul / softmax / logsumexp) -- neither shares code with the
C oracle or with the product, which are both tested against these files.
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from np_reference import np_fill_normal, np_make_qkv, torch_attention  # noqa: E402
from ringattention_amd.configs import WORKLOADS, Workload  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
SLICE = 1 << 18


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    # 1. full expected outputs of cfg1 (non-causal) and of a small causal bf16 case
    cases = {"cfg1": WORKLOADS["cfg1"], "causal_small": Workload("causal_small", 1, 2, 128, 2, 128, "bf16", 11, True)}
    for name, w in cases.items():
        q, k, v = np_make_qkv(w)
        o, lse = torch_attention(q, k, v, w.dtype, causal=w.causal)
        np.savez_compressed(os.path.join(HERE, f"{name}_expected.npz"),
                            o_f32=o.astype(np.float32), lse_f64=lse.astype(np.float64),
                            q_sha=np.array(sha(q)), k_sha=np.array(sha(k)), v_sha=np.array(sha(v)))
    # 2. checksums of the seeded inputs of every workload: whole tensors where small, the
    #    first and last 2^18 elements of each tensor where large (the generator is counter
    #    based, so any slice can be produced on its own)
    sums = {}
    for name, w in WORKLOADS.items():
        n = w.batch * w.heads * w.seq * w.dim
        ent = {"n_per_tensor": n, "dtype": w.dtype, "seed": w.seed}
        for ti, (tname, sigma) in enumerate((("q", w.sigma_qk), ("k", w.sigma_qk), ("v", w.sigma_v))):
            base = ti * n
            if n <= (1 << 22):
                ent[tname] = {"full": sha(np_fill_normal(n, w.dtype, w.seed, base, sigma))}
            else:
                ent[tname] = {"head": sha(np_fill_normal(SLICE, w.dtype, w.seed, base, sigma)),
                              "tail": sha(np_fill_normal(SLICE, w.dtype, w.seed, base + n - SLICE, sigma))}
        sums[name] = ent
    with open(os.path.join(HERE, "input_checksums.json"), "w") as f:
        json.dump({"slice": SLICE, "workloads": sums}, f, indent=1, sort_keys=True)
    # 3. a few raw generator values (bit patterns) for a quick known-answer check
    kat = {"fp16_seed0_first8": np_fill_normal(8, "fp16", 0).tolist(),
           "bf16_seed3_offset1000_first8": np_fill_normal(8, "bf16", 3, 1000).tolist(),
           "fp16_seed4_sigma3_first8": np_fill_normal(8, "fp16", 4, 0, 3.0).tolist()}
    with open(os.path.join(HERE, "generator_kat.json"), "w") as f:
        json.dump(kat, f, indent=1, sort_keys=True)
    print("wrote fixtures to", HERE)


if __name__ == "__main__":
    main()
