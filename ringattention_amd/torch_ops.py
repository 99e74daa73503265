"""torch.Tensor front end: `torch.ops.ringattn.fwd`, registered by libringattn_torch.so.

The op follows the conventions the reference's include/attention_api.cuh:12-18 sets for a
torch extension (inputs device-resident and contiguous, checked with its CHECK_INPUT
wording) and runs ringattn_fwd of the C ABI on torch's current stream.  Plans (parameters
+ device tables) are cached inside the extension per parameter set AND stream (at most 16,
least recently used first out), so forwards on different streams never share a plan.
"""
import os

import torch

from ._build import TORCH_LIB_PATH

_loaded = False


def load():
    """Register ringattn::fwd with the dispatcher; raise if the extension has not been built."""
    global _loaded
    if _loaded:
        return
    if not os.path.exists(TORCH_LIB_PATH):
        raise RuntimeError(
            f"{TORCH_LIB_PATH} is missing: the torch front end has not been built. "
            "Run `python -c 'import __graft_entry__ as g; g.build()'` at the repository root.")
    torch.ops.load_library(TORCH_LIB_PATH)
    _loaded = True


def ring_attention_fwd(q, k, v, seqlen, causal=False, softmax_scale=0.0, zigzag=False):
    """Ring-attention forward for all len(seqlen) virtual ranks.

    q [B, H, S, d], k / v [B, H_kv, S, d] fp16 or bf16 device tensors, seqlen: tokens per rank
    (sum = S).  Returns (out [B, H, S, d] in the input dtype, lse [B, H, S] float32)."""
    load()
    return torch.ops.ringattn.fwd(q, k, v, [int(c) for c in seqlen], bool(causal), float(softmax_scale), bool(zigzag))
