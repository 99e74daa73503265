"""The reference-shaped entry point that allocates nothing (its table of ring steps lives in a
static device scratch) against the allocating one, through the C ABI: same bits, on two calls
in a row, the second on a smaller input (the scratch keeps the first call's contents)."""
import numpy as np
import pytest
import torch

from ringattention_amd import _lib, api

pytestmark = pytest.mark.gpu


def _run_pair(npes, seqlen, dim, dtype, causal, mype, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    S = sum(seqlen)
    c = seqlen[mype]
    start = sum(seqlen[:mype])
    k = torch.randn(S, dim, generator=g).to(dtype).cuda()
    v = torch.randn(S, dim, generator=g).to(dtype).cuda()
    q = torch.randn(S, dim, generator=g).to(dtype)[start:start + c].contiguous().cuda()
    out_a = torch.full((c, dim), 7.0, dtype=dtype, device="cuda")
    out_b = torch.full((c, dim), -7.0, dtype=dtype, device="cuda")
    lse_a = torch.full((c,), 3.0, dtype=torch.float32, device="cuda")
    lse_b = torch.full((c,), -3.0, dtype=torch.float32, device="cuda")
    api.ring_attention(q, k, v, out_a, npes, mype, seqlen, dim, max(seqlen), lse=lse_a, causal=causal)
    api.ring_attention_noalloc(q, k, v, out_b, npes, mype, seqlen, dim, max(seqlen), lse=lse_b, causal=causal)
    torch.cuda.synchronize()
    assert torch.isfinite(out_a.float()).all()
    assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16)), "O differs from the allocating entry point"
    assert torch.equal(lse_a.view(torch.int32), lse_b.view(torch.int32)), "LSE differs from the allocating entry point"


def test_noalloc_entry_matches_allocating_entry_twice_in_a_row():
    # first a larger call, then a smaller one on the same (dirty) scratch
    _run_pair(4, [640, 512, 384, 512], 128, torch.bfloat16, True, 3, seed=101)
    _run_pair(3, [100, 130, 77], 64, torch.float16, False, 1, seed=102)
    _run_pair(2, [256, 256], 128, torch.float16, True, 0, seed=103)


def test_noalloc_entry_without_lse_and_on_a_side_stream():
    seqlen, dim, mype = [256, 192], 64, 1
    g = torch.Generator(device="cpu").manual_seed(7)
    k = torch.randn(sum(seqlen), dim, generator=g).half().cuda()
    v = torch.randn(sum(seqlen), dim, generator=g).half().cuda()
    q = torch.randn(seqlen[mype], dim, generator=g).half().cuda()
    out_a, out_b = torch.empty_like(q), torch.empty_like(q)
    api.ring_attention(q, k, v, out_a, 2, mype, seqlen, dim, 256)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    api.ring_attention_noalloc(q, k, v, out_b, 2, mype, seqlen, dim, 256, stream=side)
    side.synchronize()
    assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16))


def test_noalloc_entry_limits():
    lib = _lib.load()
    assert lib.ringattn_noalloc_scratch_bytes() == 4096
    # the scratch holds the table of ring steps: 32 bytes + 32 per visible step, so 64 ranks fit ...
    _run_pair(64, [64] * 64, 64, torch.float16, False, 17, seed=104)
    _run_pair(8, [4096] * 8, 128, torch.bfloat16, True, 7, seed=105)      # ... whatever the lengths
    # ... and a longer ring is refused as everywhere else
    npes, c, dim = 65, 32, 64
    q = torch.zeros(c, dim, dtype=torch.float16, device="cuda")
    kv = torch.zeros(npes * c, dim, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.RingattnError) as e:
        api.ring_attention_noalloc(q, kv, kv, torch.empty_like(q), npes, 0, [c] * npes, dim, c)
    assert e.value.code == 2              # RINGATTN_ERR_NPES
