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


def test_noalloc_entry_under_stream_capture_allocates_nothing():
    """What the entry is for: a caller that records it into a graph.  After one warm call outside the capture (the
    first call on a device looks up the scratch address), the call is captured on a side stream -- an allocation, a
    host copy or a synchronisation inside it would fail the capture --, the graph is replayed twice with eager work
    in between, and every replay gives the bits of the allocating entry point."""
    seqlen, dim, mype, npes = [512, 384, 512], 128, 2, 3
    g = torch.Generator(device="cpu").manual_seed(11)
    k = torch.randn(sum(seqlen), dim, generator=g).bfloat16().cuda()
    v = torch.randn(sum(seqlen), dim, generator=g).bfloat16().cuda()
    q = torch.randn(seqlen[mype], dim, generator=g).bfloat16().cuda()
    ref, out = torch.empty_like(q), torch.empty_like(q)
    lse_ref = torch.empty(seqlen[mype], dtype=torch.float32, device="cuda")
    lse = torch.empty_like(lse_ref)
    api.ring_attention(q, k, v, ref, npes, mype, seqlen, dim, max(seqlen), lse=lse_ref, causal=True)
    api.ring_attention_noalloc(q, k, v, out, npes, mype, seqlen, dim, max(seqlen), lse=lse, causal=True)   # warm
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        api.ring_attention_noalloc(q, k, v, out, npes, mype, seqlen, dim, max(seqlen), lse=lse, causal=True, stream=side)
    for _ in range(2):
        out.fill_(5.0)
        lse.fill_(5.0)
        (k.float() @ v.float().t()).sum().item()      # the program's own eager work and a synchronisation in between
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
        assert torch.equal(lse.view(torch.int32), lse_ref.view(torch.int32))


def test_noalloc_calls_in_flight_on_several_streams():
    """Each call's table takes its own slice of the scratch, so a handful of calls may be in flight at once."""
    dim, npes = 128, 4
    seqlen = [1024] * npes
    gen = torch.Generator(device="cpu").manual_seed(12)
    k = torch.randn(sum(seqlen), dim, generator=gen).half().cuda()
    v = torch.randn(sum(seqlen), dim, generator=gen).half().cuda()
    qs = [torch.randn(1024, dim, generator=gen).half().cuda() for _ in range(npes)]
    refs = [torch.empty_like(x) for x in qs]
    outs = [torch.empty_like(x) for x in qs]
    for r in range(npes):
        api.ring_attention(qs[r], k, v, refs[r], npes, r, seqlen, dim, 1024, causal=True)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(npes)]
    for rep in range(3):
        for r in range(npes):
            api.ring_attention_noalloc(qs[r], k, v, outs[r], npes, r, seqlen, dim, 1024, causal=True, stream=streams[r])
    for s in streams:
        s.synchronize()
    for r in range(npes):
        assert torch.equal(outs[r].view(torch.int16), refs[r].view(torch.int16)), r
