"""The torch front end (dispatcher op ringattn::fwd over the C ABI)."""
import pytest
import torch

from ringattention_amd import api, torch_ops
from ringattention_amd.configs import Workload


def test_op_is_registered_and_checks_inputs_like_the_reference_header():
    torch_ops.load()
    schema = str(torch.ops.ringattn.fwd.default._schema)
    assert schema.startswith("ringattn::fwd(Tensor q, Tensor k, Tensor v, int[] seqlen")
    x = torch.zeros(1, 1, 256, 64, dtype=torch.float16)
    # include/attention_api.cuh:12-13: "#x must be a CUDA tensor" -- answered before any GPU work
    with pytest.raises(RuntimeError, match="q must be a CUDA tensor"):
        torch_ops.ring_attention_fwd(x, x, x, [128, 128])


@pytest.mark.gpu
def test_op_matches_the_c_abi_bit_for_bit():
    w = Workload("torch_op", 2, 4, 128, 4, 256, "bf16", 61, True)
    q, k, v = (api.bits_to_tensor(x, w.dtype) for x in api.make_qkv_bits(w))
    k2, v2 = k[:, :2].contiguous(), v[:, :2].contiguous()            # grouped-query: 2 KV heads for 4 query heads
    for kk, vv, kvh, zig in ((k, v, 0, False), (k2, v2, 2, False), (k, v, 0, True)):
        plan = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, True, kv_heads=kvh,
                                 layout="zigzag" if zig else "contiguous")
        o_ref, l_ref = plan.forward(q, kk, vv)
        for _ in range(2):                                           # second call reuses the cached plan
            out, lse = torch_ops.ring_attention_fwd(q, kk, vv, [w.chunk] * w.npes, causal=True, zigzag=zig)
            torch.cuda.synchronize()
            assert torch.equal(out, o_ref) and torch.equal(lse, l_ref)
        plan.close()
    side = torch.cuda.Stream()                                       # follows torch's current stream
    with torch.cuda.stream(side):
        out, lse = torch_ops.ring_attention_fwd(q, k, v, [w.chunk] * w.npes, causal=True)
    side.synchronize()
    plan = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, True)
    o_ref, _ = plan.forward(q, k, v)
    torch.cuda.synchronize()
    plan.close()
    assert torch.equal(out, o_ref)
    # CHECK_CONTIGUOUS (include/attention_api.cuh:14-15) and the shape checks
    with pytest.raises(RuntimeError, match="k must be contiguous"):
        torch_ops.ring_attention_fwd(q, k.transpose(2, 3).contiguous().transpose(2, 3), v, [w.chunk] * w.npes)
    with pytest.raises(RuntimeError, match="seqlen must sum to S"):
        torch_ops.ring_attention_fwd(q, k, v, [w.chunk] * (w.npes - 1))
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        torch_ops.ring_attention_fwd(q.float(), k.float(), v.float(), [w.chunk] * w.npes)


@pytest.mark.gpu
def test_two_streams_with_the_same_shapes_do_not_share_a_workspace():
    # forwards of the same shape issued on two streams at once: each stream has its own plan and
    # workspace, so both results are bit-equal to what the same calls give one after the other
    w = Workload("torch_two_streams", 1, 8, 128, 8, 512, "bf16", 62, True)
    seqlen = [w.chunk] * w.npes
    qa, ka, va = (api.bits_to_tensor(x, w.dtype) for x in api.make_qkv_bits(w))
    qb, kb, vb = (api.bits_to_tensor(x, w.dtype) for x in api.make_qkv_bits(Workload("other", 1, 8, 128, 8, 512, "bf16", 63, True)))
    ref_a = torch_ops.ring_attention_fwd(qa, ka, va, seqlen, causal=True)
    ref_b = torch_ops.ring_attention_fwd(qb, kb, vb, seqlen, causal=True)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    res_a, res_b = [], []
    for _ in range(6):
        with torch.cuda.stream(s1):
            res_a.append(torch_ops.ring_attention_fwd(qa, ka, va, seqlen, causal=True))
        with torch.cuda.stream(s2):
            res_b.append(torch_ops.ring_attention_fwd(qb, kb, vb, seqlen, causal=True))
    s1.synchronize()
    s2.synchronize()
    for out, lse in res_a:
        assert torch.equal(out, ref_a[0]) and torch.equal(lse, ref_a[1])
    for out, lse in res_b:
        assert torch.equal(out, ref_b[0]) and torch.equal(lse, ref_b[1])


@pytest.mark.gpu
def test_plan_cache_is_bounded():
    # more distinct shapes than the cache holds: old plans are destroyed, results stay right
    w = Workload("torch_cache", 1, 2, 64, 2, 128, "fp16", 64, False)
    q, k, v = (api.bits_to_tensor(x, w.dtype) for x in api.make_qkv_bits(w))
    free0 = torch.cuda.mem_get_info()[0]
    first = None
    for i in range(40):
        seqlen = [128 + 2 * i, 128 - 2 * i]                       # 40 different plans
        out, lse = torch_ops.ring_attention_fwd(q, k, v, seqlen)
        if i == 0:
            first = (out.clone(), lse.clone())
    out, lse = torch_ops.ring_attention_fwd(q, k, v, [128, 128])    # the first plan again (evicted by now, re-created)
    torch.cuda.synchronize()
    assert torch.equal(out, first[0]) and torch.equal(lse, first[1])
    # 40 plans of ~0.27 MB workspace each would not show here anyway; the point is that nothing grows without bound
    assert free0 - torch.cuda.mem_get_info()[0] < (256 << 20)
