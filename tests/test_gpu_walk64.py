"""ring_walk64_kernel (64 query rows per wave, d = 128, carried softmax state; ringattn_walk64.hip) against the CPU
oracle on inputs chosen for its own corner cases, and against ring_walk_kernel on the same inputs.

The kernel takes the exponentials of a tile against the reference maximum as it stands and only looks at the row
maximum (moving the reference, rescaling l and acc-O as in csrc/ring_attention.cu:226-232, redoing the tile) when a sum
of four of them exceeds 2^14.  Logits that keep rising along the key sequence force that path again and again: in the
steady iterations, in the masked tiles of a diagonal chunk and in a wave's last iterations.  Same tolerances as
everywhere: max-abs 1e-2 on O, 1e-3 relative on LSE (test_gpu_parity.check_rows)."""
import numpy as np
import pytest
import torch

from np_reference import bits_to_float64, float32_to_bits
from ringattention_amd import api
from ringattention_amd.configs import Workload
from test_gpu_parity import check_rows, forward

pytestmark = pytest.mark.gpu


def rising_logits(w, slope, period=0):
    """Q, K, V of workload `w` with one coordinate of K growing along the sequence (or sawtooth-wise with `period`)
    and the same coordinate of Q fixed at 4: logit(q, key j) grows by 4 * slope * scale per key."""
    q, k, v = api.make_qkv_bits(w)
    qf = bits_to_float64(q, w.dtype).astype(np.float32)
    kf = bits_to_float64(k, w.dtype).astype(np.float32)
    j = np.arange(w.seq, dtype=np.float32)
    if period:
        j = j % period
    qf[..., 0] = 4.0
    kf[..., 0] = slope * j
    return float32_to_bits(qf, w.dtype).reshape(q.shape), float32_to_bits(kf, w.dtype).reshape(k.shape), v


@pytest.mark.parametrize("w,slope,period", [
    # the row maximum climbs by about 400 (natural units) over the sequence: dozens of reference moves per row
    (Workload("rise_nc", 1, 2, 128, 4, 1024, "bf16", 41, False), 0.28, 0),
    (Workload("rise_c", 1, 2, 128, 4, 1024, "bf16", 42, True), 0.28, 0),
    (Workload("rise_c16", 2, 1, 128, 2, 1280, "fp16", 43, True), 0.1, 0),
    # a sawtooth: the maximum jumps at every tooth's end and nothing later in the tooth reaches it
    (Workload("saw_nc", 1, 3, 128, 3, 768, "fp16", 44, False), 0.4, 300),
    # steep enough for the exponentials to overflow to infinity against a stale reference
    (Workload("steep_c", 1, 1, 128, 2, 1024, "bf16", 45, True), 4.0, 0),
    # the d = 64 instantiation (half the MFMAs per tile, 4 KB tiles)
    (Workload("rise64_c", 1, 2, 64, 4, 1024, "bf16", 46, True), 0.2, 0),
    (Workload("saw64_nc", 2, 1, 64, 3, 768, "fp16", 47, False), 0.3, 300),
], ids=lambda x: x.name if isinstance(x, Workload) else None)
def test_reference_moves_inside_the_hand_scheduled_loop(oracle, w, slope, period):
    q, k, v = rising_logits(w, slope, period)
    out, lse = forward(w, q, k, v)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    check_rows(oracle, w, q, k, v, out, lse, np.arange(w.rows))


@pytest.mark.parametrize("w", [
    Workload("w_nc", 2, 3, 128, 4, 512, "bf16", 51, False),
    Workload("w_c", 1, 4, 128, 8, 256, "fp16", 52, True),          # 8-tile chunks: a change of chunk every other trip
    Workload("w_c1", 1, 2, 128, 1, 2048, "bf16", 53, True),        # one chunk, all of it diagonal
    Workload("w_min", 1, 2, 128, 4, 128, "bf16", 54, True),        # the shortest chunks the kernel takes (4 tiles)
    Workload("w_big", 1, 2, 128, 2, 1024, "fp16", 55, False, sigma_qk=3.0),
    Workload("w_tiny", 1, 2, 128, 1, 128, "bf16", 56, True),       # half a q tile: two waves own no row at all
    Workload("w_short", 2, 1, 128, 2, 160, "fp16", 57, False),     # heads shorter than what the load streams run ahead
    Workload("w64_nc", 2, 3, 64, 4, 512, "fp16", 58, False),       # d = 64
    Workload("w64_c", 1, 4, 64, 8, 256, "bf16", 59, True),
    Workload("w64_tiny", 1, 2, 64, 1, 128, "fp16", 60, True),
    Workload("w64_big", 1, 2, 64, 2, 1024, "fp16", 61, False, sigma_qk=3.0),
], ids=lambda w: w.name)
def test_both_kernels_agree(oracle, w, monkeypatch):
    """The same forward with and without RINGATTN_WIDE=0 (which keeps it on ring_walk_kernel): both against the oracle,
    and against each other within two units in the last place of the row's largest element (the two kernels move
    their reference maxima at different times, so the probabilities are rounded at different scales)."""
    q, k, v = api.make_qkv_bits(w)
    monkeypatch.delenv("RINGATTN_WIDE", raising=False)
    out_w, lse_w = forward(w, q, k, v)
    check_rows(oracle, w, q, k, v, out_w, lse_w, np.arange(w.rows))
    monkeypatch.setenv("RINGATTN_WIDE", "0")
    out_b, lse_b = forward(w, q, k, v)
    check_rows(oracle, w, q, k, v, out_b, lse_b, np.arange(w.rows))
    a, b = out_w.double().cpu().numpy().reshape(-1, w.dim), out_b.double().cpu().numpy().reshape(-1, w.dim)
    big = np.maximum(np.abs(a), np.abs(b)).max(axis=1, keepdims=True)
    mant = 10 if w.dtype == "fp16" else 7
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(big, 2.0 ** -14))) - mant)
    assert (np.abs(a - b) <= 2 * ulp).all()
    assert np.abs(lse_w.double().cpu().numpy() - lse_b.double().cpu().numpy()).max() <= 1e-4


def test_wide_kernel_with_grouped_heads_and_unequal_ranks(oracle):
    """Shapes the kernel takes beyond plain equal chunks: grouped-query heads and ranks of different lengths
    (multiples of 32, at least 128).  (The zigzag layout at d = 128 is covered by test_gpu_parity.test_zigzag_layout.)"""
    # grouped-query heads
    w = Workload("w_gqa", 1, 4, 128, 4, 512, "bf16", 61, True)
    q, k, v = api.make_qkv_bits(w)
    k, v = k[:, :2].copy(), v[:, :2].copy()
    plan = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, kv_heads=2)
    try:
        out, lse = plan.forward(*(api.bits_to_tensor(x, w.dtype) for x in (q, k, v)))
        torch.cuda.synchronize()
    finally:
        plan.close()
    k_full, v_full = np.repeat(k, 2, axis=1), np.repeat(v, 2, axis=1)
    check_rows(oracle, w, q, k_full, v_full, out, lse, np.arange(w.rows))
    # ranks of different lengths
    seqlen = (512, 128, 384, 160)
    S = sum(seqlen)
    wu = Workload("w_uneq", 1, 2, 128, 1, S, "fp16", 62, True)
    q, k, v = api.make_qkv_bits(wu)
    plan = api.RingAttention(len(seqlen), list(seqlen), 128, 1, 2, "fp16", True)
    try:
        out, lse = plan.forward(*(api.bits_to_tensor(x, "fp16") for x in (q, k, v)))
        torch.cuda.synchronize()
    finally:
        plan.close()
    check_rows(oracle, wu, q, k, v, out, lse, np.arange(wu.rows))


@pytest.mark.parametrize("w,half", [
    (Workload("p_nc", 1, 3, 128, 4, 512, "bf16", 71, False), False),
    (Workload("p_c", 2, 2, 128, 4, 384, "fp16", 72, True), False),
    (Workload("p_c_half", 1, 2, 128, 8, 256, "fp16", 73, True), True),
    (Workload("p_min", 1, 2, 128, 3, 128, "bf16", 74, True), False),   # four-tile chunks, a q tile and a half per head
    (Workload("p_rise", 1, 2, 128, 2, 1024, "bf16", 75, True), False),
], ids=lambda x: x.name if isinstance(x, Workload) else None)
def test_chunk_by_chunk_walk_with_partials(oracle, w, half, monkeypatch):
    """The forward that keeps the ring steps apart (a partial (O, LSE) per chunk, merged at the end) on
    ring_walk64_kernel, which then walks every chunk as a sequence of its own: against the oracle, against the same
    forward on ring_walk_kernel (RINGATTN_WIDE_PARTIALS=0), and, bit for bit, against the steps launched one by one
    with a separate merge.  (RINGATTN_WIDE_PARTIALS=1: left to itself the library takes this kernel for per-step
    partials only in causal forwards with at least 2048 keys per chunk.)"""
    q, k, v = rising_logits(w, 0.25) if w.name == "p_rise" else api.make_qkv_bits(w)
    qd, kd, vd = (api.bits_to_tensor(x, w.dtype) for x in (q, k, v))

    def run():
        plan = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, step_partials=True,
                                 half_partials=half)
        try:
            out, lse = plan.forward(qd, kd, vd)
            o_shape, l_shape = plan.parts_shapes()
            o_parts = torch.zeros(o_shape, dtype=plan.part_dtype, device="cuda")
            l_parts = torch.full(l_shape, float("-inf"), dtype=torch.float32, device="cuda")
            for s in range(w.npes):
                plan.block_forward(s, qd, kd, vd, o_parts[s], l_parts[s])
            out_m, lse_m = plan.merge_ring(o_parts, l_parts)
            torch.cuda.synchronize()
        finally:
            plan.close()
        assert torch.equal(out.view(torch.int16), out_m.view(torch.int16)) and torch.equal(lse, lse_m)
        return out, lse

    monkeypatch.delenv("RINGATTN_WIDE", raising=False)
    monkeypatch.setenv("RINGATTN_WIDE_PARTIALS", "1")
    out_w, lse_w = run()
    check_rows(oracle, w, q, k, v, out_w, lse_w, np.arange(w.rows))
    monkeypatch.setenv("RINGATTN_WIDE_PARTIALS", "0")
    out_b, lse_b = run()
    a, b = out_w.double().cpu().numpy().reshape(-1, w.dim), out_b.double().cpu().numpy().reshape(-1, w.dim)
    big = np.maximum(np.abs(a), np.abs(b)).max(axis=1, keepdims=True)
    mant = 10 if w.dtype == "fp16" else 7
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(big, 2.0 ** -14))) - mant)
    assert (np.abs(a - b) <= (3 if half else 2) * ulp).all()
    assert np.abs(lse_w.double().cpu().numpy() - lse_b.double().cpu().numpy()).max() <= 1e-4


def test_first_launch_of_a_process_gives_the_bits_of_later_ones():
    """A forward as the very first kernel of a fresh process (cold instruction cache and address translation: the waves
    of a workgroup then drift apart as they never do later) against the same forward repeated: bit for bit.  Four fresh
    processes, two with per-step partials and two with the state carried."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys, torch\n"
        "sys.path.insert(0, %r)\n"
        "from ringattention_amd import api\n"
        "from ringattention_amd.configs import Workload\n"
        "partials = sys.argv[1] == '1'\n"
        "w = Workload('first', 1, 3, 128, 4, 512, 'bf16', 71, not partials)\n"
        "q, k, v = (api.bits_to_tensor(x, w.dtype) for x in api.make_qkv_bits(w))\n"
        "plan = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, step_partials=partials)\n"
        "o1, l1 = plan.forward(q, k, v); torch.cuda.synchronize()\n"
        "o2, l2 = plan.forward(q, k, v); torch.cuda.synchronize()\n"
        "assert plan.forward_kernel() == 'ring_walk64_kernel'\n"
        "assert torch.equal(o1.view(torch.int16), o2.view(torch.int16)) and torch.equal(l1, l2)\n" % root)
    env = dict(os.environ, RINGATTN_WIDE_PARTIALS="1")
    env.pop("RINGATTN_WIDE", None)
    for partials in ("1", "0", "1", "0"):
        r = subprocess.run([sys.executable, "-c", code, partials], env=env, capture_output=True, text=True, timeout=110)
        assert r.returncode == 0, r.stderr[-2000:]


def test_wide_partials_in_row_major_and_rank_local_buffers(monkeypatch):
    """The chunk-by-chunk kernel writing caller-held partials: with a row's steps next to each other
    (RINGATTN_FLAG_ROW_PARTIALS), and into one rank's buffers with heads no longer than a chunk of 256 rows (the load
    streams then go round the head's first four tiles).  Bit for bit the forward that keeps its partials in the
    workspace."""
    monkeypatch.delenv("RINGATTN_WIDE", raising=False)
    monkeypatch.setenv("RINGATTN_WIDE_PARTIALS", "1")
    w = Workload("p_rows", 1, 2, 128, 4, 256, "bf16", 81, True)
    q, k, v = (api.bits_to_tensor(x, w.dtype) for x in api.make_qkv_bits(w))
    ref = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, step_partials=True)
    out, lse = ref.forward(q, k, v)
    assert ref.forward_kernel() == "ring_walk64_kernel"
    ref.close()
    plan = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, row_partials=True)
    o_shape, l_shape = plan.parts_shapes()
    o_parts = torch.zeros(o_shape, dtype=plan.part_dtype, device="cuda")
    l_parts = torch.full(l_shape, float("-inf"), dtype=torch.float32, device="cuda")
    for s in range(w.npes):
        plan.block_forward(s, q, k, v, o_parts, l_parts)
    out_r, lse_r = plan.merge_ring(o_parts, l_parts)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), out_r.view(torch.int16)) and torch.equal(lse, lse_r)
    plan.close()
    plan = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal)
    c = w.chunk
    for r in range(w.npes):
        q_r = q[:, :, r * c:(r + 1) * c].contiguous()
        o_shape, l_shape = plan.rank_parts_shapes(r)
        o_parts = torch.zeros(o_shape, dtype=plan.part_dtype, device="cuda")
        l_parts = torch.full(l_shape, float("-inf"), dtype=torch.float32, device="cuda")
        for s in range(w.npes):
            j = (r + s) % w.npes
            plan.rank_step_forward(r, s, q_r, k[:, :, j * c:(j + 1) * c].contiguous(), v[:, :, j * c:(j + 1) * c].contiguous(),
                                   o_parts[s], l_parts[s])
        o_r, l_r = plan.rank_merge(r, o_parts, l_parts)
        torch.cuda.synchronize()
        assert torch.equal(o_r.view(torch.int16), out[:, :, r * c:(r + 1) * c].view(torch.int16)), f"rank {r}"
        assert torch.equal(l_r, lse[:, :, r * c:(r + 1) * c]), f"rank {r}"
    plan.close()


def test_random_wide_plans_against_oracle(oracle, monkeypatch):
    """A seeded sweep over the shapes ring_walk64_kernel takes: 1 to 8 ranks of 128 to 1024 tokens each (multiples of
    32, unequal), batch, grouped heads, both head dimensions and types, the causal mask in both layouts, an explicit scale,
    graph replay, the state carried or per-step partials (on this kernel at d = 128: RINGATTN_WIDE_PARTIALS=1).  Every plan
    must report this kernel (d = 64 with per-step partials: the other one); up to 3000 rows of each (the first and the last
    q tile of a head, chunk edges, random ones) against the oracle."""
    monkeypatch.delenv("RINGATTN_WIDE", raising=False)
    monkeypatch.setenv("RINGATTN_WIDE_PARTIALS", "1")
    rng = np.random.default_rng(4242)
    for case in range(60):
        P = int(rng.integers(1, 9))
        causal = bool(rng.integers(0, 2))
        zigzag = causal and bool(rng.integers(0, 2))
        lens = [32 * int(rng.integers(4, 33)) for _ in range(P)]
        if zigzag:
            lens = [64 * max(4, c // 64) for c in lens]      # both halves of a rank: multiples of 32, at least 128
        dtype = str(rng.choice(["fp16", "bf16"]))
        d = 64 if case % 4 == 1 else 128
        B, hkv, group = int(rng.integers(1, 3)), int(rng.integers(1, 3)), int(rng.integers(1, 3))
        H, S = hkv * group, sum(lens)
        scale = float(rng.choice([0.0, 0.0, 0.05]))
        graph = bool(rng.integers(0, 2))
        steps_apart = case % 3 == 2
        tag = (f"case {case}: P={P} lens={lens} B={B} H={H} hkv={hkv} d={d} {dtype} causal={causal} zigzag={zigzag} "
               f"scale={scale} graph={graph} step_partials={steps_apart}")
        print(tag, flush=True)
        w = Workload("wide_rand", B, H, d, 1, S, dtype, 3000 + case, causal)
        q, _, _ = api.make_qkv_bits(w)
        _, k, v = api.make_qkv_bits(Workload("wide_rand_kv", B, hkv, d, 1, S, dtype, 4000 + case, causal))
        order = api.zigzag_order(lens) if zigzag else np.arange(S)
        inv = torch.from_numpy(np.argsort(order)).cuda()
        qd, kd, vd = (api.bits_to_tensor(np.ascontiguousarray(x[:, :, order]), dtype) for x in (q, k, v))
        plan = api.RingAttention(P, lens, d, B, H, dtype, causal, softmax_scale=scale, graph=graph,
                                 kv_heads=hkv if group > 1 else 0, layout="zigzag" if zigzag else "contiguous",
                                 step_partials=steps_apart)
        try:
            assert plan.forward_kernel() == ("ring_walk_kernel" if d == 64 and steps_apart else "ring_walk64_kernel"), tag
            out, lse = plan.forward(qd, kd, vd)
            if graph:
                out2, lse2 = plan.forward(qd, kd, vd, torch.empty_like(out), torch.empty_like(lse))
                torch.cuda.synchronize()
                assert torch.equal(out, out2) and torch.equal(lse, lse2), tag
            torch.cuda.synchronize()
        finally:
            plan.close()
        rows = np.arange(w.rows)
        if len(rows) > 3000:
            head = rows[:S]
            edges = np.concatenate([np.cumsum(lens)[:-1] + o for o in (-1, 0, 1)]) if P > 1 else np.zeros(0, int)
            pick = np.concatenate([head[:256], head[-256:], edges, (B * H - 1) * S + head[-256:],
                                   rng.choice(rows, 2000, replace=False)])
            rows = np.unique(pick.astype(np.int64))
        k_full, v_full = (np.repeat(x, group, axis=1) for x in (k, v))
        check_rows(oracle, w, q, k_full, v_full, out[:, :, inv].contiguous(), lse[:, :, inv].contiguous(), rows,
                   scale=scale if scale > 0 else None)
