"""Pins oracle/attention_oracle.c (the CPU checker) against things it shares no code with:
library routines (torch CPU float64, scipy), brute force, closed forms and invariants.
Each check is chosen so that a plausible slip in the oracle -- a dropped scale, base-2
instead of base-e, an off-by-one causal mask, a transposed operand, a missing rescale of
the running sum -- makes it fail."""
import math
import os

import numpy as np
import pytest
import scipy.special
import torch

from np_reference import bits_to_float64, float32_to_bits, np_make_qkv, torch_attention
from ringattention_amd.configs import WORKLOADS, Workload

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def rand_bits(rng, shape, dtype, sigma=1.0):
    return float32_to_bits((sigma * rng.standard_normal(shape)).astype(np.float32), dtype)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 1, 96, 64), (2, 3, 160, 128), (1, 2, 33, 16)])
def test_direct_matches_torch_library(oracle, dtype, causal, shape):
    rng = np.random.default_rng(hash((dtype, causal, shape)) % 2**32)
    q, k, v = (rand_bits(rng, shape, dtype) for _ in range(3))
    o, lse = oracle.attention_rows(q, k, v, dtype, causal=causal)
    o_ref, lse_ref = torch_attention(q, k, v, dtype, causal=causal)
    assert np.abs(o - o_ref.reshape(-1, shape[-1])).max() < 1e-13
    assert np.abs(lse - lse_ref.reshape(-1)).max() < 1e-12


def test_direct_matches_scipy_with_explicit_scale(oracle):
    rng = np.random.default_rng(5)
    q, k, v = (rand_bits(rng, (1, 1, 40, 32), "fp16") for _ in range(3))
    scale = 0.37  # not 1/sqrt(d): catches a hard-wired scale
    o, lse = oracle.attention_rows(q, k, v, "fp16", scale=scale)
    qf, kf, vf = (bits_to_float64(x, "fp16")[0, 0] for x in (q, k, v))
    s = scale * qf @ kf.T
    assert np.abs(lse - scipy.special.logsumexp(s, axis=-1)).max() < 1e-12
    assert np.abs(o - scipy.special.softmax(s, axis=-1) @ vf).max() < 1e-13


def test_brute_force_tiny(oracle):
    rng = np.random.default_rng(1)
    B, H, S, d = 1, 2, 8, 4
    q, k, v = (rand_bits(rng, (B, H, S, d), "bf16") for _ in range(3))
    qf, kf, vf = (bits_to_float64(x, "bf16") for x in (q, k, v))
    for causal in (False, True):
        o, lse = oracle.attention_rows(q, k, v, "bf16", causal=causal)
        for h in range(H):
            for i in range(S):
                keys = range(i + 1) if causal else range(S)
                logits = [sum(qf[0, h, i, c] * kf[0, h, t, c] for c in range(d)) / math.sqrt(d) for t in keys]
                z = sum(math.exp(x) for x in logits)
                for c in range(d):
                    want = sum(math.exp(x) * vf[0, h, t, c] for x, t in zip(logits, keys)) / z
                    assert abs(o[h * S + i, c] - want) < 1e-14
                assert abs(lse[h * S + i] - math.log(z)) < 1e-13


def test_closed_forms(oracle):
    rng = np.random.default_rng(2)
    shape = (1, 2, 64, 32)
    S = shape[2]
    q, k, v = (rand_bits(rng, shape, "fp16") for _ in range(3))
    vf = bits_to_float64(v, "fp16")
    zero = np.zeros(shape, dtype=np.uint16)
    # Q = 0: uniform weights.  O = mean of visible V rows, LSE = ln(#visible keys)
    o, lse = oracle.attention_rows(zero, k, v, "fp16")
    assert np.abs(o.reshape(2, S, 32) - vf[0].mean(axis=1, keepdims=True)).max() < 1e-14
    assert np.abs(lse - math.log(S)).max() < 1e-14
    o, lse = oracle.attention_rows(zero, k, v, "fp16", causal=True)
    prefix = np.cumsum(vf[0], axis=1) / np.arange(1, S + 1)[None, :, None]
    assert np.abs(o.reshape(2, S, 32) - prefix).max() < 1e-14
    assert np.abs(lse.reshape(2, S) - np.log(np.arange(1, S + 1))[None]).max() < 1e-14
    # K = 0 gives the same as Q = 0
    o2, lse2 = oracle.attention_rows(q, zero, v, "fp16", causal=True)
    assert np.array_equal(o2, o) and np.array_equal(lse2, lse)
    # constant V: O is that constant whatever the weights are
    vc = np.full(shape, float32_to_bits(np.array([1.5], np.float32), "fp16")[0], dtype=np.uint16)
    o, _ = oracle.attention_rows(q, k, vc, "fp16")
    assert np.abs(o - 1.5).max() < 1e-14
    # causal row 0 sees only key 0: O = V[0], LSE = scale * q0.k0
    o, lse = oracle.attention_rows(q, k, v, "fp16", causal=True, rows=np.array([0, S]))
    qf, kf = bits_to_float64(q, "fp16"), bits_to_float64(k, "fp16")
    for x, h in enumerate((0, 1)):
        assert np.abs(o[x] - vf[0, h, 0]).max() == 0.0
        assert abs(lse[x] - (qf[0, h, 0] @ kf[0, h, 0]) / math.sqrt(32)) < 1e-14


def test_dominant_key_and_reference_fill(oracle, ralib):
    # the reference's own deterministic fill (csrc/ring_attention.cu:731-741) drives the
    # softmax into saturation: every query's weight collapses onto the last key
    import ctypes
    m, n = 256, 64
    buf = np.empty((m, n), dtype=np.uint16)
    assert ralib.ringattn_fill_reference_pattern(buf.ctypes.data_as(ctypes.c_void_p), 0, m, n) == 0
    want = np.fromfunction(lambda i, j: i / 130.0 + j / 110.0 + i * j / 600.0, (m, n)).astype(np.float32)
    assert np.array_equal(buf, float32_to_bits(want, "fp16"))
    x = buf.reshape(1, 1, m, n)
    o, lse = oracle.attention_rows(x, x, x, "fp16", rows=np.arange(64, m))
    vf = bits_to_float64(x, "fp16")[0, 0]
    assert np.abs(o - vf[-1]).max() < 1e-2  # rows past the first few dozen collapse onto key m-1


@pytest.mark.parametrize("causal", [False, True])
def test_ring_form_equals_direct_and_is_order_independent(oracle, causal):
    rng = np.random.default_rng(3)
    P, c, d = 4, 32, 16
    shape = (2, 2, P * c, d)
    q, k, v = (rand_bits(rng, shape, "bf16", 2.0) for _ in range(3))
    rows = rng.choice(2 * 2 * P * c, 64, replace=False)
    o, lse = oracle.attention_rows(q, k, v, "bf16", causal=causal, rows=rows)
    o_r, lse_r = oracle.ring_rows(q, k, v, "bf16", [c] * P, rows, causal=causal, tile=8)
    assert np.abs(o_r - o).max() < 1e-13 and np.abs(lse_r - lse).max() < 1e-12
    for order in ([3, 1, 0, 2], [2, 3, 1, 0]):
        o_p, lse_p = oracle.ring_rows(q, k, v, "bf16", [c] * P, rows, causal=causal, tile=8, order=order)
        assert np.abs(o_p - o).max() < 1e-13 and np.abs(lse_p - lse).max() < 1e-12
    # unequal chunk lengths (per-rank seqlen[] of the reference, csrc/ring_attention.cu:753)
    o_u, lse_u = oracle.ring_rows(q, k, v, "bf16", [40, 24, 8, 56], rows, causal=causal, tile=16)
    assert np.abs(o_u - o).max() < 1e-13 and np.abs(lse_u - lse).max() < 1e-12


def test_ring_partials_follow_the_ring_schedule(oracle):
    # rank r at step s holds the partial against chunk (r + s) mod P
    rng = np.random.default_rng(4)
    P, c, d = 3, 16, 8
    q, k, v = (rand_bits(rng, (1, 1, P * c, d), "fp16") for _ in range(3))
    rows = np.array([5, c + 3, 2 * c + 9])
    _, _, po, pl = oracle.ring_rows(q, k, v, "fp16", [c] * P, rows, tile=4, want_parts=True)
    qf, kf, vf = (bits_to_float64(x, "fp16")[0, 0] for x in (q, k, v))
    for x, row in enumerate(rows):
        r = row // c
        for s in range(P):
            j = (r + s) % P
            sl = slice(j * c, (j + 1) * c)
            logits = (kf[sl] @ qf[row]) / math.sqrt(d)
            assert abs(pl[x, s] - scipy.special.logsumexp(logits)) < 1e-13
            assert np.abs(po[x, s] - scipy.special.softmax(logits) @ vf[sl]).max() < 1e-14


def test_causal_ring_partials_against_scipy(oracle):
    # causal ring, unequal chunks: rank r at step s meets chunk j = (r + s) mod P; j > r gives no
    # partial (LSE -inf), j == r the keys up to the row's own position, j < r the whole chunk
    rng = np.random.default_rng(14)
    seqlen, d = [12, 20, 8, 16], 8
    P, S = len(seqlen), sum(seqlen)
    start = np.concatenate([[0], np.cumsum(seqlen)])
    q, k, v = (rand_bits(rng, (1, 2, S, d), "bf16") for _ in range(3))
    rows = np.arange(2 * S)
    o, lse, po, pl = oracle.ring_rows(q, k, v, "bf16", seqlen, rows, causal=True, tile=5, want_parts=True)
    qf, kf, vf = (bits_to_float64(x, "bf16") for x in (q, k, v))
    for x in rows:
        h, pos = divmod(int(x), S)
        r = int(np.searchsorted(start, pos, side="right") - 1)
        seen = 0
        for s in range(P):
            j = (r + s) % P
            if j > r:
                assert pl[x, s] == -np.inf
                continue
            hi = pos + 1 if j == r else start[j + 1]
            sl = slice(start[j], hi)
            seen += hi - start[j]
            logits = (kf[0, h, sl] @ qf[0, h, pos]) / math.sqrt(d)
            assert abs(pl[x, s] - scipy.special.logsumexp(logits)) < 1e-13
            assert np.abs(po[x, s] - scipy.special.softmax(logits) @ vf[0, h, sl]).max() < 1e-14
        assert seen == pos + 1                    # the visible steps cover keys 0..pos exactly once
    # and the merged rows equal plain causal attention
    o_ref, lse_ref = torch_attention(q, k, v, "bf16", causal=True)
    assert np.abs(o - o_ref.reshape(-1, d)).max() < 1e-13 and np.abs(lse - lse_ref.reshape(-1)).max() < 1e-12


def test_block_partial_with_a_shifted_diagonal_against_scipy(oracle):
    # mask_mode 1 with diag_offset: key t visible to row i iff t <= i + diag_offset
    rng = np.random.default_rng(15)
    cq, ck, d, off = 10, 24, 16, 7
    q = rand_bits(rng, (cq, d), "fp16")
    k, v = (rand_bits(rng, (ck, d), "fp16") for _ in range(2))
    o, lse = oracle.block_partial(q, k, v, "fp16", mask_mode=1, diag_offset=off, tile=6)
    qf, kf, vf = (bits_to_float64(x, "fp16") for x in (q, k, v))
    for i in range(cq):
        logits = (kf[:i + off + 1] @ qf[i]) / math.sqrt(d)
        assert abs(lse[i] - scipy.special.logsumexp(logits)) < 1e-13
        assert np.abs(o[i] - scipy.special.softmax(logits) @ vf[:i + off + 1]).max() < 1e-14


def test_ring_rows_with_rounded_probabilities(oracle):
    # round_p: the PV product uses p rounded to the storage type, the row sum the unrounded p.
    # Rebuilt here with numpy on ONE tile per chunk (then the max is the chunk max and p = softmax numerators).
    rng = np.random.default_rng(16)
    P, c, d = 3, 16, 8
    q, k, v = (rand_bits(rng, (1, 1, P * c, d), "bf16") for _ in range(3))
    rows = np.array([0, 7, c + 2, 2 * c + 15])
    o, lse, po, pl = oracle.ring_rows(q, k, v, "bf16", [c] * P, rows, tile=c, round_p=True, want_parts=True)
    o_exact, lse_exact = oracle.ring_rows(q, k, v, "bf16", [c] * P, rows, tile=c)
    assert np.array_equal(lse, lse_exact)                     # sums come from the unrounded p
    qf, kf, vf = (bits_to_float64(x, "bf16")[0, 0] for x in (q, k, v))
    for x, row in enumerate(rows):
        r = row // c
        for s in range(P):
            j = (r + s) % P
            logits = (kf[j * c:(j + 1) * c] @ qf[row]) / math.sqrt(d)
            p = np.exp(logits - logits.max())
            p_rounded = bits_to_float64(float32_to_bits(p.astype(np.float32), "bf16"), "bf16")
            want = p_rounded @ vf[j * c:(j + 1) * c] / p.sum()
            assert np.abs(po[x, s] - want).max() < 1e-6       # p passes through float32 on its way to bf16 here
    assert 0 < np.abs(o - o_exact).max() < 2e-2


def test_block_partial_matches_library_and_rounding_of_p_is_small(oracle):
    rng = np.random.default_rng(6)
    c, d = 48, 32
    q, k, v = (rand_bits(rng, (c, d), "bf16") for _ in range(3))
    for mask_mode in (0, 1):
        o, lse = oracle.block_partial(q, k, v, "bf16", mask_mode=mask_mode, tile=16)
        o_ref, lse_ref = torch_attention(q[None, None], k[None, None], v[None, None], "bf16", causal=bool(mask_mode))
        assert np.abs(o - o_ref[0, 0]).max() < 1e-13 and np.abs(lse - lse_ref[0, 0]).max() < 1e-12
        o_rp, lse_rp = oracle.block_partial(q, k, v, "bf16", mask_mode=mask_mode, tile=16, round_p=True)
        assert np.array_equal(lse_rp, lse)            # the sum uses unrounded p
        assert 0 < np.abs(o_rp - o).max() < 2e-2      # bf16 p: ~2^-9 relative per term


def test_merge_algebra(oracle):
    rng = np.random.default_rng(7)
    n, rows, d = 5, 33, 8
    op = rng.standard_normal((n, rows, d))
    lp = 3.0 * rng.standard_normal((n, rows))
    o, lse = oracle.merge(op, lp)
    w = scipy.special.softmax(lp, axis=0)
    assert np.abs(lse - scipy.special.logsumexp(lp, axis=0)).max() < 1e-13
    assert np.abs(o - np.einsum("nr,nrd->rd", w, op)).max() < 1e-13
    # commutative
    perm = [3, 0, 4, 1, 2]
    o2, lse2 = oracle.merge(op[perm], lp[perm])
    assert np.abs(o2 - o).max() < 1e-14 and np.abs(lse2 - lse).max() < 1e-14
    # associative: merge(merge(a, b), c...) == merge(all)
    o_ab, l_ab = oracle.merge(op[:2], lp[:2])
    o3, lse3 = oracle.merge(np.concatenate([o_ab[None], op[2:]]), np.concatenate([l_ab[None], lp[2:]]))
    assert np.abs(o3 - o).max() < 1e-14 and np.abs(lse3 - lse).max() < 1e-13
    # identity element: a part with LSE = -inf changes nothing, whatever its O holds
    op_id = np.concatenate([op, np.full((1, rows, d), 7.0)])
    lp_id = np.concatenate([lp, np.full((1, rows), -np.inf)])
    o4, lse4 = oracle.merge(op_id, lp_id)
    assert np.array_equal(o4, o) and np.array_equal(lse4, lse)
    # a partial merged with itself: same O, LSE + ln 2
    o5, lse5 = oracle.merge(np.stack([op[0], op[0]]), np.stack([lp[0], lp[0]]))
    assert np.abs(o5 - op[0]).max() < 1e-15 and np.abs(lse5 - lp[0] - math.log(2)).max() < 1e-14
    # all parts empty
    o6, lse6 = oracle.merge(op[:2], np.full((2, rows), -np.inf))
    assert np.all(o6 == 0) and np.all(np.isneginf(lse6))


def test_storage_rounding_matches_torch(oracle):
    rng = np.random.default_rng(8)
    x32 = np.concatenate([rng.standard_normal(20000) * np.exp(rng.uniform(-12, 12, 20000)),
                          [0.0, -0.0, 65504.0, 65520.0, 1e-8, 6e-8, 3e-5, 1.0 + 2**-11, 1.0 + 3 * 2**-11]]).astype(np.float32)
    x = x32.astype(np.float64)  # exactly representable in float32: no double rounding on torch's side
    for dtype, tdt in (("fp16", torch.float16), ("bf16", torch.bfloat16)):
        got = oracle.round_to(x, dtype)
        want = torch.from_numpy(x32).to(tdt).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(got, want), dtype
        assert np.array_equal(oracle.widen(got, dtype), bits_to_float64(want, dtype))
    # a double that float32 rounding would push onto the wrong bf16 neighbour
    tricky = np.array([1.0 + 2.0**-8 + 2.0**-40])  # just above the bf16 midpoint of [1, 1 + 2^-7]
    assert oracle.widen(oracle.round_to(tricky, "bf16"), "bf16")[0] == 1.0 + 2.0**-7


def test_golden_fixtures(oracle):
    for name, w in (("cfg1", WORKLOADS["cfg1"]), ("causal_small", Workload("causal_small", 1, 2, 128, 2, 128, "bf16", 11, True))):
        g = np.load(os.path.join(GOLD, f"{name}_expected.npz"))
        q, k, v = np_make_qkv(w)
        o, lse = oracle.attention_rows(q, k, v, w.dtype, causal=w.causal)
        assert np.abs(o - g["o_f32"].reshape(-1, w.dim)).max() < 1e-6   # fixture stored as float32
        assert np.abs(lse - g["lse_f64"].reshape(-1)).max() < 1e-12
