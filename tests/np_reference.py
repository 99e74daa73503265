"""Independent restatements used to pin the C oracle and the C input generator.

Nothing here shares code with oracle/attention_oracle.c or with the product library:
  * np_fill_normal   -- the seeded generator (splitmix64 counters -> Box-Muller -> float32
                        -> fp16/bf16), written with numpy integer arithmetic;
  * torch_attention  -- softmax(scale Q K^T [+ mask]) V and logsumexp with torch CPU
                        float64 library routines (matmul, softmax, logsumexp), the math of
                        the reference's csrc/self_attention.py:22-26 plus scale and mask;
  * bits <-> float helpers built on numpy / torch dtype conversion.
"""
import numpy as np
import torch

GAMMA = np.uint64(0x9E3779B97F4A7C15)


def _mix64(z):
    z = z.astype(np.uint64)
    z ^= z >> np.uint64(30)
    z *= np.uint64(0xBF58476D1CE4E5B9)
    z ^= z >> np.uint64(27)
    z *= np.uint64(0x94D049BB133111EB)
    z ^= z >> np.uint64(31)
    return z


def float32_to_bits(f32, dtype):
    f32 = np.ascontiguousarray(f32, dtype=np.float32)
    if dtype == "fp16":
        return f32.astype(np.float16).view(np.uint16)
    u = f32.view(np.uint32).astype(np.uint64)
    u = u + np.uint64(0x7FFF) + ((u >> np.uint64(16)) & np.uint64(1))
    return (u >> np.uint64(16)).astype(np.uint16)


def bits_to_float64(bits, dtype):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    if dtype == "fp16":
        return bits.view(np.float16).astype(np.float64)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32).astype(np.float64)


def np_fill_normal(n, dtype, seed, offset=0, sigma=1.0):
    with np.errstate(over="ignore"):
        key = _mix64(np.array([seed], dtype=np.uint64) + GAMMA)[0]
        e = np.arange(offset, offset + n, dtype=np.uint64)
        x1 = _mix64(key + (np.uint64(2) * e + np.uint64(1)) * GAMMA)
        x2 = _mix64(key + (np.uint64(2) * e + np.uint64(2)) * GAMMA)
    u1 = ((x1 >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)
    u2 = ((x2 >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(6.283185307179586476925286766559 * u2)
    return float32_to_bits((sigma * z).astype(np.float32), dtype)


def np_make_qkv(w):
    n = w.batch * w.heads * w.seq * w.dim
    shape = (w.batch, w.heads, w.seq, w.dim)
    q = np_fill_normal(n, w.dtype, w.seed, 0, w.sigma_qk).reshape(shape)
    k = np_fill_normal(n, w.dtype, w.seed, n, w.sigma_qk).reshape(shape)
    v = np_fill_normal(n, w.dtype, w.seed, 2 * n, w.sigma_v).reshape(shape)
    return q, k, v


def torch_attention(q_bits, k_bits, v_bits, dtype, causal=False, scale=None):
    """Library-routine attention in float64.  Inputs uint16 [B, H, S, d].  Returns (O, LSE) numpy."""
    q = torch.from_numpy(bits_to_float64(q_bits, dtype))
    k = torch.from_numpy(bits_to_float64(k_bits, dtype))
    v = torch.from_numpy(bits_to_float64(v_bits, dtype))
    d = q.shape[-1]
    scale = d ** -0.5 if scale is None else scale
    s = torch.matmul(q, k.transpose(-1, -2)) * scale
    if causal:
        S = q.shape[-2]
        mask = torch.ones(S, S, dtype=torch.bool).tril()
        s = s.masked_fill(~mask, float("-inf"))
    o = torch.matmul(torch.softmax(s, dim=-1), v)
    lse = torch.logsumexp(s, dim=-1)
    return o.numpy(), lse.numpy()
