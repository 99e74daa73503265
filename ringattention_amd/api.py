"""Host-side mirror of the reference's entry points on top of the C ABI.

`RingAttention` is a plan (parameters + workspace, created once) with `forward`,
`block_forward` and `merge` methods; `ring_attention` has the reference's
`ring_attention(q, k, v, out, npes, mype, seqlen, dim, max_seq)` argument list
(csrc/ring_attention.cu:706).  torch is used only to own device memory and to name
the stream; every computation goes through libringattn.so.
"""
import ctypes

import numpy as np
import torch

from . import _lib
from ._lib import RingattnParams, check

DTYPE_CODE = {"fp16": 0, "bf16": 1, torch.float16: 0, torch.bfloat16: 1}
TORCH_DTYPE = {0: torch.float16, 1: torch.bfloat16}
FLAG_GRAPH = 1
FLAG_TIMING = 2
FLAG_HALF_PARTIALS = 4
FLAG_STEP_PARTIALS = 8
FLAG_ROW_PARTIALS = 16
LAYOUT_CODE = {"contiguous": 0, "zigzag": 1}


def _stream_ptr(stream=None):
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _check_meta(t, name, dtype=None, shape=None):
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, not {tuple(t.shape)}")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{name} must have dtype {dtype}")


def _check_place(t, name):
    if not t.is_cuda:
        raise ValueError(f"{name} must be a device tensor")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _check_tensors(*specs):
    """specs: (tensor, name, dtype or None, shape or None).  Shapes and dtypes of ALL tensors against
    what the plan expects first (the C ABI sees raw pointers only: a wrongly sized buffer would become
    an out-of-bounds access on the device), then the conventions of include/attention_api.cuh:12-18:
    device-resident and contiguous."""
    for t, name, dtype, shape in specs:
        _check_meta(t, name, dtype, shape)
    for t, name, _, _ in specs:
        _check_place(t, name)


def _check_tensor(t, name, dtype=None, shape=None):
    _check_tensors((t, name, dtype, shape))


def make_params(npes, seqlen, dim, batch=1, heads=1, dtype="fp16", causal=False, softmax_scale=0.0, flags=0,
                kv_heads=0, layout=0):
    arr = (ctypes.c_int * len(seqlen))(*[int(x) for x in seqlen])
    p = RingattnParams(int(npes), ctypes.cast(arr, _lib.c_int_p), int(dim), float(softmax_scale), int(batch),
                       int(heads), DTYPE_CODE[dtype], int(bool(causal)), int(flags), int(kv_heads), int(layout))
    p._keepalive = arr
    return p


class RingAttention:
    """A forward plan for P virtual ring ranks on one GPU."""

    def __init__(self, npes, chunk, dim, batch=1, heads=1, dtype="fp16", causal=False, softmax_scale=0.0, graph=False,
                 kv_heads=0, layout="contiguous", timing=False, half_partials=False, workspace=None,
                 step_partials=False, row_partials=False):
        """`chunk`: tokens per rank -- one int for equal chunks or a list of npes lengths
        (the per-PE seqlen[] of csrc/ring_attention.cu:753).  `kv_heads`: heads of K and V for
        grouped-query attention (0 = same as `heads`).  `layout`: "contiguous" (rank r holds
        the tokens after those of rank r-1) or "zigzag" (rank r holds a low and a high
        half-chunk; see zigzag_order).  `step_partials`: forward() keeps the ring steps apart (a
        partial (O, LSE) per step in the workspace, merged at the end: the arithmetic of
        block_forward + merge_ring) instead of carrying the softmax state through all steps in
        registers.  `half_partials`: keep per-step partial O in fp16 (half the workspace and merge
        traffic; needs |V| < 65504).  `workspace`: a (device address, bytes) pair the caller owns
        and keeps alive, instead of an allocation by the plan (only a step_partials plan needs one).
        `row_partials`: caller-held per-step partials are [B, H, S, npes, d] / [B, H, S, npes] (a row's steps next to
        each other) instead of [npes, B, H, S, d] / [npes, B, H, S]; block_forward / rank_step_forward then take the
        whole buffers for every step."""
        self.lib = _lib.load()
        self.seqlen = [int(chunk)] * npes if isinstance(chunk, int) else [int(x) for x in chunk]
        if len(self.seqlen) != npes:
            raise ValueError("need one length per rank")
        self.npes, self.chunk, self.dim, self.batch, self.heads = npes, chunk, dim, batch, heads
        self.dtype_code = DTYPE_CODE[dtype]
        self.torch_dtype = TORCH_DTYPE[self.dtype_code]
        self.causal = bool(causal)
        self.part_dtype = torch.float16 if half_partials else torch.float32
        self.row_partials = bool(row_partials)
        self.seq = sum(self.seqlen)
        self.kv_heads = kv_heads if kv_heads else heads
        self.params = make_params(npes, self.seqlen, dim, batch, heads, dtype, causal, softmax_scale,
                                  (FLAG_GRAPH if graph else 0) | (FLAG_TIMING if timing else 0)
                                  | (FLAG_HALF_PARTIALS if half_partials else 0)
                                  | (FLAG_STEP_PARTIALS if step_partials else 0)
                                  | (FLAG_ROW_PARTIALS if row_partials else 0), kv_heads,
                                  LAYOUT_CODE[layout])
        self.handle = ctypes.c_void_p()
        ws_ptr, ws_bytes = (None, 0) if workspace is None else (ctypes.c_void_p(int(workspace[0])), int(workspace[1]))
        check(self.lib.ringattn_plan_create(ctypes.byref(self.params), ws_ptr, ws_bytes, ctypes.byref(self.handle)),
              "ringattn_plan_create")

    def close(self):
        if self.handle:
            check(self.lib.ringattn_plan_destroy(self.handle), "ringattn_plan_destroy")
            self.handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _shape(self):
        return (self.batch, self.heads, self.seq, self.dim)

    def parts_shapes(self):
        """Shapes of caller-held per-step partials (O, LSE) for merge_ring: slot-major, or a row's steps adjacent."""
        b, h, s, d = self._shape()
        if self.row_partials:
            return (b, h, s, self.npes, d), (b, h, s, self.npes)
        return (self.npes, b, h, s, d), (self.npes, b, h, s)

    def rank_parts_shapes(self, rank):
        """parts_shapes() for the rank-local calls (rank_step_forward, rank_merge): the rank's rows only."""
        b, h, rows, d = self.batch, self.heads, self.seqlen[rank], self.dim
        if self.row_partials:
            return (b, h, rows, self.npes, d), (b, h, rows, self.npes)
        return (self.npes, b, h, rows, d), (self.npes, b, h, rows)

    def _qkv_specs(self, q, k, v):
        kv_shape = (self.batch, self.kv_heads, self.seq, self.dim)
        return [(q, "q", self.torch_dtype, self._shape()), (k, "k", self.torch_dtype, kv_shape),
                (v, "v", self.torch_dtype, kv_shape)]

    def forward(self, q, k, v, out=None, lse=None, stream=None):
        _check_tensors(*self._qkv_specs(q, k, v))
        if out is None:
            out = torch.empty_like(q)
        if lse is None:
            lse = torch.empty(self._shape()[:3], dtype=torch.float32, device=q.device)
        _check_tensors((out, "out", self.torch_dtype, self._shape()), (lse, "lse", torch.float32, self._shape()[:3]))
        check(self.lib.ringattn_fwd(self.handle, _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _stream_ptr(stream)),
              "ringattn_fwd")
        return out, lse

    def block_forward(self, step, q, k, v, o_part=None, lse_part=None, stream=None):
        specs = self._qkv_specs(q, k, v)
        # slot-major partials: the slot of this step; row-major (row_partials): the whole buffers, for every step
        o_shape, l_shape = self.parts_shapes() if self.row_partials else (self._shape(), self._shape()[:3])
        if o_part is not None:
            specs.append((o_part, "o_part", self.part_dtype, o_shape))
        if lse_part is not None:
            specs.append((lse_part, "lse_part", torch.float32, l_shape))
        _check_tensors(*specs)
        if o_part is None:
            o_part = torch.zeros(o_shape, dtype=self.part_dtype, device=q.device)
        if lse_part is None:
            lse_part = torch.full(l_shape, float("-inf"), dtype=torch.float32, device=q.device)
        check(self.lib.ringattn_block_fwd(self.handle, int(step), _ptr(q), _ptr(k), _ptr(v), _ptr(o_part),
                                          _ptr(lse_part), _stream_ptr(stream)), "ringattn_block_fwd")
        return o_part, lse_part

    def rank_step_forward(self, rank, step, q, k_chunk, v_chunk, o_part=None, lse_part=None, stream=None):
        """One ring step of one rank on rank-local tensors (q: the rank's rows; k_chunk, v_chunk: the
        chunk of rank (rank + step) % npes).  Returns the rank-local partial (O, LSE); on a plan with row_partials
        o_part and lse_part are the rank's whole [B, H, rows, npes, d] / [B, H, rows, npes] buffers at every step."""
        if not (0 <= rank < self.npes and 0 <= step < self.npes):
            raise ValueError("rank and step must be in [0, npes)")
        rows, kv_rows = self.seqlen[rank], self.seqlen[(rank + step) % self.npes]
        o_shape, l_shape = (self.batch, self.heads, rows, self.dim), (self.batch, self.heads, rows)
        if self.row_partials:
            o_shape, l_shape = self.rank_parts_shapes(rank)
        specs = [(q, "q", self.torch_dtype, (self.batch, self.heads, rows, self.dim)),
                 (k_chunk, "k_chunk", self.torch_dtype, (self.batch, self.kv_heads, kv_rows, self.dim)),
                 (v_chunk, "v_chunk", self.torch_dtype, (self.batch, self.kv_heads, kv_rows, self.dim))]
        if o_part is not None:
            specs.append((o_part, "o_part", self.part_dtype, o_shape))
        if lse_part is not None:
            specs.append((lse_part, "lse_part", torch.float32, l_shape))
        _check_tensors(*specs)
        if o_part is None:
            o_part = torch.zeros(o_shape, dtype=self.part_dtype, device=q.device)
        if lse_part is None:
            lse_part = torch.full(l_shape, float("-inf"), dtype=torch.float32, device=q.device)
        check(self.lib.ringattn_rank_step_fwd(self.handle, int(rank), int(step), _ptr(q), _ptr(k_chunk), _ptr(v_chunk),
                                              _ptr(o_part), _ptr(lse_part), _stream_ptr(stream)), "ringattn_rank_step_fwd")
        return o_part, lse_part

    def rank_merge(self, rank, o_parts, lse_parts, out=None, lse=None, stream=None):
        """Merge of one rank's per-step partials [npes, B, H, rows, d] / [npes, B, H, rows]
        ([B, H, rows, npes, d] / [B, H, rows, npes] on a plan with row_partials)."""
        if not 0 <= rank < self.npes:
            raise ValueError("rank must be in [0, npes)")
        rows = self.seqlen[rank]
        o_shape, l_shape = self.rank_parts_shapes(rank)
        _check_tensors((o_parts, "o_parts", self.part_dtype, o_shape), (lse_parts, "lse_parts", torch.float32, l_shape))
        if out is None:
            out = torch.empty((self.batch, self.heads, rows, self.dim), dtype=self.torch_dtype, device=o_parts.device)
        if lse is None:
            lse = torch.empty((self.batch, self.heads, rows), dtype=torch.float32, device=o_parts.device)
        _check_tensor(out, "out", self.torch_dtype, (self.batch, self.heads, rows, self.dim))
        _check_tensor(lse, "lse", torch.float32, (self.batch, self.heads, rows))
        check(self.lib.ringattn_rank_merge(self.handle, int(rank), _ptr(o_parts), _ptr(lse_parts), _ptr(out), _ptr(lse),
                                           _stream_ptr(stream)), "ringattn_rank_merge")
        return out, lse

    def launch_times(self):
        """Milliseconds of each block-attention launch of the last forward (plan made with timing=True): a forward
        is one launch, so one value."""
        n = ctypes.c_int()
        check(self.lib.ringattn_plan_launch_times(self.handle, None, 0, ctypes.byref(n)), "ringattn_plan_launch_times")
        ms = (ctypes.c_float * max(1, n.value))()
        check(self.lib.ringattn_plan_launch_times(self.handle, ms, n.value, ctypes.byref(n)), "ringattn_plan_launch_times")
        return [ms[i] for i in range(n.value)]

    def forward_kernel(self):
        """Name of the kernel forward() launches (as it appears in a kernel trace)."""
        name = self.lib.ringattn_plan_forward_kernel(self.handle)
        return name.decode() if name else None

    def work_items(self, step=-1):
        """The plan's block-attention jobs as (q_start, q_len, kv_start, kv_len, diag_off, slot)
        tuples: those of ring step `step`, or of the whole forward in launch order (step -1)."""
        n = ctypes.c_int()
        check(self.lib.ringattn_plan_work_items(self.handle, int(step), None, 0, ctypes.byref(n)), "ringattn_plan_work_items")
        items = (_lib.RingattnWorkItem * max(1, n.value))()
        check(self.lib.ringattn_plan_work_items(self.handle, int(step), items, n.value, ctypes.byref(n)),
              "ringattn_plan_work_items")
        return [(w.q_start, w.q_len, w.kv_start, w.kv_len, w.diag_off, w.slot) for w in items[:n.value]]

    def merge_regions(self):
        """(start, len, active-slot bitmask) of the row ranges the ring merge handles separately."""
        cap = 4 * self.npes
        st, ln, act = (ctypes.c_int * cap)(), (ctypes.c_int * cap)(), (ctypes.c_uint64 * cap)()
        n = ctypes.c_int()
        check(self.lib.ringattn_plan_merge_regions(self.handle, st, ln, act, cap, ctypes.byref(n)),
              "ringattn_plan_merge_regions")
        return [(st[i], ln[i], act[i]) for i in range(n.value)]

    def merge_ring(self, o_parts, lse_parts, out=None, lse=None, stream=None):
        """Ring-aware merge of caller-held per-step partials [npes, B, H, S, d] / [npes, B, H, S]
        ([B, H, S, npes, d] / [B, H, S, npes] on a plan with row_partials)."""
        o_shape, l_shape = self.parts_shapes()
        _check_tensors((o_parts, "o_parts", self.part_dtype, o_shape), (lse_parts, "lse_parts", torch.float32, l_shape))
        if out is None:
            out = torch.empty(self._shape(), dtype=self.torch_dtype, device=o_parts.device)
        if lse is None:
            lse = torch.empty(self._shape()[:3], dtype=torch.float32, device=o_parts.device)
        _check_tensor(out, "out", self.torch_dtype, self._shape())
        _check_tensor(lse, "lse", torch.float32, self._shape()[:3])
        check(self.lib.ringattn_merge_ring(self.handle, _ptr(o_parts), _ptr(lse_parts), _ptr(out), _ptr(lse),
                                           _stream_ptr(stream)), "ringattn_merge_ring")
        return out, lse


def zigzag_order(seqlen):
    """Row permutation of the zigzag layout: element i is the sequence position of memory row i.

    Rank r (seqlen[r] rows, back to back in memory) holds a low and a high half.  In the
    sequence the low halves of ranks 0..P-1 come first, then the high halves of ranks P-1..0.
    `x_memory = x_sequence[zigzag_order(seqlen)]`; invert with numpy.argsort.
    """
    half = [int(c) // 2 for c in seqlen]
    P = len(half)
    low_pos = np.concatenate(([0], np.cumsum(half)))              # start of rank r's low half
    high_pos = low_pos[P] + np.concatenate(([0], np.cumsum(half[::-1])))  # start of the i-th high half (rank P-1-i)
    rows = []
    for r in range(P):
        rows.append(np.arange(low_pos[r], low_pos[r] + half[r]))
        rows.append(np.arange(high_pos[P - 1 - r], high_pos[P - 1 - r] + half[r]))
    return np.concatenate(rows).astype(np.int64)


def merge(o_parts, lse_parts, dtype, stream=None):
    """n-way (O, LSE) merge.  o_parts [n, rows, d] fp32, lse_parts [n, rows] fp32."""
    lib = _lib.load()
    if o_parts.dim() != 3:
        raise ValueError("o_parts must be [n_parts, rows, dim]")
    n, rows, d = o_parts.shape
    _check_tensors((o_parts, "o_parts", torch.float32, None), (lse_parts, "lse_parts", torch.float32, (n, rows)))
    code = DTYPE_CODE[dtype]
    out = torch.empty((rows, d), dtype=TORCH_DTYPE[code], device=o_parts.device)
    lse = torch.empty((rows,), dtype=torch.float32, device=o_parts.device)
    check(lib.ringattn_merge(_ptr(o_parts), _ptr(lse_parts), n, rows, d, code, _ptr(out), _ptr(lse), _stream_ptr(stream)),
          "ringattn_merge")
    return out, lse


def _check_rank_call(q, k, v, out, lse, npes, mype, seqlen, dim):
    if len(seqlen) != npes or not 0 <= mype < npes:
        raise ValueError("seqlen must hold npes lengths and mype must be in [0, npes)")
    rows, total = int(seqlen[mype]), int(sum(seqlen))
    specs = [(q, "q", None, (rows, dim)), (k, "k", q.dtype, (total, dim)), (v, "v", q.dtype, (total, dim)),
             (out, "out", q.dtype, (rows, dim))]
    if lse is not None:
        specs.append((lse, "lse", torch.float32, (rows,)))
    _check_tensors(*specs)


def ring_attention(q, k, v, out, npes, mype, seqlen, dim, max_seq, lse=None, causal=False, softmax_scale=0.0):
    """Reference-shaped call (csrc/ring_attention.cu:706): one head, rank `mype` only.

    q [seqlen[mype], dim] is the rank's block, k / v [sum(seqlen), dim] hold all ranks'
    chunks, out [seqlen[mype], dim].  Blocks until done, like the reference (:721).
    """
    lib = _lib.load()
    _check_rank_call(q, k, v, out, lse, npes, mype, seqlen, dim)
    arr = (ctypes.c_int * len(seqlen))(*[int(x) for x in seqlen])
    check(lib.ringattn_ring_attention(_ptr(q), _ptr(k), _ptr(v), _ptr(out),
                                      _ptr(lse) if lse is not None else None, int(npes), int(mype), arr, int(dim),
                                      int(max_seq), DTYPE_CODE[q.dtype], int(bool(causal)), float(softmax_scale)),
          "ringattn_ring_attention")
    return out


def ring_attention_noalloc(q, k, v, out, npes, mype, seqlen, dim, max_seq, lse=None, causal=False, softmax_scale=0.0,
                           stream=None):
    """ring_attention() through the entry point that allocates nothing (its table of ring steps lives in a
    static device scratch); asynchronous on `stream`."""
    lib = _lib.load()
    _check_rank_call(q, k, v, out, lse, npes, mype, seqlen, dim)
    arr = (ctypes.c_int * len(seqlen))(*[int(x) for x in seqlen])
    check(lib.ringattn_ring_attention_noalloc(_ptr(q), _ptr(k), _ptr(v), _ptr(out),
                                              _ptr(lse) if lse is not None else None, int(npes), int(mype), arr,
                                              int(dim), int(max_seq), DTYPE_CODE[q.dtype], int(bool(causal)),
                                              float(softmax_scale), _stream_ptr(stream)),
          "ringattn_ring_attention_noalloc")
    return out


# ---- seeded inputs (counterpart of fillWithNum / initQKV, csrc/ring_attention.cu:731-748) ----

def fill_normal(n, dtype, seed, offset=0, sigma=1.0):
    """n values of N(0, sigma^2) rounded into `dtype`, as a uint16 numpy array of bit patterns."""
    lib = _lib.load()
    buf = np.empty(int(n), dtype=np.uint16)
    check(lib.ringattn_fill_normal(buf.ctypes.data_as(ctypes.c_void_p), DTYPE_CODE[dtype], int(n), int(seed), int(offset),
                                   float(sigma)), "ringattn_fill_normal")
    return buf


def make_qkv_bits(w):
    """Q, K, V of a Workload as uint16 bit patterns [B, H, S, d]; stream order Q, K, V."""
    n = w.batch * w.heads * w.seq * w.dim
    shape = (w.batch, w.heads, w.seq, w.dim)
    q = fill_normal(n, w.dtype, w.seed, 0, w.sigma_qk).reshape(shape)
    k = fill_normal(n, w.dtype, w.seed, n, w.sigma_qk).reshape(shape)
    v = fill_normal(n, w.dtype, w.seed, 2 * n, w.sigma_v).reshape(shape)
    return q, k, v


def bits_to_tensor(bits, dtype, device="cuda"):
    """uint16 bit patterns -> torch tensor of the 16-bit float dtype on `device`."""
    t = torch.from_numpy(bits.view(np.int16)).view(TORCH_DTYPE[DTYPE_CODE[dtype]])
    return t.to(device)
