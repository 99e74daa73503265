"""The C ABI without a GPU: every symbol declared in include/ringattn.h is exported, and
argument validation (which precedes every HIP call) returns the documented codes."""
import ctypes
import os
import re

import numpy as np
import pytest

from ringattention_amd import _lib
from ringattention_amd._lib import RingattnParams

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OK, E_NULL, E_NPES, E_DIM, E_DTYPE, E_SEQLEN, E_SHAPE, E_WS, E_RANK, E_PLAN, E_HIP, E_ALLOC, E_ALIGN = range(13)
STEP_PARTIALS = 8   # RINGATTN_FLAG_STEP_PARTIALS


def params(npes=2, seqlen=(128, 128), dim=64, batch=1, heads=1, dtype=0, causal=0, flags=0, scale=0.0, kv_heads=0, layout=0):
    arr = (ctypes.c_int * max(1, len(seqlen)))(*seqlen)
    p = RingattnParams(npes, ctypes.cast(arr, _lib.c_int_p), dim, scale, batch, heads, dtype, causal, flags, kv_heads, layout)
    p._keep = arr
    return p


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ringattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ringattn_[a-z_0-9]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(ralib):
    names = declared_functions()
    assert len(names) >= 11
    for n in names:
        assert hasattr(ralib, n), f"{n} declared in ringattn.h but not exported"
    assert set(names) == set(_lib.SYMBOLS), "ctypes binding and header disagree"


def test_header_constants_match_error_strings(ralib):
    text = open(os.path.join(ROOT, "include", "ringattn.h")).read()
    codes = {k: int(v) for k, v in re.findall(r"#define (RINGATTN_(?:OK|ERR_[A-Z]+)) (\d+)", text)}
    assert codes["RINGATTN_OK"] == 0 and codes["RINGATTN_ERR_ALIGN"] == E_ALIGN and len(codes) == 13
    msgs = [ralib.ringattn_strerror(c).decode() for c in range(13)]
    assert len(set(msgs)) == 13 and "unknown" in ralib.ringattn_strerror(99).decode()


def test_parameter_validation(ralib):
    wb = ralib.ringattn_workspace_bytes
    assert wb(ctypes.byref(params())) == 0          # the softmax state is carried in registers: no partials to park
    assert wb(ctypes.byref(params(flags=STEP_PARTIALS))) == 2 * 256 * 65 * 4
    assert wb(ctypes.byref(params(seqlen=(128, 384), flags=STEP_PARTIALS))) == 2 * 512 * 65 * 4   # unequal per-rank lengths are fine
    h = ctypes.c_void_p()

    def create(p):
        return ralib.ringattn_plan_create(ctypes.byref(p) if p is not None else None, None, 0, ctypes.byref(h))

    assert create(None) == E_NULL
    assert ralib.ringattn_plan_create(ctypes.byref(params()), None, 0, None) == E_NULL
    assert create(params(npes=0)) == E_NPES
    assert create(params(npes=-3)) == E_NPES
    assert create(params(npes=65, seqlen=(128,) * 65)) == E_NPES
    p = params()
    p.h_seqlen = None
    assert create(p) == E_NULL
    for bad_dim in (0, 32, 96, 256):
        assert create(params(dim=bad_dim)) == E_DIM
    assert create(params(dtype=2)) == E_DTYPE
    assert create(params(dtype=-1)) == E_DTYPE
    assert wb(ctypes.byref(params(seqlen=(128, 200), flags=STEP_PARTIALS))) == 2 * 328 * 65 * 4   # nor need they be multiples of the tile
    assert wb(ctypes.byref(params(seqlen=(1, 3), flags=STEP_PARTIALS))) == 2 * 4 * 65 * 4
    assert create(params(seqlen=(0, 128))) == E_SEQLEN
    assert create(params(seqlen=(0, 0))) == E_SEQLEN
    assert create(params(seqlen=(-128, -128))) == E_SEQLEN
    assert create(params(batch=0)) == E_SHAPE
    assert create(params(heads=-1)) == E_SHAPE
    assert create(params(scale=float("nan"))) == E_SHAPE
    assert create(params(heads=8, kv_heads=3)) == E_SHAPE     # kv_heads must divide heads
    assert create(params(heads=8, kv_heads=-2)) == E_SHAPE
    assert create(params(layout=2)) == E_SHAPE                # unknown layout
    assert create(params(layout=1, causal=1, seqlen=(128, 129))) == E_SEQLEN     # zigzag halves a rank: even lengths
    for bad in (params(npes=0), params(dim=7), params(seqlen=(64, -64))):
        assert wb(ctypes.byref(bad)) == 0
    assert wb(None) == 0


def test_workspace_counts_only_visible_steps(ralib):
    # a plan that keeps the ring steps apart: one partial row per query row and VISIBLE ring step
    # (causal ranks hold r + 1 steps, not npes)
    wb = ralib.ringattn_workspace_bytes
    row = (128 + 1) * 4
    assert wb(ctypes.byref(params(npes=8, seqlen=(4096,) * 8, dim=128, heads=32, causal=1))) == 0
    dense = wb(ctypes.byref(params(npes=8, seqlen=(4096,) * 8, dim=128, heads=32, causal=0, flags=STEP_PARTIALS)))
    causal = wb(ctypes.byref(params(npes=8, seqlen=(4096,) * 8, dim=128, heads=32, causal=1, flags=STEP_PARTIALS)))
    assert dense == 8 * 32 * 32768 * row
    assert causal == 36 * 32 * 4096 * row and causal * 64 == dense * 36       # 36 of the 64 (rank, step) pairs
    # zigzag: the low half of rank r sees r + 1 steps, the high half all 8: (36 + 64) / 2 of 64 chunk-steps
    zig = wb(ctypes.byref(params(npes=8, seqlen=(4096,) * 8, dim=128, heads=32, causal=1, layout=1, flags=STEP_PARTIALS)))
    assert zig == (36 + 64) * 32 * 2048 * row
    # fp16 partials (flag 4): 2 dim + 4 bytes per partial row
    half = wb(ctypes.byref(params(npes=8, seqlen=(4096,) * 8, dim=128, heads=32, causal=1, flags=4 | STEP_PARTIALS)))
    assert half == 36 * 32 * 4096 * (2 * 128 + 4)
    # ragged, unequal ranks
    lens = (100, 333, 1, 77)
    ragged = wb(ctypes.byref(params(npes=4, seqlen=lens, dim=64, causal=1, flags=STEP_PARTIALS)))
    assert ragged == sum((r + 1) * n for r, n in enumerate(lens)) * (64 + 1) * 4


def test_plan_lifetime_with_caller_workspace(ralib):
    # a caller-provided workspace needs no HIP call, so the plan life cycle runs on a CPU host
    p = params(flags=STEP_PARTIALS)
    need = ralib.ringattn_workspace_bytes(ctypes.byref(p))
    ws = np.zeros(need // 4 + 8, dtype=np.float32)
    base = ws.ctypes.data + (-ws.ctypes.data % 16)
    h = ctypes.c_void_p()
    assert ralib.ringattn_plan_create(ctypes.byref(p), ctypes.c_void_p(base), need - 1, ctypes.byref(h)) == E_WS
    assert ralib.ringattn_plan_create(ctypes.byref(p), ctypes.c_void_p(base + 4), need, ctypes.byref(h)) == E_ALIGN
    assert ralib.ringattn_plan_create(ctypes.byref(p), ctypes.c_void_p(base), need, ctypes.byref(h)) == OK
    assert h.value
    # argument checks of the compute entry points come before any HIP work
    x = ctypes.c_void_p(base)
    assert ralib.ringattn_fwd(h, None, x, x, x, x, None) == E_NULL
    assert ralib.ringattn_fwd(h, x, x, x, x, None, None) == E_NULL
    assert ralib.ringattn_fwd(h, ctypes.c_void_p(base + 2), x, x, x, x, None) == E_ALIGN
    assert ralib.ringattn_block_fwd(h, 2, x, x, x, x, x, None) == E_RANK
    assert ralib.ringattn_block_fwd(h, -1, x, x, x, x, x, None) == E_RANK
    assert ralib.ringattn_block_fwd(h, 0, x, x, None, x, x, None) == E_NULL
    # the rank-local entry points
    assert ralib.ringattn_rank_step_fwd(h, 2, 0, x, x, x, x, x, None) == E_RANK
    assert ralib.ringattn_rank_step_fwd(h, 0, -1, x, x, x, x, x, None) == E_RANK
    assert ralib.ringattn_rank_step_fwd(h, 0, 0, x, None, x, x, x, None) == E_NULL
    assert ralib.ringattn_rank_step_fwd(h, 0, 0, x, x, x, ctypes.c_void_p(base + 8), x, None) == E_ALIGN
    assert ralib.ringattn_rank_merge(h, 5, x, x, x, x, None) == E_RANK
    assert ralib.ringattn_rank_merge(h, 0, x, x, None, x, None) == E_NULL
    assert ralib.ringattn_plan_destroy(h) == OK
    assert ralib.ringattn_plan_destroy(h) == E_PLAN          # double destroy
    assert ralib.ringattn_rank_step_fwd(h, 0, 0, x, x, x, x, x, None) == E_PLAN
    assert ralib.ringattn_fwd(h, x, x, x, x, x, None) == E_PLAN  # use after destroy
    assert ralib.ringattn_plan_destroy(None) == E_PLAN


def test_merge_and_reference_entry_validation(ralib):
    buf = np.zeros(4096, dtype=np.float32)
    x = ctypes.c_void_p(buf.ctypes.data + (-buf.ctypes.data % 16))
    m = ralib.ringattn_merge
    assert m(None, x, 2, 8, 64, 0, x, x, None) == E_NULL
    assert m(x, x, 0, 8, 64, 0, x, x, None) == E_NPES
    assert m(x, x, 2, 8, 48, 0, x, x, None) == E_DIM
    assert m(x, x, 2, 8, 64, 5, x, x, None) == E_DTYPE
    assert m(x, x, 2, -1, 64, 0, x, x, None) == E_SHAPE
    ra = ralib.ringattn_ring_attention
    sl = (ctypes.c_int * 2)(128, 128)
    assert ra(x, x, x, x, None, 2, 2, sl, 64, 128, 0, 0, 0.0) == E_RANK
    assert ra(x, x, x, x, None, 2, -1, sl, 64, 128, 0, 0, 0.0) == E_RANK
    assert ra(x, x, x, x, None, 2, 0, sl, 64, 64, 0, 0, 0.0) == E_SEQLEN   # max_seq below a chunk
    assert ra(None, x, x, x, None, 2, 0, sl, 64, 128, 0, 0, 0.0) == E_NULL
    assert ra(x, x, x, x, None, 2, 0, sl, 80, 128, 0, 0, 0.0) == E_DIM
    assert ra(x, x, x, x, None, 0, 0, sl, 64, 128, 0, 0, 0.0) == E_NPES
    f = ralib.ringattn_fill_normal
    assert f(None, 0, 4, 0, 0, 1.0) == E_NULL
    assert f(x, 3, 4, 0, 0, 1.0) == E_DTYPE
    assert f(x, 0, -4, 0, 0, 1.0) == E_SHAPE


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libringattn.so"))
    with pytest.raises(RuntimeError, match="has not been built"):
        _lib.load()


def _plan_on_host(ralib, p):
    # a plan that carries the softmax state needs no workspace, so creating it makes no HIP call
    assert ralib.ringattn_workspace_bytes(ctypes.byref(p)) == 0
    h = ctypes.c_void_p()
    assert ralib.ringattn_plan_create(ctypes.byref(p), None, 0, ctypes.byref(h)) == OK
    return h


def _work_items(ralib, h, step):
    n = ctypes.c_int()
    assert ralib.ringattn_plan_work_items(h, step, None, 0, ctypes.byref(n)) == OK
    items = (_lib.RingattnWorkItem * max(1, n.value))()
    assert ralib.ringattn_plan_work_items(h, step, items, n.value, ctypes.byref(n)) == OK
    return [items[i] for i in range(n.value)]


@pytest.mark.parametrize("seqlen,causal,layout", [
    ((256, 256, 256, 256), 0, 0), ((256, 256, 256, 256), 1, 0), ((256, 256, 256, 256), 1, 1), ((256, 256, 256, 256), 0, 1),
    ((256, 768, 512), 1, 1), ((512, 256, 256, 768, 256), 1, 1), ((128, 384, 256), 1, 0), ((512,), 1, 1),
    ((256,) * 9, 1, 1), ((256,) * 16, 1, 0), ((256,) * 16, 1, 1),
    ((100, 333, 1, 77), 1, 0), ((100, 333, 1, 77), 0, 0), ((130, 70, 2, 258), 1, 1), ((7,), 1, 0),   # ragged lengths
])
def test_schedule_covers_every_visible_pair_exactly_once(ralib, seqlen, causal, layout):
    from ringattention_amd.api import zigzag_order
    P, S = len(seqlen), sum(seqlen)
    h = _plan_on_host(ralib, params(npes=P, seqlen=seqlen, causal=causal, layout=layout))
    start = np.concatenate([[0], np.cumsum(seqlen)])
    rank_of = np.repeat(np.arange(P), seqlen)
    pos = zigzag_order(seqlen) if layout == 1 else np.arange(S)    # sequence position of memory row i
    want = (pos[None, :] <= pos[:, None]) if causal else np.ones((S, S), bool)

    def coverage(items):
        cover = np.zeros((S, S), np.int32)
        slots = [set() for _ in range(S)]
        for w in items:
            assert w.q_len > 0 and w.kv_len > 0
            r = rank_of[w.q_start]
            j = (r + w.slot) % P                                    # ring discipline: step s visits rank (r + s) mod P
            assert start[r] <= w.q_start and w.q_start + w.q_len <= start[r + 1]
            assert start[j] <= w.kv_start and w.kv_start + w.kv_len <= start[j + 1]
            vis = np.ones((w.q_len, w.kv_len), bool)
            if w.diag_off >= 0:
                assert w.diag_off + w.q_len <= w.kv_len
                vis = np.arange(w.kv_len)[None, :] <= np.arange(w.q_len)[:, None] + w.diag_off
            cover[w.q_start:w.q_start + w.q_len, w.kv_start:w.kv_start + w.kv_len] += vis
            for row in range(w.q_start, w.q_start + w.q_len):
                assert w.slot not in slots[row]                     # one partial per row and slot
                slots[row].add(w.slot)
        return cover, slots

    cover, slots = coverage(_work_items(ralib, h, -1))
    assert np.array_equal(cover, want.astype(np.int32))
    per_step = [w for s in range(P) for w in _work_items(ralib, h, s)]
    assert all(w.slot == s for s in range(P) for w in _work_items(ralib, h, s))
    cover2, _ = coverage(per_step)
    assert np.array_equal(cover2, cover)
    # merge regions: a partition of the rows, each with exactly the slots that were written
    n = ctypes.c_int()
    cap = 4 * P
    st, ln, act = (ctypes.c_int * cap)(), (ctypes.c_int * cap)(), (ctypes.c_uint64 * cap)()
    assert ralib.ringattn_plan_merge_regions(h, st, ln, act, cap, ctypes.byref(n)) == OK
    seen = np.zeros(S, np.int32)
    for i in range(n.value):
        seen[st[i]:st[i] + ln[i]] += 1
        for row in range(st[i], st[i] + ln[i]):
            assert {s for s in range(64) if act[i] >> s & 1} == slots[row]
    assert np.all(seen == 1)
    if causal and layout == 1 and len(set(seqlen)) == 1:           # zigzag: every rank does the same work
        work = [want[start[r]:start[r + 1]].sum() for r in range(P)]
        assert max(work) - min(work) <= seqlen[0]                   # equal up to the diagonal's own width
    assert ralib.ringattn_plan_destroy(h) == OK


def test_zigzag_order_small_case():
    from ringattention_amd.api import zigzag_order
    # two ranks of 4 rows: rank 0 holds positions 0,1 and 6,7; rank 1 holds 2,3 and 4,5
    assert zigzag_order([4, 4]).tolist() == [0, 1, 6, 7, 2, 3, 4, 5]
    o = zigzag_order([256, 768, 512])
    assert sorted(o.tolist()) == list(range(1536))
    assert o[:128].tolist() == list(range(128)) and o[128] == 1536 - 128   # rank 0: first low half, last high half


def test_header_is_plain_c(tmp_path):
    # the boundary is a C ABI: the header must compile as C99 (no C++, no HIP, no torch types)
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_header.c"
    src.write_text('#include "ringattn.h"\nint main(void) { ringattn_params p; (void)p; return ringattn_strerror(0) == 0; }\n')
    res = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                          "-c", str(src), "-o", str(tmp_path / "use_header.o")], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_plans_from_many_threads(ralib):
    # the live-plan registry is shared: creating, inspecting and destroying plans from several
    # threads at once must neither crash nor confuse handles
    import threading
    errors = []

    def worker(seed):
        try:
            rng = np.random.default_rng(seed)
            for _ in range(200):
                P = int(rng.integers(1, 9))
                lens = tuple(int(2 * rng.integers(1, 300)) for _ in range(P))
                causal = int(rng.integers(0, 2))
                h = _plan_on_host(ralib, params(npes=P, seqlen=lens, causal=causal, layout=int(rng.integers(0, 2))))
                items = _work_items(ralib, h, -1)
                want = sum(1 for r in range(P) for s in range(P) if not causal or (r + s) % P <= r) if not causal else None
                if not causal:
                    assert len(items) == P * P == want
                assert ralib.ringattn_plan_destroy(h) == OK
                assert ralib.ringattn_plan_destroy(h) == E_PLAN
        except Exception as e:   # noqa: BLE001 - reported below
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_python_front_end_refuses_wrongly_shaped_tensors(ralib):
    # The C ABI takes raw pointers: every tensor is checked against the plan's geometry before the
    # call, so a mis-sized buffer is a ValueError and never an out-of-bounds access on the device.
    import torch
    from ringattention_amd import api
    P, c, d, B, H = 4, 128, 64, 2, 3
    plan = api.RingAttention(P, c, d, B, H, "fp16", False)   # needs no workspace; host only: never launched
    S = P * c
    good = torch.zeros(B, H, S, d, dtype=torch.float16)
    with pytest.raises(ValueError, match="k must have shape"):
        plan.forward(good, good[:, :, :-1], good)
    with pytest.raises(ValueError, match="q must have dtype"):
        plan.forward(good.float(), good, good)
    with pytest.raises(ValueError, match="q must be a device tensor"):          # right shape, wrong place
        plan.forward(good, good, good)
    with pytest.raises(ValueError, match="o_part must have shape"):
        plan.block_forward(0, good, good, good, o_part=torch.zeros(B, H, S - 1, d), lse_part=torch.zeros(B, H, S))
    with pytest.raises(ValueError, match="k_chunk must have shape"):
        plan.rank_step_forward(1, 2, good[:, :, :c], good[:, :, :c + 1], good[:, :, :c])
    with pytest.raises(ValueError, match="rank and step"):
        plan.rank_step_forward(P, 0, good[:, :, :c], good[:, :, :c], good[:, :, :c])
    with pytest.raises(ValueError, match="lse_parts must have shape"):
        plan.rank_merge(0, torch.zeros(P, B, H, c, d), torch.zeros(P, B, H, c + 1))
    with pytest.raises(ValueError, match="o_parts must have shape"):
        plan.merge_ring(torch.zeros(P - 1, B, H, S, d), torch.zeros(P, B, H, S))
    with pytest.raises(ValueError, match="lse_parts must have shape"):
        api.merge(torch.zeros(3, 64, d), torch.zeros(3, 65), "fp16")
    q1 = torch.zeros(c, d, dtype=torch.float16)
    kv = torch.zeros(S, d, dtype=torch.float16)
    for entry in (api.ring_attention, api.ring_attention_noalloc):
        with pytest.raises(ValueError, match="k must have shape"):
            entry(q1, kv[:-1], kv, torch.zeros_like(q1), P, 0, [c] * P, d, c)
        with pytest.raises(ValueError, match="out must have shape"):
            entry(q1, kv, kv, torch.zeros(c + 1, d, dtype=torch.float16), P, 0, [c] * P, d, c)
        with pytest.raises(ValueError, match="mype"):
            entry(q1, kv, kv, torch.zeros_like(q1), P, P, [c] * P, d, c)
    plan.close()
