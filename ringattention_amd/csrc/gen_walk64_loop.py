#!/usr/bin/env python3
"""Generates ringattn_walk64_loop.inc: the steady loop of ring_walk64_kernel (ringattn_walk64.hip) as ONE
inline-assembly statement with hand-allocated registers and a hand-made instruction order.

    python3 gen_walk64_loop.py            # rewrites ringattn_walk64_loop.inc (d = 128) and ringattn_walk64_loop_d64.inc next to this file
    python3 gen_walk64_loop.py --check    # exit status 1 if a committed file differs

Why by hand: one wave per SIMD has nobody to hide behind.  Within an iteration the matrix work (S(u+1) = K(u+1) Q^T
and O += P(u-1) V(u-1) for both 32-query blocks of the wave: 32 MFMAs) and the vector work (P(u) = exp2(S(u) k2 - m k2),
row sums, the row maximum of S(u+1): about 140 instructions) are independent, and the loop is only fast if they are
issued evenly interleaved (one MFMA, then four or five vector instructions) with every LDS fragment read several
MFMAs ahead of its use.  The compiler, given the same loop as C++, keeps Q in AccVGPRs and copies it back for every
MFMA, serialises the fragment reads behind waits and puts the exponentials after the MFMAs.

At d = 64 a tile has half the MFMAs (16) for the same vector work, seven to eight vector instructions go behind each, a
K or V tile is 4 KB (one 1 KB piece per wave), acc-O takes a[0:63] and Q a[64:95]; everything else is the same text.

Register map (d = 128; fixed; the C++ side hands its values over in exactly these registers):
    a[0:127]    acc-O: block b, head-dim block db at a[64 b + 16 db .. +15]
    a[128:191]  Q (B operands): block b, slice ks at a[128 + 32 b + 4 ks .. +3]
    v[0:63]     scores, two buffers of 2 x 16: buffer f, block b at v[32 f + 16 b .. +15]; exponentials are taken in place
    v[64:95]    probabilities (B operands), two buffers: buffer f, block b, half t2 at v[64 + 16 f + 8 b + 4 t2 .. +3]
    v[96:127]   the eight K fragments of a tile; v[128:159] the eight V^T fragments
    v[160:175]  LDS offsets of the K fragments (8), of the V^T fragments (4), global offsets of this wave's tile pieces (K 2, V 2)
    v[176:187]  m (2), m k2 (2), row sums (2 x 4);  v[192:199] temporaries
    v[200:231]  the exponentials of the tile before rounding, v[232:239] their sums (four per block)
    s[36:37] K load pointer, s38 tiles left in its chunk, s39 LDS address of the list entry of the chunk after it;
    s[40:43] the same for V;  s[44:45] / s[46:47] first row of the head in K / V, s48 k2, s49 / s50 LDS address of this
    wave's first piece in K / V ring slot 0, s51 the iteration u, s52 the first u whose score tile u+1 is not computed,
    s53 set to 2 when the workgroup's last iteration is done, s54 the first u whose score tile gets the causal mask, s55 the last iteration;
    v[190:191] mask limits of the two blocks
"""
import os
import sys

def _knob(name, default):
    return int(os.environ.get("W64_" + name, default))


NBUF = 8
UNROLL = 8      # iterations per trip: ring slots are immediates
LEAD = _knob('LEAD', 3)        # a fragment read is issued this many MFMAs ahead of the MFMA that needs it
HEAD_VALU = _knob('HEAD', 4)   # vector instructions in front of the first MFMA of an iteration
PREREAD = _knob('PREREAD', 4)     # K fragments of the next iteration read at the end of this one


def configure(d):
    """The head dimension the text is generated for."""
    global D, KS, DB, ROWB, TILE, PIECES, LOADS_IN_FLIGHT, SHARE, MASK_AT
    D = d
    KS, DB = d // 16, d // 32          # contraction slices of QK^T, 32-wide blocks of the head dim in PV
    ROWB = 2 * d                       # bytes per row
    TILE = 32 * ROWB                   # bytes per tile
    PIECES = TILE // 4096              # 1 KB pieces of a tile per wave
    LOADS_IN_FLIGHT = 3 * 2 * PIECES   # at the barrier: the loads of the last three iterations (two tiles each)
    # vector instructions behind an even / odd MFMA
    SHARE = (_knob('SHARE_A', 3), _knob('SHARE_B', 4)) if d == 128 else (_knob('SHARE_A', 7), _knob('SHARE_B', 8))
    MASK_AT = 2 * KS + 3    # the mask of tile u+1 is applied (if at all) behind this MFMA: the last QK MFMA is index 2 KS - 1


configure(128)


def O(b, db):
    return "a[%d:%d]" % (16 * (DB * b + db), 16 * (DB * b + db) + 15)


def Q(b, ks):
    base = 32 * DB + 4 * (KS * b + ks)
    return "a[%d:%d]" % (base, base + 3)


def Sreg(f, b, e):
    return "v%d" % (32 * f + 16 * b + e)


def Svec(f, b):
    return "v[%d:%d]" % (32 * f + 16 * b, 32 * f + 16 * b + 15)


def Pvec(f, b, t2):
    base = 64 + 16 * f + 8 * b + 4 * t2
    return "v[%d:%d]" % (base, base + 3)


def Preg(f, b, t2, k):
    return "v%d" % (64 + 16 * f + 8 * b + 4 * t2 + k)


def KF(ks):
    return "v[%d:%d]" % (96 + 4 * ks, 96 + 4 * ks + 3)


def VF(i):
    return "v[%d:%d]" % (128 + 4 * i, 128 + 4 * i + 3)


def VFlo(i):
    return "v[%d:%d]" % (128 + 4 * i, 128 + 4 * i + 1)


def VFhi(i):
    return "v[%d:%d]" % (128 + 4 * i + 2, 128 + 4 * i + 3)


KOFF = lambda ks: "v%d" % (160 + ks)
VOFF = lambda db: "v%d" % (168 + db)
GOFFK = lambda j: "v%d" % (172 + j)
GOFFV = lambda j: "v%d" % (174 + j)
M = lambda b: "v%d" % (176 + b)
MS = lambda b: "v%d" % (178 + b)
LS = lambda b, i: "v%d" % (180 + 4 * b + i)
CAND = lambda b: "v%d" % (188 + b)
TMP = lambda i: "v%d" % (192 + i)
PX = lambda b, e: "v%d" % (200 + 16 * b + e)      # exponentials of the tile, unrounded
TS = lambda b, i: "v%d" % (232 + 4 * b + i)       # their sums, four per block
# There is no row maximum in the loop: the exponentials are taken against the reference as it stands, and only when a
# sum of four of them exceeds 2^14 (or is not a number) is the row maximum looked at, the reference moved and the
# tile's exponentials redone (redo_routine)

S_KHEAD, S_VHEAD = (44, 45), (46, 47)
S_K2, S_LDSK, S_LDSV = "s48", "s49", "s50"
S_C, S_STOP, S_FAR, S_MW1, S_N = "s51", "s52", "s53", "s54", "s55"
S_T = lambda i: "s%d" % (56 + i)
VLIM = lambda b: "v%d" % (190 + b)


class Stream:
    """Scalar registers of a load stream: pointer to the next tile, tiles left in its chunk, LDS address of the
    list entry (byte offset from the head, tiles) of the chunk after it."""

    def __init__(self, base, head, lds, ring):
        self.lo, self.hi = "s%d" % base, "s%d" % (base + 1)
        self.ptr = "s[%d:%d]" % (base, base + 1)
        self.left = "s%d" % (base + 2)
        self.next = "s%d" % (base + 3)
        self.head = ("s%d" % head[0], "s%d" % head[1])
        self.lds = lds
        self.ring = ring


KST = Stream(36, S_KHEAD, S_LDSK, 0)
VST = Stream(40, S_VHEAD, S_LDSV, 1)
_sites = []   # (label number, stream) of every place a stream may enter its next chunk
_redo = []    # (label number, score buffer) of every place the speculative exponentials may give up


def tile_load(st, slot, goff):
    """The pieces of one tile this wave loads, then the step of the stream to the next tile (the change of chunk is out
    of line)."""
    site = len(_sites)
    _sites.append((site, st))
    ld = "s_nop 0 ;" if _knob('NOLOADS', 0) else ""   # timing only
    out = [
        "s_add_u32 m0, %s, %d" % (st.lds, slot * TILE),
        "s_sub_u32 %s, %s, 1" % (st.left, st.left),
        ld + "global_load_lds_dwordx4 %s, %s" % (goff(0), st.ptr),
    ]
    if PIECES == 2:
        out += [
            "s_add_u32 m0, %s, %d" % (st.lds, slot * TILE + 1024),
            "s_nop 0",
            ld + "global_load_lds_dwordx4 %s, %s" % (goff(1), st.ptr),
        ]
    out += [
        "s_add_u32 %s, %s, %d" % (st.lo, st.lo, TILE),
        "s_addc_u32 %s, %s, 0" % (st.hi, st.hi),
        "s_cmp_eq_u32 %s, 0" % st.left,
        "s_cbranch_scc1 3%02df" % site,
        "4%02d:" % site,
    ]
    return out


def chunk_changes():
    """Out of line: the stream enters its next chunk, whose entry (byte offset from the head, tiles) the kernel's
    prologue left in LDS."""
    out = []
    for site, st in _sites:
        out.append("3%02d:" % site)
        out += ["v_mov_b32 %s, %s" % (TMP(6), st.next),
                "ds_read_b64 v[%s:%s], %s" % (TMP(6)[1:], TMP(7)[1:], TMP(6)),
                "s_add_u32 %s, %s, 8" % (st.next, st.next),
                "s_waitcnt lgkmcnt(0)",
                "v_readfirstlane_b32 %s, %s" % (S_T(0), TMP(6)),
                "v_readfirstlane_b32 %s, %s" % (st.left, TMP(7)),
                "s_nop 3",
                "s_add_u32 %s, %s, %s" % (st.lo, st.head[0], S_T(0)),
                "s_addc_u32 %s, %s, 0" % (st.hi, st.head[1]),
                "s_branch 4%02db" % site]
    return out


def k_prereads(i_next):
    """The first K fragments of iteration i_next (tile u+1 of that iteration)."""
    slot = (i_next + 1) % NBUF
    return ["ds_read_b128 %s, %s offset:%d" % (KF(ks), KOFF(ks), slot * TILE) for ks in range(min(PREREAD, KS))]


def exp_stream(cur, cvt):
    """P = exp2(S k2 - m k2) of the score buffer `cur`, both blocks interleaved element by element: the unrounded
    values to PX, their sums (four per block) to TS, the rounded pairs to the probability buffer `cur`.  The three
    steps of an element (scale-and-subtract, exponential, sum / conversion) are DEPTH elements apart."""
    elems = [(b, e) for e in range(16) for b in range(2)]
    valu = []
    DEPTH = _knob('DEPTH', 8)

    def emit_step(kind, k):
        b, e = elems[k]
        if kind == 0:
            valu.append("v_fma_f32 %s, %s, %s, -%s" % (PX(b, e), Sreg(cur, b, e), S_K2, MS(b)))
        elif kind == 1:
            op = "v_mov_b32" if _knob('EXPMOV', 0) else "v_exp_f32"   # (timing only: what the transcendental itself costs)
            valu.append("%s %s, %s" % (op, PX(b, e), PX(b, e)))
        else:
            if e >= 4:
                first = PX(b, e - 4) if e < 8 else TS(b, e & 3)
                valu.append("v_add_f32 %s, %s, %s" % (TS(b, e & 3), first, PX(b, e)))
            if e & 1:   # the pair (e - 1, e) is complete
                valu.append("%s %s, %s, %s" % (cvt, Preg(cur, b, e // 8, (e % 8) // 2), PX(b, e - 1), PX(b, e)))
    for k in range(len(elems) + 2 * DEPTH):
        if k < len(elems):
            emit_step(0, k)
        if 0 <= k - DEPTH < len(elems):
            emit_step(1, k - DEPTH)
        if 0 <= k - 2 * DEPTH < len(elems):
            emit_step(2, k - 2 * DEPTH)
    return valu


def redo_routine(cur, cvt):
    """Out of line: the exponentials of the tile in score buffer `cur` came out too large for the standing reference
    (a sum of four above 2^14).  All MFMAs of the iteration are issued and acc-O holds the tiles before this one, so
    the reference moves to the row maximum at once -- l and acc-O rescaled as in csrc/ring_attention.cu:226-232 -- and
    the exponentials are taken again.  s57 says where to go back to."""
    out = ["85%d:" % cur, "s_nop 15"]
    for stp in range(4):
        for b in range(2):
            for c in range(2):
                t = TMP(2 * b + c)
                first = M(b) if stp == 0 else t
                out.append("v_max3_f32 %s, %s, %s, %s" % (t, first, Sreg(cur, b, 4 * stp + 2 * c), Sreg(cur, b, 4 * stp + 2 * c + 1)))
    for b in range(2):
        out.append("v_max_f32 %s, %s, %s" % (TMP(2 * b), TMP(2 * b), TMP(2 * b + 1)))
    for b in range(2):
        out.append("v_mov_b32 %s, %s" % (TMP(2 * b + 1), TMP(2 * b)))
    for b in range(2):
        out += ["s_nop 1", "v_permlane32_swap_b32 %s, %s" % (TMP(2 * b), TMP(2 * b + 1))]
    out.append("s_nop 1")
    for b in range(2):
        out.append("v_max_f32 %s, %s, %s" % (M(b), TMP(2 * b), TMP(2 * b + 1)))        # the new reference
    for b in range(2):
        out.append("v_mul_f32 %s, %s, %s" % (TMP(4 + b), S_K2, M(b)))                  # m k2
    for b in range(2):
        out.append("v_sub_f32 %s, %s, %s" % (TMP(6 + b), MS(b), TMP(4 + b)))           # old m k2 - new m k2
    for b in range(2):
        out.append("v_exp_f32 %s, %s" % (TMP(6 + b), TMP(6 + b)))                      # alpha
    for b in range(2):
        out.append("v_mov_b32 %s, %s" % (MS(b), TMP(4 + b)))
    out.append("s_nop 1")
    for b in range(2):
        for q in range(4):
            out.append("v_mul_f32 %s, %s, %s" % (LS(b, q), LS(b, q), TMP(6 + b)))
    # acc-O, eight registers at a time through the (dead) exponential buffer
    per_block = 16 * DB
    for b in range(2):
        for r0 in range(0, per_block, 8):
            for r in range(8):
                out.append("v_accvgpr_read_b32 %s, a%d" % (PX(0, r), per_block * b + r0 + r))
            for r in range(8):
                out.append("v_mul_f32 %s, %s, %s" % (PX(0, r), PX(0, r), TMP(6 + b)))
            for r in range(8):
                out.append("v_accvgpr_write_b32 a%d, %s" % (per_block * b + r0 + r, PX(0, r)))
    out += exp_stream(cur, cvt)
    for site, c in _redo:
        if c == cur:
            out += ["s_cmp_eq_u32 %s, %d" % (S_T(1), site), "s_cbranch_scc1 86%02db" % site]
    out.append("s_branch 199f")   # not reached
    return out


def iteration(i, mfma, cvt, do_qk=True, do_sm=True, do_pv=True):
    """Iteration u = 8 g + i of the steady loop: S(u+1) = K(u+1) Q^T, P(u) from S(u), O += P(u-1) V(u-1).
    Without do_qk / do_sm: the iterations after a wave's last score tile (no instruction order to speak of)."""
    cur, nxt = i & 1, (i & 1) ^ 1
    kslot, vslot = (i + 1) % NBUF, (i + NBUF - 1) % NBUF
    out = []
    # the barrier of the pair of iterations and this iteration's tile loads: in front of everything, or (MISC_AT > 0,
    # full iterations only) worked in behind the first MFMAs.  The K fragments the first MFMAs use were landed a
    # barrier ago; the V fragments of this iteration are only read behind this barrier.
    misc = []
    if i % 2 == 0:
        misc += ["s_waitcnt vmcnt(%d)" % LOADS_IN_FLIGHT] + ([] if _knob('NOBARRIER', 0) else ["s_barrier"])
        misc += tile_load(KST, (i + 7) % NBUF, GOFFK)
        misc += tile_load(KST, i % NBUF, GOFFK)
    else:
        misc += tile_load(VST, (i + 4) % NBUF, GOFFV)
        misc += tile_load(VST, (i + 5) % NBUF, GOFFV)
    MISC_AT = _knob('MISC_AT', 2) if (do_qk and do_pv) else 0
    if not MISC_AT:
        out += misc
        misc = []
    # ---- the three instruction streams of the iteration
    mf = []   # (text, index of the last fragment read it needs)
    reads = []  # fragment reads in the order they are issued
    if do_qk:
        for ks in range(KS):
            reads.append("ds_read_b128 %s, %s offset:%d" % (KF(ks), KOFF(ks), kslot * TILE))
            for b in range(2):
                src_c = "0" if ks == 0 else Svec(nxt, b)
                mf.append(("%s %s, %s, %s, %s" % (mfma, Svec(nxt, b), KF(ks), Q(b, ks), src_c), len(reads) - 1))
    n_qk = len(mf)
    for t2 in (range(2) if do_pv else ()):
        for db in range(DB):
            idx = DB * t2 + db
            off = vslot * TILE + 16 * t2 * ROWB
            reads.append("ds_read_b64_tr_b16 %s, %s offset:%d" % (VFlo(idx), VOFF(db), off))
            reads.append("ds_read_b64_tr_b16 %s, %s offset:%d" % (VFhi(idx), VOFF(db), off + 8 * ROWB))
            for b in range(2):
                mf.append(("%s %s, %s, %s, %s" % (mfma, O(b, db), VF(idx), Pvec(nxt, b, t2), O(b, db)), len(reads) - 1))
    need_at = [min(j for j, (_, r) in enumerate(mf) if r >= k) for k in range(len(reads))]

    valu = exp_stream(cur, cvt) if (do_sm and not _knob('NOEXP', 0)) else []
    spec_check = []
    if do_sm:
        for b in range(2):
            spec_check.append("v_max3_f32 %s, %s, %s, %s" % (TMP(b), TS(b, 0), TS(b, 1), TS(b, 2)))
        for b in range(2):
            spec_check.append("v_max_f32 %s, %s, %s" % (TMP(b), TMP(b), TS(b, 3)))
        spec_check.append("v_max_f32 %s, %s, %s" % (TMP(0), TMP(0), TMP(1)))
        spec_check.append("v_cmp_nge_f32_e32 vcc, 0x46800000, %s" % TMP(0))   # above 2^14, or not a number
        spec_check.append("SPECBRANCH")
        for b in range(2):
            for q in range(4):
                spec_check.append("v_add_f32 %s, %s, %s" % (LS(b, q), LS(b, q), TS(b, q)))
    n_exp_valu = len(valu)
    tail = []
    if do_qk:   # the mask limits move on by a tile
        for b in range(2):
            valu.append("v_subrev_u32_e32 %s, 32, %s" % (VLIM(b), VLIM(b)))

    # ---- interleave
    issued = min(PREREAD, KS) if do_qk else 0   # the first K fragments are on their way (read at the end of the previous iteration)
    if not do_qk:
        out.append("s_waitcnt lgkmcnt(0)")   # K fragments read ahead for a product that does not take place

    def issue_reads_upto(j_next):
        nonlocal issued
        res = []
        while issued < len(reads) and need_at[issued] <= j_next + LEAD:
            res.append(reads[issued])
            issued += 1
        return res

    if _knob('NOREADS', 0):
        import re as _re   # timing only: the products run on zero fragments
        reads = ["v_mov_b32 v%s, 0" % _re.search(r"v\[(\d+):", r).group(1) for r in reads]
    out += issue_reads_upto(0)
    vi = 0
    out += valu[vi:vi + HEAD_VALU]
    vi += HEAD_VALU
    masked = False
    waited = -1   # fragment reads up to this index are known to have returned
    BUDGET = _knob('BUDGET', 0)   # > 0: cycles of other work behind an MFMA (v_exp 8, anything else 4); 0: by count
    for j, (text, r) in enumerate(mf):
        spent = 0
        if r > waited or _knob('WAITALL', 0):
            out.append("s_waitcnt lgkmcnt(%d)" % min(issued - (r + 1), 15))
            waited = r
            spent += 4
        out.append(text)
        more = issue_reads_upto(j + 1)
        out += more
        spent += 4 * len(more)
        if do_qk and j == MASK_AT:
            # tile u+1 lies in this wave's masked range: the mask is applied out of line
            out += ["s_cmp_ge_i32 %s, %s" % (S_C, S_MW1), "s_cbranch_scc1 5%d0f" % i, "6%d0:" % i]
            masked = True
            spent += 8
        share = SHARE[j % 2]
        n_here = 0
        if MISC_AT and j + 1 >= MISC_AT:
            take = _knob('MISC_N', 3)
            while misc and take > 0:
                ln = misc.pop(0)
                out.append(ln)
                if not ln.endswith(":"):
                    take -= 1
                    n_here += 1
            # a label must not be separated from the branch in front of it by later insertions: flush a dangling one
            while misc and misc[0].endswith(":"):
                out.append(misc.pop(0))
        while vi < len(valu) and (vi < n_exp_valu or masked or not do_qk):
            # (the mask limits only move on once the mask has had its chance)
            cost = 8 if valu[vi].startswith("v_exp") else 4
            if (BUDGET and spent + cost > BUDGET) or (not BUDGET and n_here >= share):
                break
            out.append(valu[vi])
            vi += 1
            n_here += 1
            spent += cost
    assert not misc, "the tile loads did not fit behind the MFMAs"
    out += valu[vi:]
    if do_qk:
        out += k_prereads((i + 1) % UNROLL)
    for ln in spec_check:
        if ln == "SPECBRANCH":
            site = len(_redo)
            _redo.append((site, cur))
            out += ["s_cbranch_vccnz 8%02df" % site, "86%02d:" % site]
        else:
            out.append(ln)
    out += tail
    if _knob('SLEEP', 0):
        out.append("s_sleep %d" % _knob('SLEEP', 0))   # experiment: idle cycles (64 each)
    out.append("s_add_u32 %s, %s, 1" % (S_C, S_C))
    return out


def mask_code(i):
    """Out of line: the causal mask on S(u+1) of iteration i (buffer nxt): -inf where key > limit."""
    nxt = (i & 1) ^ 1
    out = ["5%d0:" % i, "v_mov_b32 %s, 0xff800000" % TMP(6)]
    for b in range(2):
        for e in range(16):
            key = 8 * (e >> 2) + (e & 3)
            out.append("v_cmp_gt_i32_e32 vcc, %d, %s" % (key, VLIM(b)))
            out.append("v_cndmask_b32_e32 %s, %s, %s, vcc" % (Sreg(nxt, b, e), Sreg(nxt, b, e), TMP(6)))
    out.append("s_branch 6%d0b" % i)
    return out


def loop_text(mfma, cvt):
    del _sites[:]
    del _redo[:]
    lines = k_prereads(0)
    lines.append("200:")
    for i in range(UNROLL):
        lines += iteration(i, mfma, cvt)
        lines += ["s_cmp_ge_i32 %s, %s" % (S_C, S_STOP),      # the next iteration has no score tile to compute
                  "s_cbranch_scc1 7%d0f" % ((i + 1) % UNROLL)]
    lines.append("s_branch 200b")
    # the last two iterations of the wave that compute: exponentials of the last score tile and the PV product before
    # it, then the last PV product; entered at ring position p.  After them the wave only keeps loading its share of
    # the tiles and meeting the barriers until the workgroup's last iteration (N).
    for p in range(UNROLL):
        lines.append("7%d0:" % p)
        lines += iteration(p, mfma, cvt, do_qk=False, do_sm=True)
        lines += iteration((p + 1) % UNROLL, mfma, cvt, do_qk=False, do_sm=False)
        lines.append("s_branch 9%d0f" % ((p + 2) % UNROLL))
    for p in range(UNROLL):
        lines.append("9%d0:" % p)
        lines += ["s_cmp_gt_i32 %s, %s" % (S_C, S_N), "s_cbranch_scc1 198f"]
        lines += iteration(p, mfma, cvt, do_qk=False, do_sm=False, do_pv=False)
        if p == UNROLL - 1:
            lines.append("s_branch 900b")
    for i in range(UNROLL):
        lines += mask_code(i)
    lines += chunk_changes()
    for site, cur in _redo:
        lines += ["8%02d:" % site, "s_mov_b32 %s, %d" % (S_T(1), site), "s_branch 85%df" % cur]
    for cur in range(2):
        lines += redo_routine(cur, cvt)
    lines.append("198:")
    lines.append("s_mov_b32 %s, 2" % S_FAR)
    lines.append("199:")
    lines.append("s_waitcnt lgkmcnt(0)")   # fragments read ahead are dropped: the C++ side reads them again
    return lines


def operands():
    outs, ins = [], []
    for b in range(2):
        for db in range(DB):
            outs.append('"+{%s}"(oacc[%d][%d])' % (O(b, db), b, db))
    for b in range(2):
        outs.append('"+{%s}"(sacc[%d])' % (Svec(0, b), b))
    for b in range(2):
        for t2 in range(2):
            outs.append('"+{%s}"(pprev[%d][%d])' % (Pvec(1, b, t2), b, t2))
    for b in range(2):
        for i in range(4):
            outs.append('"+{%s}"(ls[%d][%d])' % (LS(b, i), b, i))
    for b in range(2):
        outs.append('"+{%s}"(m[%d])' % (M(b), b))
    for b in range(2):
        outs.append('"+{%s}"(ms[%d])' % (MS(b), b))
    for st, n in ((KST, "k"), (VST, "v")):
        outs += ['"+{%s}"(%s_lo)' % (st.lo, n), '"+{%s}"(%s_hi)' % (st.hi, n), '"+{%s}"(%s_left)' % (st.left, n),
                 '"+{%s}"(%s_next)' % (st.next, n)]
    outs += ['"+{%s}"(asm_u)' % S_C, '"+{%s}"(asm_far)' % S_FAR]
    for b in range(2):
        outs.append('"+{%s}"(vlim[%d])' % (VLIM(b), b))
    for b in range(2):
        for ks in range(KS):
            ins.append('"{%s}"(qf[%d][%d])' % (Q(b, ks), b, ks))
    for ks in range(KS):
        ins.append('"{%s}"(koff_a[%d])' % (KOFF(ks), ks))
    for db in range(DB):
        ins.append('"{%s}"(voff_a[%d])' % (VOFF(db), db))
    for j in range(PIECES):
        ins.append('"{%s}"(goff_k[%d])' % (GOFFK(j), j))
    for j in range(PIECES):
        ins.append('"{%s}"(goff_v[%d])' % (GOFFV(j), j))
    ins += ['"{%s}"(kh_lo)' % KST.head[0], '"{%s}"(kh_hi)' % KST.head[1], '"{%s}"(vh_lo)' % VST.head[0], '"{%s}"(vh_hi)' % VST.head[1],
            '"{%s}"(k2_bits)' % S_K2, '"{%s}"(lds_dst_k)' % S_LDSK, '"{%s}"(lds_dst_v)' % S_LDSV,
            '"{%s}"(asm_stop)' % S_STOP, '"{%s}"(asm_mw1)' % S_MW1, '"{%s}"(asm_n)' % S_N]
    clob = ["v%d" % r for r in list(range(32, 80)) + list(range(96, 160)) + [188, 189] + list(range(192, 240))]
    clob += ["s56", "s57", "vcc", "scc", "m0", "memory"]
    return outs, ins, clob


def render(d=128):
    configure(d)
    res = ["// Generated by gen_walk64_loop.py -- do not edit.  The steady loop of ring_walk64_kernel: see the generator for the",
           "// register map and the instruction order.  Expects the kernel's variables by name.", ""]
    for dt, (mfma, cvt) in enumerate((("v_mfma_f32_32x32x16_f16", "v_cvt_pk_f16_f32"),
                                      ("v_mfma_f32_32x32x16_bf16", "v_cvt_pk_bf16_f32"))):
        res.append("%sif constexpr (DT == %d) {" % ("" if dt == 0 else "} else ", dt))
        res.append("asm volatile(")
        for ln in loop_text(mfma, cvt):
            res.append('    "%s\\n\\t"' % ln)
        outs, ins, clob = operands()
        res.append("    : " + ",\n      ".join(outs))
        res.append("    : " + ",\n      ".join(ins))
        res.append("    : " + ", ".join('"%s"' % c for c in clob) + ");")
    res.append("}")
    return "\n".join(res) + "\n"


FILES = {128: "ringattn_walk64_loop.inc", 64: "ringattn_walk64_loop_d64.inc"}

if __name__ == "__main__":
    here = os.environ.get("W64_OUT_DIR") or os.path.dirname(os.path.abspath(__file__))
    status = 0
    for d, name in FILES.items():
        path = os.path.join(here, name)
        if d == 128 and os.environ.get("W64_OUT"):
            path = os.environ["W64_OUT"]
        text = render(d)
        if "--check" in sys.argv:
            with open(path) as f:
                status |= 0 if f.read() == text else 1
            continue
        with open(path, "w") as f:
            f.write(text)
        print("wrote", path, len(text.split("\n")), "lines")
    sys.exit(status)
