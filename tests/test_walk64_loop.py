"""The hand-scheduled loop of ring_walk64_kernel (ringattention_amd/csrc/gen_walk64_loop.py -> ringattn_walk64_loop.inc
for d = 128, ringattn_walk64_loop_d64.inc for d = 64):
the committed file is what the generator writes, and the instruction stream it writes keeps the promises the hardware
does not check -- every MFMA finds its LDS fragments returned (the s_waitcnt lgkmcnt counts are derived from the order
of the reads), nothing reads a score tile too soon after the MFMA that wrote it, and an iteration holds the work it
should.  Runs on the CPU; needs no GPU and no hipcc (the compiled kernel's resources are checked in
test_kernel_resources.py)."""
import importlib.util
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ringattention_amd", "csrc")


@pytest.fixture(scope="module")
def gen():
    spec = importlib.util.spec_from_file_location("gen_walk64_loop", os.path.join(CSRC, "gen_walk64_loop.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("d", [128, 64])
def test_committed_loop_is_what_the_generator_writes(gen, d):
    with open(os.path.join(CSRC, gen.FILES[d])) as f:
        assert f.read() == gen.render(d)


def regs(token):
    """Register numbers of one operand: v12, v[4:7], a[0:15] -> ('v', [..]) ; anything else -> (None, [])."""
    m = re.fullmatch(r"-?([va])(\d+)", token)
    if m:
        return m.group(1), [int(m.group(2))]
    m = re.fullmatch(r"-?([va])\[(\d+):(\d+)\]", token)
    if m:
        return m.group(1), list(range(int(m.group(2)), int(m.group(3)) + 1))
    return None, []


def operands(line):
    op, _, rest = line.partition(" ")
    rest = rest.split(" offset:")[0]
    return op, [t.strip() for t in rest.split(",")] if rest else []


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("dtype_ops", [("v_mfma_f32_32x32x16_f16", "v_cvt_pk_f16_f32"), ("v_mfma_f32_32x32x16_bf16", "v_cvt_pk_bf16_f32")])
def test_steady_iterations_hold_their_work_and_wait_for_their_fragments(gen, dtype_ops, d):
    mfma, cvt = dtype_ops
    gen.configure(d)
    preread = min(gen.PREREAD, gen.KS)
    del gen._sites[:]
    del gen._redo[:]
    for i in range(gen.UNROLL):
        lines = gen.iteration(i, mfma, cvt)
        ops = [operands(l)[0] for l in lines if not l.endswith(":")]
        assert sum(o == mfma for o in ops) == d // 4                      # half for S(u+1) = K Q^T, half for O += P V
        assert sum(o.startswith("ds_read") for o in ops) == 3 * d // 16   # d / 16 K fragments, d / 8 halves of V^T fragments
        assert sum(o == "global_load_lds_dwordx4" for o in ops) == d // 32   # this wave's pieces of two tiles
        assert sum(o == "v_exp_f32" for o in ops) == 32                   # one exponential per score
        assert sum(o == "s_barrier" for o in ops) == (1 if i % 2 == 0 else 0)
        assert not any(o.startswith(("scratch_", "buffer_", "flat_")) for o in ops)
        # LDS reads return in order: replay the queue, and require every fragment register an MFMA reads to be back
        outstanding = []                  # reads not yet waited for, oldest first: the registers each one writes
        for ks in range(preread):         # (the first K fragments were read ahead by the iteration before)
            outstanding.append({("v", r) for r in regs(gen.KF(ks))[1]})
        last_writer = {}                  # score register -> index of the MFMA that wrote it
        n = 0
        for line in lines:
            if line.endswith(":"):
                continue
            op, args = operands(line)
            n += 1
            if op.startswith("ds_read"):
                outstanding.append({(regs(args[0])[0], r) for r in regs(args[0])[1]})
            elif op == "s_waitcnt" and "lgkmcnt" in line:
                keep = int(re.search(r"lgkmcnt\((\d+)\)", line).group(1))
                outstanding = outstanding[len(outstanding) - keep:] if keep < len(outstanding) else outstanding
            elif op == mfma:
                in_flight = set().union(*outstanding) if outstanding else set()
                for tok in args[1:3]:
                    f, rr = regs(tok)
                    assert not ({(f, r) for r in rr} & in_flight), (i, line)
                f, rr = regs(args[0])
                if f == "v":
                    for r in rr:
                        last_writer[r] = n
            elif op.startswith("v_") and op != mfma:
                # an MFMA of eight passes needs 11 wait states before a vector instruction touches its result
                for tok in args:
                    f, rr = regs(tok)
                    for r in rr:
                        if f == "v" and r in last_writer:
                            assert n - last_writer[r] > 11, (i, line)
        # what is still out at the end are the K fragments read ahead for the next iteration
        assert len(outstanding) == preread
    gen.configure(128)


@pytest.mark.parametrize("d", [128, 64])
def test_loop_text_has_every_exit_and_no_stray_label(gen, d):
    gen.configure(d)
    lines = gen.loop_text("v_mfma_f32_32x32x16_bf16", "v_cvt_pk_bf16_f32")
    labels = [l[:-1] for l in lines if l.endswith(":")]
    assert len(labels) == len(set(labels))
    for l in lines:
        m = re.match(r"s_c?branch\w*\s+(\d+)([fb])$", l)
        if m:
            assert m.group(1) in labels, l
    # forward / backward references point the right way
    pos = {lab: k for k, lab in enumerate(l[:-1] if l.endswith(":") else None for l in lines) if lab}
    for k, l in enumerate(lines):
        m = re.match(r"s_c?branch\w*\s+(\d+)([fb])$", l)
        if m:
            assert (pos[m.group(1)] > k) == (m.group(2) == "f"), l
    gen.configure(128)
