"""What the compiler made of the attention kernel: every instantiation must fit two waves per
SIMD (256 registers), the carried-state ones without scratch memory, and the steady key loops of
the d = 128 ones -- the loops that hold 64 MFMAs, four 32-key blocks -- must carry one barrier per
two tiles and no scratch access.
Compiles the kernel to assembly for gfx950; needs hipcc but no GPU."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def loops_of(asm):
    """(label, instructions) of every innermost loop of a function body: from the block the
    compiler marks as the loop header to the last branch back to it (or to the block of wait
    and barrier it sometimes places right in front of the header)."""
    lines = asm.split("\n")
    where = {}
    for i, line in enumerate(lines):
        m = re.match(r"^(\.LBB\d+_\d+):", line)
        if m:
            where[m.group(1)] = i
    out = []
    for i, line in enumerate(lines):
        if "Inner Loop Header" not in line:
            continue
        head = max((k for k in where.values() if k <= i), default=None)
        if head is None:
            continue
        targets = {lab for lab, k in where.items() if head - 12 <= k <= head}
        last = None
        for j in range(i + 1, len(lines)):
            m = re.match(r"^\s*s_(?:cbranch_\w+|branch)\s+(\.LBB\d+_\d+)\s*$", lines[j])
            if m and m.group(1) in targets:
                last = j
        if last is not None:
            body = [l.strip() for l in lines[i + 1:last + 1]]
            out.append((lines[head].split(":")[0], [l for l in body if l and not l.startswith((";", "."))]))
    return out


def compile_to_asm(source, out):
    """Assembly of one kernel source plus the compiler's per-kernel resource remarks."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    from ringattention_amd import _build
    src = os.path.join(_build.CSRC, source)
    flags = [f for f in _build.HIPCC_FLAGS if f not in ("-shared", "-fPIC", "-pthread")]
    res = subprocess.run([hipcc] + flags + ["-S", "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage",
                                            "-I", os.path.join(ROOT, "include"), "-I", _build.CSRC, src, "-o", str(out)],
                         capture_output=True, text=True, timeout=900)
    assert res.returncode == 0, res.stderr[-2000:]
    usage = {}
    name = None
    for line in res.stderr.split("\n"):
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            usage[name] = {}
        for key in ("VGPRs", "ScratchSize [bytes/lane]", "Occupancy [waves/SIMD]", "LDS Size [bytes/block]"):
            m = re.search(re.escape(key) + r": (\d+)", line)
            if m and name:
                usage[name][key] = int(m.group(1))
    return out.read_text(), usage


def steady_loops(asm, kernel):
    start = asm.index("\n" + kernel + ":")
    end = asm.index(".amdhsa_kernel " + kernel, start)
    return [(lab, ins) for lab, ins in loops_of(asm[start:end]) if sum(i.startswith("v_mfma") for i in ins) == 64]


def test_walk_kernel_runs_two_waves_per_simd_without_spills(tmp_path):
    asm, usage = compile_to_asm("ringattn_walk.hip", tmp_path / "walk.s")
    walks = {n: u for n, u in usage.items() if "ring_walk_kernel" in n}
    # {fp16, bf16} x {64, 128} x {carried state; partials as fp32; partials as fp16}
    assert len(walks) == 12
    for n, u in walks.items():
        carried = n.endswith("Lb0ELb1EEEvNS_9BlockArgsE")
        # the carried-state variants must not spill at all; the others (which also hold the merge of a workgroup's
        # partials, three 64-register batches in flight) may around that merge, never in the steady loops
        assert u["ScratchSize [bytes/lane]"] == 0 or not carried, (n, u)
        assert u["VGPRs"] <= 256, (n, u)                       # eight waves per workgroup, one workgroup per compute unit
        if carried and "Li64E" in n:
            assert u["VGPRs"] <= 128, (n, u)                   # d = 64: two workgroups per compute unit (+12 % measured)
        # K and V rings; the variants that merge park the partial LSEs of their 256 rows there afterwards
        assert u["LDS Size [bytes/block]"] == (32768 if carried and "Li64E" in n else 65536), (n, u)
        if "Li128E" in n:
            steady = steady_loops(asm, n)
            assert len(steady) == 4, (n, len(steady))          # plain and masked groups, for each half of the workgroup
            for lab, ins in steady:
                # one barrier per two tiles (where partials are emitted the first one of a chunk may have been
                # taken before the stores, which puts it on a side path of the loop)
                assert sum(i.startswith("s_barrier") for i in ins) in ((2,) if carried else (1, 2)), (n, lab)
                assert not any(i.startswith("scratch_") for i in ins), (n, lab)


def test_walk64_kernel_runs_one_wave_per_simd(tmp_path):
    """ring_walk64_kernel (64 query rows per wave) is laid out for one wave per SIMD: more than 256 registers, the two
    eight-tile rings plus the chunk list in LDS, and next to no scratch (none inside the hand-scheduled loop, which
    is inline assembly)."""
    asm, usage = compile_to_asm("ringattn_walk64.hip", tmp_path / "walk64.s")
    kernels = {n: u for n, u in usage.items() if "ring_walk64_kernel" in n}
    # fp16, bf16 x (d = 128: state carried, fp32 partials, fp16 partials; d = 64: state carried)
    assert len(kernels) == 8
    for n, u in kernels.items():
        d64 = "ELi64E" in n
        assert u["Occupancy [waves/SIMD]"] == 1, (n, u)
        assert u["LDS Size [bytes/block]"] == 2 * 8 * (4096 if d64 else 8192) + 8 * (64 + 4), (n, u)
        # the plain-code path of waves with a single score tile, and the code between the passes of the instantiations
        # that emit a partial per chunk
        assert u["ScratchSize [bytes/lane]"] <= (128 if "ELb1ELb0EE" in n else 448), (n, u)
        start = asm.index("\n" + n + ":")
        body = asm[start:asm.index(".amdhsa_kernel " + n, start)]
        blocks = body.split(";;#ASMSTART")[1:]
        loop = max((b.split(";;#ASMEND")[0] for b in blocks), key=len)
        assert loop.count("v_mfma_f32_32x32x16") >= 8 * (16 if d64 else 32)    # eight unrolled iterations of 32 (16) MFMAs, and the tails
        assert "scratch_" not in loop


@pytest.mark.parametrize("source", ["ringattn_walk.hip", "ringattn_walk64.hip"])
def test_no_lds_transfer_reads_a_scalar_register_fresh_from_a_vector_instruction(source, tmp_path):
    """A vector instruction that writes a scalar register (v_readfirstlane, v_readlane, a compare into a register
    pair) must be five wait states ahead of a memory instruction that reads that register as its base address; the
    direct-to-LDS loads of these kernels sit in inline assembly, where the compiler inserts no such wait.  Every
    global_load_lds in the compiled code is checked against the instructions in front of it."""
    asm, _ = compile_to_asm(source, tmp_path / "hazard.s")
    lines = asm.split("\n")
    loads = 0
    for i, line in enumerate(lines):
        m = re.search(r"global_load_lds_dwordx4 \S+, s\[(\d+):(\d+)\]", line)
        if not m:
            continue
        loads += 1
        lo, hi = int(m.group(1)), int(m.group(2))
        wait_states, j = 0, i - 1
        while j > 0 and wait_states < 5:
            t = lines[j].strip()
            j -= 1
            if not t or t[0] in ";." or t.endswith(":"):
                continue
            w = re.match(r"(?:v_readfirstlane_b32|v_readlane_b32) s(\d+),", t) or re.match(r"v_cmp\S* s\[(\d+):", t)
            assert not (w and lo <= int(w.group(1)) <= hi), (i, t, line.strip(), wait_states)
            nop = re.match(r"s_nop (\d+)", t)
            wait_states += int(nop.group(1)) + 1 if nop else 1
    assert loads > 100
