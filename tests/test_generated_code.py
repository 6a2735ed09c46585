"""Checks on the machine code hipcc generates for the hand-scheduled GEMM kernels (no GPU needed):
what the compiler may not know about the inline assembly, it must be told.

The copies into LDS are inline assembly because the compiler would otherwise wait for all of them in
front of every LDS read.  The price is that the compiler trusts the statement's clobber list: an
`s_add_i32` inside it writes SCC, and when the list did not say so one build kept the carry of a
64-bit pointer addition alive across a copy (`s_add_u32`, copy, `s_addc_u32`), which reads an operand
panel that crosses a 4 GiB boundary 4 GiB too low.  These tests look for that pattern, and for
spills, in the code as built."""
import os
import re
import shutil
import subprocess

import pytest

from flash_muon_amd import build

SRC = os.path.join(build.CSRC, "fm_gemm_fast.hip")

# scalar ALU operations that write SCC (all but moves, multiplies and a few others do)
_SCC_WRITERS = re.compile(
    r"^(s_add_[iu]32|s_sub_[iu]32|s_addc_u32|s_subb_u32|s_cmp\w*|s_bitcmp\w*|s_and\w*|s_or\w*|s_xor\w*|s_nand\w*|"
    r"s_nor\w*|s_xnor\w*|s_not\w*|s_lshl\w*|s_lshr\w*|s_ashr\w*|s_min_[iu]32|s_max_[iu]32|s_abs\w*|s_bfe\w*|"
    r"s_absdiff\w*|s_wqm\w*|s_quadmask\w*|s_bcnt\w*)\b")
_SCC_READERS = re.compile(r"^(s_addc_u32|s_subb_u32|s_cselect_b(32|64)|s_cbranch_scc[01]|s_cmov\w*)\b")


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    if shutil.which(build.HIPCC) is None and not os.path.exists(build.HIPCC):
        pytest.skip("no hipcc here")
    out = tmp_path_factory.mktemp("asm") / "fm_gemm_fast.s"
    cmd = [build.HIPCC, *[f for f in build.FLAGS if f != "-fPIC"], "-S", "--cuda-device-only", SRC, "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return out.read_text().split("\n")


def _is_code(t):
    return bool(t) and not t.startswith(";") and not t.startswith(".") and not t.endswith(":")


def test_no_scc_value_lives_across_an_assembly_statement_that_writes_scc(assembly):
    kernel, in_asm, scc_set_at, clobbered_at, found = None, False, None, None, []
    for i, line in enumerate(assembly):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel, scc_set_at, clobbered_at = m.group(1), None, None
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if t.endswith(":") and not t.startswith(";"):      # a new basic block: what is live is not followed further
            scc_set_at, clobbered_at = None, None
            continue
        if not _is_code(t):
            continue
        if in_asm:
            if _SCC_WRITERS.match(t) and scc_set_at is not None:
                clobbered_at = i + 1
            continue
        if _SCC_READERS.match(t) and scc_set_at is not None and clobbered_at is not None:
            found.append("%s: SCC set in line %d, overwritten inside an asm statement in line %d, read in line %d (%s)"
                         % (kernel, scc_set_at, clobbered_at, i + 1, t))
        if _SCC_WRITERS.match(t):
            scc_set_at, clobbered_at = i + 1, None
    assert not found, "\n".join(found)


def test_every_assembly_statement_that_writes_scc_says_so():
    text = open(SRC).read()
    bad = []
    for m in re.finditer(r"asm volatile\((.*?)\);", text, re.S):
        body = m.group(1)
        instrs = re.findall(r"\b(s_[a-z0-9_]+)\b", body.split("::")[0] if "::" in body else body)
        if any(_SCC_WRITERS.match(x) for x in instrs) and '"scc"' not in body:
            bad.append(body.strip().split("\n")[0][:100])
    assert not bad, bad


def test_every_assembly_statement_that_writes_m0_says_so():
    """The copies set M0 themselves; declared, the register is the compiler's to avoid around them."""
    text = open(SRC).read()
    bad = []
    for m in re.finditer(r"asm volatile\((.*?)\);", text, re.S):
        body = m.group(1)
        code = body.split("::")[0] if "::" in body else body
        if re.search(r"\bs_[a-z0-9_]+\s+m0\b", code) and '"m0"' not in body:
            bad.append(body.strip().split("\n")[0][:100])
    assert not bad, bad


def test_gemm_kernels_do_not_spill(assembly):
    """One wave per SIMD owns all 512 registers of a lane; a spill means scratch traffic inside the
    MFMA loop or the write-out."""
    sizes = {}
    kernel = None
    for line in assembly:
        m = re.match(r"\s*\.amdhsa_kernel\s+(\S+)", line)
        if m:
            kernel = m.group(1)
        m = re.match(r"\s*\.amdhsa_private_segment_fixed_size\s+(\d+)", line)
        if m and kernel:
            sizes[kernel] = int(m.group(1))
    gemm = {k: v for k, v in sizes.items() if "gemm_nt" in k}
    assert len(gemm) >= 6, sorted(sizes)           # rounds x 4 instances, reduce x 2, mid x 2
    assert all(v == 0 for v in gemm.values()), {k: v for k, v in gemm.items() if v}


def test_every_copy_finds_the_m0_its_statement_or_the_one_before_it_set(assembly):
    """A copy into LDS takes its destination from M0.  Most statements set M0 and copy in one; the
    main loop of the whole tiles sets M0 in one statement and copies in a later one, with MFMAs and
    LDS reads between them.  In the code as built every copy must follow a write of M0 from an
    assembly statement with nothing between them that writes M0 or leaves the straight line (a label, a
    branch), and no M0 set for a copy may be followed by another such write before its copy."""
    m0_write = re.compile(r"^(s_\w+)\s+m0\b")
    kernel, in_asm, pending, bad, copies = None, False, None, [], 0
    for i, line in enumerate(assembly):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel, pending = m.group(1), None
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if t.endswith(":") and not t.startswith(";"):
            if pending is not None:
                bad.append("%s: a label in line %d between the M0 of line %d and its copy" % (kernel, i + 1, pending))
            pending = None
            continue
        if not _is_code(t):
            continue
        if m0_write.match(t):
            if not in_asm:
                bad.append("%s: line %d writes M0 outside an assembly statement (%s)" % (kernel, i + 1, t))
            elif pending is not None:
                bad.append("%s: M0 of line %d overwritten in line %d before its copy" % (kernel, pending, i + 1))
            pending = i + 1
            continue
        if t.startswith("global_load_lds"):
            copies += 1
            if pending is None:
                bad.append("%s: copy in line %d without an M0 set for it" % (kernel, i + 1))
            pending = None
            continue
        if pending is not None and re.match(r"^(s_cbranch|s_branch|s_setpc|s_swappc|s_endpgm)", t):
            bad.append("%s: line %d leaves the straight line between the M0 of line %d and its copy" % (kernel, i + 1, pending))
            pending = None
    assert copies > 100
    assert not bad, "\n".join(bad[:20])


def test_the_main_loops_move_no_sums_between_registers(assembly):
    """The 256 sums of a wave fill every accumulation register, so the register allocation has nowhere to
    move one through but the vector registers.  Built in three pieces (first stage, six stages, last
    stages), the loop of the kernels whose write-out reads an operand E came out with 800 and 1700 such
    moves per tile where the pieces meet, and one build of it with spills; as one loop it has none.
    Counted here: moves from, to and between accumulation registers among the 16x16x32 MFMAs of the main
    loop of every kernel, which come first in its code (the plain write-out keeps its three pieces and the
    23 sums that its first stage parks in vector registers: 92 reads and 92 writes)."""
    kernel, counts = None, {}
    for line in assembly:
        m = re.match(r"^(_Z\w*gemm_nt_rounds_kernel\w*):", line)
        if m:
            kernel = m.group(1)
            with_e = "ILb0ELi1E" in kernel or "ILb0ELi2E" in kernel
            per_stage = 128 if "ELi4EEE" in kernel else 64     # whole tiles, half tiles
            # one loop of 6 stages behind the MFMAs that clear the sums, or 1 + 6 + 5 stages
            counts[kernel] = {"mfma": 0, "moves": 0, "loop": 6 * per_stage + per_stage // 2 if with_e else 12 * per_stage}
            continue
        if re.match(r"^_Z\w+:", line):
            kernel = None
        if kernel is None:
            continue
        t = line.strip()
        c = counts[kernel]
        if t.startswith("v_mfma_f32_16x16x32"):
            c["mfma"] += 1
        elif t.startswith("v_accvgpr_") and 0 < c["mfma"] < c["loop"]:
            c["moves"] += 1
    assert len(counts) == 8, sorted(counts)          # (f16, plain) + bf16 x 3 write-outs, whole and half tiles
    for k, c in counts.items():
        with_e = "ILb0ELi1E" in k or "ILb0ELi2E" in k
        assert c["mfma"] >= c["loop"], (k, c)
        assert c["moves"] <= (0 if with_e else 200), (k, c)
