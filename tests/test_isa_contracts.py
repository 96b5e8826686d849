"""What the hand-written assembly in the kernels relies on, checked on the compiler's output.

The compiler inserts the wait states gfx90a-and-later hardware needs between dependent
instructions, but only around instructions it can see -- not around inline assembly:
  * a vector-memory instruction must not read an SGPR that a VALU instruction (v_readfirstlane,
    v_cmp with a scalar destination, ...) wrote within the five instructions before it;
  * a VALU instruction must not read an SGPR that a VALU instruction wrote within the two before it.
`dma_load` (kernels_gemm.hip: s_mov m0 / s_nop / global_load_lds) relies on its scalar operands
coming from scalar instructions; `set_lane2` (kernels_gate.hip) carries its own s_nop.  This test
compiles both files to gfx950 assembly (no GPU needed) and checks every assembly block along every
path that reaches it (fall-through, branches from other blocks, loop back-edges).

The GEMM's k loops also wait for their global->LDS loads with hand-counted `s_waitcnt vmcnt(n)`:
that count is right only while those loads are the only vector-memory instructions a wave issues
between the first and the last of them, which the second test checks for every instantiation."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "cuspamm_amd", "csrc")


def _isa(src, tmp_path):
    from cuspamm_amd import build
    out = os.path.join(str(tmp_path), src.replace(".hip", ".s"))
    cmd = [build.HIPCC] + [f for f in build.CFLAGS if f != "-Wall"] + build.GEMM_FLAGS + ["-S", "--cuda-device-only",
                                                                                      os.path.join(CSRC, src), "-o", out]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-2000:]
    return open(out).read()


def _sgprs(token):
    """SGPR numbers named by one operand: s5 -> {5}, s[10:11] -> {10, 11}, vcc -> {'vcc'}."""
    token = token.strip().rstrip(",")
    m = re.fullmatch(r"s(\d+)", token)
    if m:
        return {int(m.group(1))}
    m = re.fullmatch(r"s\[(\d+):(\d+)\]", token)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    if token in ("vcc", "vcc_lo", "vcc_hi"):
        return {"vcc"}
    return set()


def _instructions(text):
    """(mnemonic, operands, inside an inline-assembly block) per instruction line, in order; a label
    line gives ("label:", [name], False)."""
    out, in_asm = [], False
    for line in text.splitlines():
        s = line.strip()
        if s.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if s.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not s or s.startswith((";", "/")):
            continue
        s = s.split(";")[0].strip()
        if not s:
            continue
        m = re.fullmatch(r"([.\w$]+):", s)
        if m:
            out.append(("label:", [m.group(1)], False))
            continue
        if s.startswith("."):
            continue
        parts = s.split(None, 1)
        ops = [o.strip() for o in parts[1].split(",")] if len(parts) > 1 else []
        out.append((parts[0], ops, in_asm))
    return out


def _valu_written_sgprs(mnemonic, ops):
    """SGPRs a VALU instruction writes (scalar destination of a v_ instruction)."""
    if not mnemonic.startswith("v_") or not ops:
        return set()
    written = _sgprs(ops[0])
    if mnemonic.startswith(("v_cmp", "v_cmpx")) and mnemonic.endswith("_e32"):
        written |= {"vcc"}
    if re.match(r"v_(add|sub|subrev)_co_", mnemonic) and len(ops) > 1:
        written |= _sgprs(ops[1])
    return written


def _wait_states(mnemonic, ops):
    if mnemonic == "s_nop" and ops:
        return int(ops[0], 0) + 1
    return 1


def _hazards(ins, reader, need):
    """Every (reader index, offending instruction index) where an inline-assembly `reader` reads an SGPR
    that a VALU instruction wrote fewer than `need` wait states earlier, along ANY path: at a label
    the walk goes on into the fall-through predecessor and into every block that branches there
    (loop back-edges included)."""
    labels = {ops[0]: i for i, (mn, ops, _) in enumerate(ins) if mn == "label:"}
    branches = {}
    for i, (mn, ops, _) in enumerate(ins):
        if mn.startswith(("s_branch", "s_cbranch")) and ops and ops[0] in labels:
            branches.setdefault(ops[0], []).append(i)
    found, checked = [], 0

    def walk(j, states, read, origin, seen):
        while j >= 0 and states < need:
            pmn, pops, _ = ins[j]
            if pmn == "label:":
                for b in branches.get(pops[0], []):
                    if (b, states) not in seen:
                        seen.add((b, states))
                        walk(b, states, read, origin, seen)         # the branch itself is one wait state, counted there
                if j > 0 and ins[j - 1][0] == "s_branch":
                    return                                          # no fall-through into this label
                j -= 1
                continue
            if _valu_written_sgprs(pmn, pops) & read:
                found.append((origin, j))
            states += _wait_states(pmn, pops)
            j -= 1

    for i, (mn, ops, in_asm) in enumerate(ins):
        if not in_asm or mn != reader:
            continue
        checked += 1
        read = set()
        for o in ops:
            read |= _sgprs(o.split()[0]) if o else set()
        walk(i - 1, 0, read, i, set())
    return found, checked


@pytest.mark.parametrize("src,reader,need", [("kernels_gemm.hip", "global_load_lds_dwordx4", 5),
                                             ("kernels_gate.hip", "v_writelane_b32", 2)])
def test_assembly_blocks_keep_their_distance_from_valu_written_sgprs(tmp_path, src, reader, need):
    ins = _instructions(_isa(src, tmp_path))
    found, checked = _hazards(ins, reader, need)
    for origin, j in found:
        mn, ops, _ = ins[origin]
        pmn, pops, _ = ins[j]
        raise AssertionError("%s: %s %s reads an SGPR written too shortly before by %s %s" % (
            src, mn, ", ".join(ops), pmn, ", ".join(pops)))
    assert checked > 20, "no %s found inside assembly blocks of %s" % (reader, src)


FIXTURE_STRAIGHT = """
k:
    v_readfirstlane_b32 s4, v1
    s_mov_b32 s5, 0
    s_nop 0
    ;;#ASMSTART
    s_mov_b32 m0, s9
    s_nop 0
    global_load_lds_dwordx4 v2, s[4:5] offset:0
    ;;#ASMEND
    s_endpgm
"""
FIXTURE_BACK_EDGE = """
k:
    s_mov_b32 s4, 0
    s_mov_b32 s5, 0
    s_nop 4
.LBB0_1:
    ;;#ASMSTART
    s_mov_b32 m0, s9
    s_nop 0
    global_load_lds_dwordx4 v2, s[4:5] offset:0
    ;;#ASMEND
    s_add_u32 s8, s8, 1
    v_readfirstlane_b32 s4, v1
    s_cmp_lt_u32 s8, s10
    s_cbranch_scc1 .LBB0_1
    s_endpgm
"""
FIXTURE_OTHER_PREDECESSOR = """
k:
    s_cbranch_scc1 .LBB0_2
    v_readfirstlane_b32 s4, v1
    s_branch .LBB0_3
.LBB0_2:
    s_mov_b32 s4, 0
    s_nop 4
.LBB0_3:
    ;;#ASMSTART
    s_mov_b32 m0, s9
    s_nop 0
    global_load_lds_dwordx4 v2, s[4:5] offset:0
    ;;#ASMEND
    s_endpgm
"""
FIXTURE_CLEAN_LOOP = """
k:
    v_readfirstlane_b32 s4, v1
    s_nop 4
.LBB0_1:
    ;;#ASMSTART
    s_mov_b32 m0, s9
    s_nop 0
    global_load_lds_dwordx4 v2, s[4:5] offset:0
    ;;#ASMEND
    s_add_u32 s4, s4, 64
    s_addc_u32 s5, s5, 0
    s_cmp_lt_u32 s4, s10
    s_cbranch_scc1 .LBB0_1
    s_endpgm
"""


def test_hazard_checker_sees_hazards_across_branches():
    # the checker itself: a hazard in straight-line code, over a loop back-edge and from a second
    # predecessor block must each be reported; a loop whose address is advanced by scalar
    # instructions only must pass
    for text, want in ((FIXTURE_STRAIGHT, 1), (FIXTURE_BACK_EDGE, 1), (FIXTURE_OTHER_PREDECESSOR, 1), (FIXTURE_CLEAN_LOOP, 0)):
        found, checked = _hazards(_instructions(text), "global_load_lds_dwordx4", 5)
        assert checked == 1 and len(found) == want, (text, found)


def test_gemm_k_loops_issue_no_other_vector_memory_instruction(tmp_path):
    text = _isa("kernels_gemm.hip", tmp_path)
    kernels = re.findall(r"^(_ZN5spamm(?:6k_gemm|10k_gemm_w64)ILi\d+ELi\d+(?:ELi\d+|ELb[01])?EEE\w+):[^\n]*\n(.*?)s_endpgm", text, flags=re.S | re.M)
    # whole macro tiles by four waves: tiles 32 / 64 / 128 x ring depths 3 / 4 / 5, and the three tiles by
    # workgroups that stay (ELb1E); waves of 64 x 128 (half macro tiles, whole macro tiles by eight waves):
    # the three tiles each
    assert len([n for n, _ in kernels if "k_gemm_w64" not in n and "ELb0E" in n]) == 9
    assert len([n for n, _ in kernels if "k_gemm_w64" not in n and "ELb1E" in n]) == 3
    assert len([n for n, _ in kernels if "k_gemm_w64" in n]) == 6
    for name, body in kernels:
        mns = [mn for mn, _, _ in _instructions(body)]
        dma = [i for i, mn in enumerate(mns) if mn == "global_load_lds_dwordx4"]
        assert len(dma) >= 12, name
        other = [mn for mn in mns[dma[0]:dma[-1] + 1]
                 if mn.startswith(("global_", "flat_", "buffer_", "scratch_")) and mn != "global_load_lds_dwordx4"]
        assert not other, "%s: %s between the first and the last global->LDS load" % (name, sorted(set(other)))
        # and C is stored only after the loops have drained the ring
        stores = [i for i, mn in enumerate(mns) if mn.startswith("global_store")]
        assert stores and min(i for i in stores if i > dma[0]) > dma[-1], name
        # workgroups that stay draw their tickets with a returning atomic: it must be issued before an
        # item's first global->LDS load (then it is older than every load the counts speak of); the
        # stores of the previous item's C are older than the next item's loads in the same way
        # (a third one sits in the loop over the items with nothing kept, after the last load)
        atomics = [i for i, mn in enumerate(mns) if mn.startswith("global_atomic")]
        if "ELb1E" in name:
            assert len([i for i in atomics if i < dma[0]]) == 2 and len([i for i in atomics if i > dma[-1]]) == 1, name
            assert not any(mn.startswith("scratch_") for mn in mns), name
        else:
            assert not atomics, name
