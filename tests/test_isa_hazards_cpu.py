"""The kernels that fill LDS tiles with direct-to-LDS loads issue their LDS reads as inline assembly with their own
`s_waitcnt lgkmcnt` (otherwise the compiler drains the load pipeline in front of every read).  The price: the compiler does not
know that the destination registers of such a read are written LATER, when the read lands.  A read whose result is never
named by a wait (a prefetch past the last tile, a dead fragment) leaves the compiler free to reuse its registers while the read
is still in flight -- for an address, say -- and the late write then corrupts them.  This test compiles those sources to gfx950
assembly (no GPU needed) and walks every kernel: between a hand-issued read and the `s_waitcnt lgkmcnt(n)` that covers it, no
other instruction may read or write its destination registers.
"""
import importlib.util
import os
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "24ppopp-liger_amd")
SOURCES = ["gemm_fast.hip", "gemm_skinny_kn.hip", "attention_prefill.hip", "ceilings.hip"]   # every file that issues LDS reads by hand


def _build_recipe():
    spec = importlib.util.spec_from_file_location("liger_build_for_isa", os.path.join(PKG, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def hazards(asm_text):
    """-> (kernels checked, hand-issued reads seen, list of (kernel, instruction) that touch a register of a read in flight)"""
    found, kernels, reads = [], 0, 0
    for m in re.finditer(r"^(\w+):[^\n]*\n.*?s_endpgm", asm_text, re.S | re.M):
        name, body = m.group(1), m.group(0).splitlines()
        kernels += 1
        pending, seq, in_asm = {}, 0, False      # register -> sequence number of the read that will write it
        for line in body:
            line = line.strip()
            if line.startswith(";;#ASMSTART"):
                in_asm = True
                continue
            if line.startswith(";;#ASMEND"):
                in_asm = False
                continue
            if not line or line.startswith(";") or line.endswith(":") or line.startswith("."):
                continue
            line = line.split(";")[0]
            rd = re.match(r"ds_read\w* v\[(\d+):(\d+)\]", line)
            if rd:
                seq += 1     # every LDS read counts in lgkmcnt, the compiler's own as well
                if in_asm:
                    reads += 1
                    for r in range(int(rd.group(1)), int(rd.group(2)) + 1):
                        if r in pending:
                            found.append((name, "read into v%d while an earlier read of it is in flight" % r))
                        pending[r] = seq
                continue
            if re.match(r"ds_|s_load|s_buffer_load", line):
                seq += 1     # other users of the counter (they complete in order with the reads around them for this purpose)
            if line.startswith("s_waitcnt") and "lgkmcnt" in line:
                n = int(re.search(r"lgkmcnt\((\d+)\)", line).group(1))
                pending = {r: q for r, q in pending.items() if q > seq - n}
                continue
            regs = set()
            for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", line):
                regs.update(range(int(a), int(b) + 1))
            regs.update(int(r) for r in re.findall(r"\bv(\d+)\b", line))
            if regs & set(pending):
                found.append((name, line[:90]))
    return kernels, reads, found


def test_the_checker_sees_a_register_reused_under_a_read_in_flight():
    bad = """k1:
	;;#ASMSTART
	ds_read_b128 v[54:57], v183 offset:2048
	;;#ASMEND
	v_lshlrev_b32_e32 v54, 1, v2
	v_lshl_add_u64 v[178:179], s[8:9], 0, v[54:55]
	s_endpgm
"""
    good = bad.replace("\tv_lshlrev_b32_e32 v54", "\t;;#ASMSTART\n\ts_waitcnt lgkmcnt(0)\n\t;;#ASMEND\n\tv_lshlrev_b32_e32 v54")
    assert len(hazards(bad)[2]) == 2 and hazards(bad)[1] == 1
    assert hazards(good)[2] == []
    # a wait that leaves the newest read outstanding does not cover it
    partial = good.replace("lgkmcnt(0)", "lgkmcnt(1)")
    assert len(hazards(partial)[2]) == 2


def test_no_register_of_a_hand_issued_lds_read_is_touched_before_its_wait(tmp_path):
    recipe = _build_recipe()
    if not os.path.exists(recipe.HIPCC):
        pytest.skip("no hipcc in this image")

    def to_asm(src):
        out = str(tmp_path / (src + ".s"))
        subprocess.run([recipe.HIPCC] + recipe.HIP_FLAGS + ["-S", "--cuda-device-only", os.path.join(recipe.CSRC, src), "-o", out],
                       check=True, stdout=subprocess.PIPE, stderr=subprocess.PIPE)
        return src, open(out).read()

    with ThreadPoolExecutor(max_workers=4) as ex:
        results = list(ex.map(to_asm, SOURCES))
    total_reads = 0
    for src, text in results:
        kernels, reads, found = hazards(text)
        assert kernels > 0, src
        total_reads += reads
        assert not found, "%s: %d hazards, first: %s" % (src, len(found), found[:3])
    assert total_reads > 100     # the hand-issued reads were actually seen (the pattern still matches what the compiler prints)
