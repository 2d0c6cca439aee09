"""Static check of the hand-scheduled MFMA kernels against the compiled code.

The GEMM kernels of ``gemm_bfp8b_kernel.hpp`` issue their MFMAs and their direct-to-LDS loads as inline assembly, which the
compiler's hazard recognizer cannot look into.  Two rules of the CDNA ISA are therefore kept by the source itself, and this
test holds the compiled code to them (it compiles the units to assembly with the build's own flags, no GPU needed):

* a matrix instruction must not read a VGPR less than two wait states after a VALU instruction wrote it.  The first MFMA
  of every k step carries ``s_nop 1`` inside its statement (the one place where the compiler puts register copies of the
  operands in front of it); every other MFMA must be found two wait states or more away from any VALU write of its A and
  B operand registers, and must not sit directly behind a branch target.
* a direct load takes its LDS address from M0: every write of M0 in these kernels must be the ``s_mov_b32`` in front of
  such a load, inside the same statement.
"""
import concurrent.futures
import os
import re
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVICE = os.path.join(ROOT, "tt-buda_amd", "csrc", "device")
# the 8-wave kernel, the 4-wave kernel with the narrow tile, and the panel form with its three LDS stages
UNITS = ["gemm_bfp8b_big_bf16.hip", "gemm_bfp8b_slim_f32.hip", "gemm_bfp8b_panel_small_bf16.hip", "gemm_bfp8b_duo_slim_bf16.hip", "gemm_bfp8b_duo_small_f32.hip", "gemm_bfp8b_tall_bf16.hip", "gemm_bfp8b_duo_lean_bf16.hip"]


def build_flags():
    text = open(os.path.join(ROOT, "tt-buda_amd", "csrc", "Makefile")).read()
    m = re.search(r"^HIPFLAGS \?= (.*?)(?<!\\)\n", text, re.S | re.M)
    flags = m.group(1).replace("\\\n", " ").replace("$(ARCH)", "gfx950").split()
    return [f for f in flags if f != "-fPIC"]


def assembly(unit, outdir):
    out = os.path.join(outdir, unit.replace(".hip", ".s"))
    cmd = ["/opt/rocm/bin/hipcc"] + build_flags() + ["--cuda-device-only", "-S", os.path.join(DEVICE, unit), "-o", out]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-2000:]
    return open(out).read()


def regs(operand):
    """'v[6:9]' -> {6,7,8,9}; 'v12' -> {12}; anything else -> empty"""
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", operand)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"v(\d+)", operand)
    return {int(m.group(1))} if m else set()


def check(text):
    """(number of MFMAs seen, list of violations) for one assembly file"""
    lines = [l.strip() for l in text.split("\n")]
    lines = [l for l in lines if l and not l.startswith((";", "//")) and (not l.startswith(".") or l.endswith(":")) and not l.startswith("s_code_end")]
    n_mfma, n_direct, bad = 0, 0, []
    for i, l in enumerate(lines):
        parts = l.replace(",", " ").split()
        if parts[0].startswith("global_load_lds"):
            n_direct += 1
            if not (lines[i - 1].startswith("s_nop 0") and re.match(r"s_mov_b32 m0, ", lines[i - 2])):
                bad.append(("direct load without its own M0 write", l, lines[i - 2:i]))
        elif re.search(r"\bm0\b", l) and not parts[0].startswith("global_load_lds"):
            if not (re.match(r"s_mov_b32 m0, ", l) and i + 2 < len(lines) and lines[i + 2].split()[0].startswith("global_load_lds")):
                bad.append(("M0 touched outside a direct load", l, []))
        if not parts[0].startswith("v_mfma"):
            continue
        n_mfma += 1
        src = regs(parts[2]) | regs(parts[3])
        assert src, l
        gap, j = 0, i - 1
        while gap < 2 and j >= 0:
            p = lines[j]
            if p.endswith(":"):  # a branch target: whatever ends the other predecessor is not seen from here
                bad.append(("MFMA %d wait state(s) behind a label" % gap, l, [p]))
                break
            q = p.replace(",", " ").split()
            if q[0] == "s_nop":
                gap += int(q[1]) + 1
            else:
                is_valu = q[0].startswith("v_") and not q[0].startswith("v_mfma")
                if is_valu and len(q) > 1 and regs(q[1]) & src:
                    bad.append(("VALU write %d wait state(s) before the MFMA that reads it" % gap, l, [p]))
                gap += 1
            j -= 1
    return n_mfma, n_direct, bad


@pytest.fixture(scope="module")
def listings():
    with tempfile.TemporaryDirectory() as d, concurrent.futures.ThreadPoolExecutor(len(UNITS)) as pool:
        return dict(zip(UNITS, pool.map(lambda u: assembly(u, d), UNITS)))


@pytest.mark.parametrize("unit", UNITS)
def test_compiled_mfma_kernels_keep_the_hazard_rules(listings, unit):
    n_mfma, n_direct, bad = check(listings[unit])
    assert n_mfma >= 64 and n_direct >= 8, (n_mfma, n_direct)  # the loops are unrolled: dozens to hundreds of MFMAs per kernel
    assert not bad, bad[:5]


def test_the_checker_sees_a_violation():
    good = "s_nop 1\nv_mfma_f32_32x32x16_bf16 a[0:15], v[6:9], v[10:13], a[0:15]\n"
    assert check("v_mov_b32_e32 v7, v1\n" + good)[2] == []
    assert check("v_mov_b32_e32 v7, v1\nv_mfma_f32_32x32x16_bf16 a[0:15], v[6:9], v[10:13], a[0:15]\n")[2]
    assert check("v_mov_b32_e32 v7, v1\nds_read_b128 v[0:3], v20\nv_mfma_f32_32x32x16_bf16 a[0:15], v[6:9], v[10:13], a[0:15]\n")[2]
    assert check("v_mov_b32_e32 v7, v1\nv_add_u32_e32 v50, 1, v50\nds_read_b128 v[0:3], v20\nv_mfma_f32_32x32x16_bf16 a[0:15], v[6:9], v[10:13], a[0:15]\n")[2] == []
    assert check(".LBB0_1:\nv_mfma_f32_32x32x16_bf16 a[0:15], v[6:9], v[10:13], a[0:15]\n")[2]
    assert check("s_mov_b32 m0, s5\nv_mfma_f32_32x32x16_bf16 a[0:15], v[6:9], v[10:13], a[0:15]\n")[2]
