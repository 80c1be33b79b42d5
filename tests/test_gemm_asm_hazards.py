"""The GEMM ring kernel issues its MFMAs from inline assembly, so the compiler does not know
they are MFMAs and inserts none of the wait states the matrix pipe needs around them.  This
test compiles the kernel to assembly (hipcc cross-compiles without a GPU) and checks the two
hazards that such code can run into:

  * a vector-ALU instruction (a copy, a spill restore, v_accvgpr_*) that writes a register
    shortly before an MFMA reads it as an operand;
  * an instruction other than an MFMA that reads an MFMA's result shortly after it was issued,
    with no s_nop in between.

Fragment registers filled by ds_read are covered by the s_waitcnt the compiler places (it
does track registers through inline assembly operands), so they are not checked here."""

import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("TILEFUSION_HIPCC", "/opt/rocm/bin/hipcc")
MIN_GAP = 2        # instructions between a VALU write and the MFMA that reads it
RESULT_GAP = 6     # instructions (or an s_nop) between an MFMA and a non-MFMA reader of its result


def _regs(tok):
    """'v[4:7]' -> {v4..v7}, 'a12' -> {a12}; anything else -> empty."""
    m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", tok)
    if m:
        return {f"{m.group(1)}{i}" for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.fullmatch(r"([va])(\d+)", tok)
    return {f"{m.group(1)}{m.group(2)}"} if m else set()


def _parse(line):
    line = line.split(";")[0].strip()
    if not line or line.endswith(":") or line.startswith("."):
        return None
    parts = line.split(None, 1)
    ops = [o.strip() for o in parts[1].split(",")] if len(parts) > 1 else []
    return parts[0], ops


def _check(name, body):
    instrs = [p for p in (_parse(l) for l in body.splitlines()) if p]
    n_mfma = 0
    for i, (op, ops) in enumerate(instrs):
        if not op.startswith("v_mfma"):
            continue
        n_mfma += 1
        srcs = set().union(*[_regs(o) for o in ops[1:]])
        # (1) VALU writes just in front of the MFMA
        for back in range(1, MIN_GAP + 1):
            if i - back < 0:
                break
            pop, pops = instrs[i - back]
            if pop.startswith("v_") and not pop.startswith("v_mfma") and pops:
                clash = _regs(pops[0]) & srcs
                assert not clash, f"{name}: {pop} writes {sorted(clash)} {back} instruction(s) before an MFMA that reads it"
        # (2) non-MFMA readers of the result just behind it
        dst = _regs(ops[0])
        for fwd in range(1, RESULT_GAP + 1):
            if i + fwd >= len(instrs):
                break
            nop, nops = instrs[i + fwd]
            if nop == "s_nop" and int(nops[0]) >= 7:
                break
            if nop.startswith("v_mfma") or nop.startswith("s_") or nop.startswith("ds_read"):
                continue
            reads = set().union(*[_regs(o) for o in (nops[1:] if nop.startswith(("v_", "global_load", "ds_")) else nops)]) if nops else set()
            if nop.startswith("global_store") or nop.startswith("ds_write"):
                reads = set().union(*[_regs(o) for o in nops])
            clash = reads & dst
            assert not clash, f"{name}: {nop} reads {sorted(clash)} {fwd} instruction(s) after the MFMA that writes it"
    return n_mfma


@pytest.mark.skipif(not shutil.which(HIPCC), reason="hipcc not available")
def test_ring_kernel_has_no_unprotected_mfma_hazards():
    src = os.path.join(ROOT, "tilefusion_amd", "csrc", "gemm.hip")
    with tempfile.TemporaryDirectory() as d:
        out = os.path.join(d, "gemm.s")
        subprocess.check_call([HIPCC, "-O3", "-std=c++20", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
                               "-packed-fp32-ops", f"-I{ROOT}/include", f"-I{ROOT}/tilefusion_amd/include",
                               f"-I{ROOT}/tilefusion_amd/csrc", "-Wno-unused-command-line-argument", "--cuda-device-only",
                               "-S", "-x", "hip", src, "-o", out], stderr=subprocess.DEVNULL)
        text = open(out).read()
    kernels = re.findall(r"^(_ZN3tfk\S*gemm_ring64_kernel\S*):[^\n]*\n(.*?)s_endpgm", text, flags=re.S | re.M)
    assert len(kernels) >= 6, "ring kernel instantiations (three shapes, fp16 and fp32 output) not found"
    for name, body in kernels:
        n_mfma = _check(name, body)
        assert n_mfma >= 32, f"{name}: expected the unrolled MFMA loop, found {n_mfma} MFMAs"


def test_checker_sees_planted_hazards():
    """The checker itself: a copy right in front of an MFMA and a store right behind one."""
    ok = "v_mov_b32 v1, v9\ns_nop 1\ns_nop 1\nv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]\ns_nop 15\nv_accvgpr_read_b32 v8, a0\n"
    assert _check("ok", ok) == 1
    with pytest.raises(AssertionError, match="before an MFMA"):
        _check("bad", "v_accvgpr_write_b32 a2, v9\nv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]\n")
    with pytest.raises(AssertionError, match="after the MFMA"):
        _check("bad", "v_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]\nv_accvgpr_read_b32 v8, a1\n")
