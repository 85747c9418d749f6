"""The 16-row MFMA atoms are written as inline assembly (gemm_kernel.hip.inc: Mma<*, 16>), so the compiler places none of the
wait states an MFMA needs around them.  This test compiles a few of those kernels to gfx950 ISA (no GPU needed) and
checks the two patterns that would be wrong: a vector instruction writing a register that an MFMA reads within the next
few instructions (accumulator initialisation right before the first MFMA), and a vector instruction reading an MFMA
result too soon after it (before the drain the kernel issues ahead of the epilogue)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "frisk_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

SOURCE = """
#include "gemm_kernel.hip.inc"
namespace frisk {
template __global__ void gemm_kernel<GemmCfg<FRISK_F16, 0, 1, 256, 256, 64, 2, 2, 2, false, false, 1, 3, 16>>(GemmParams);
template __global__ void gemm_kernel<GemmCfg<FRISK_F16, 0, 0, 256, 256, 64, 2, 2, 2, false, true, 1, 3, 16>>(GemmParams);
template __global__ void gemm_kernel<GemmCfg<FRISK_BF16, 1, 1, 256, 256, 64, 2, 2, 2, false, false, 1, 3, 16>>(GemmParams);
template __global__ void gemm_kernel<GemmCfg<FRISK_I8, 1, 0, 256, 256, 128, 2, 2, 2, false, false, 1, 3, 16>>(GemmParams);
template __global__ void gemm_kernel<GemmCfg<FRISK_E4M3, 0, 1, 256, 256, 128, 2, 2, 2, false, false, 1, 3, 16>>(GemmParams);
}
"""


def _registers(text):
    out = set()
    for kind, lo, hi in re.findall(r"\b([av])\[(\d+):(\d+)\]", text):
        out.update(kind + str(r) for r in range(int(lo), int(hi) + 1))
    out.update(kind + n for kind, n in re.findall(r"\b([av])(\d+)\b", text))
    return out


def _operands(line):
    parts = line.split(None, 1)
    return parts[1].split(",") if len(parts) > 1 else []


def hazards(listing, window_before=8, window_after=12):
    found = []
    for kernel in re.split(r"\n\t\.globl\t", listing)[1:]:
        name = kernel.split("\n")[0]
        lines = [l.strip() for l in kernel.split("\n") if l.startswith("\t") and not l.strip().startswith((".", ";"))]
        for i, line in enumerate(lines):
            if not line.startswith("v_mfma"):
                continue
            ops = _operands(line)
            reads, result = _registers(",".join(ops)), _registers(ops[0])
            multiplicands = _registers(",".join(ops[1:3])) - result
            for back in range(1, window_before + 1):
                prev = lines[i - back] if i - back >= 0 else ""
                if prev.startswith("v_") and not prev.startswith("v_mfma"):
                    written = _registers((_operands(prev) or [""])[0]) & reads
                    # a multiplicand written by an ordinary vector instruction is interlocked by the hardware (only the accumulator
                    # operand needs wait states); keep two instructions of distance anyway
                    if written - multiplicands or (written and back <= 2):
                        found.append((name, prev, line))
            for fwd in range(1, window_after + 1):
                nxt = lines[i + fwd] if i + fwd < len(lines) else ""
                if nxt.startswith("v_") and not nxt.startswith("v_mfma") and _registers(",".join(_operands(nxt)[1:])) & result:
                    found.append((name, line, nxt))
    return found


def foreign_m0_uses(listing, reach=6):
    """lines that name M0 outside the transfers the kernels write themselves: s_add_u32 m0 followed, within a few
    instructions that do not name M0 (an MFMA and scalar address arithmetic may sit between the two halves of a transfer), by
    its global_load_lds_dwordx4.  The transfer writes M0 without telling the compiler, which is only sound while the
    compiler has no use of M0 of its own in the kernel."""
    lines = [l.strip() for l in listing.split("\n") if l.startswith("\t") and not l.strip().startswith((".", ";"))]
    found = []
    for i, line in enumerate(lines):
        if not re.search(r"\bm0\b", line):
            continue
        own = False
        if line.startswith("s_add_u32 m0, "):
            for nxt in lines[i + 1:i + 1 + reach]:
                if nxt.startswith("global_load_lds_dwordx4"):
                    own = True
                    break
                if re.search(r"\bm0\b", nxt):
                    break
        if not own:
            found.append(line)
    return found


def test_scanner_sees_both_patterns():
    listing = "\n\t.globl\tk\nk:\n\tv_accvgpr_mov_b32 a5, a1\n\ts_nop 0\n\tv_mfma_f32_16x16x32_f16 a[4:7], v[0:3], v[4:7], a[4:7]\n\tv_accvgpr_read_b32 v9, a6\n"
    got = hazards(listing)
    assert len(got) == 2 and got[0][1].startswith("v_accvgpr_mov") and got[1][2].startswith("v_accvgpr_read")
    assert foreign_m0_uses("\ts_add_u32 m0, s4, 0x400\n\ts_nop 0\n\tglobal_load_lds_dwordx4 v1, s[2:3]\n\ts_mov_b32 m0, s7\n\tds_read_b32 v1, v2\n") == ["s_mov_b32 m0, s7"]
    split = "\ts_add_u32 m0, s4, 0x400\n\tv_mfma_f32_16x16x32_f16 a[4:7], v[0:3], v[4:7], a[4:7]\n\ts_add_u32 s8, s8, s0\n\tglobal_load_lds_dwordx4 v1, s[8:9]\n"
    assert foreign_m0_uses(split) == [] and foreign_m0_uses(split.replace("s_add_u32 s8, s8, s0", "s_add_u32 m0, s4, 0x800")) == ["s_add_u32 m0, s4, 0x400"]
    clean = "\n\t.globl\tk\nk:\n\tv_mfma_f32_16x16x32_f16 a[4:7], v[0:3], v[4:7], a[4:7]\n\tv_mfma_f32_16x16x32_f16 a[8:11], v[0:3], v[4:7], a[8:11]\n"
    assert hazards(clean) == []


@pytest.mark.skipif(not (os.path.exists(HIPCC) or shutil.which("hipcc")), reason="needs hipcc to produce the ISA listing")
def test_inline_assembly_mfma_kernels_keep_their_wait_states(tmp_path):
    src = tmp_path / "atoms16.hip"
    src.write_text(SOURCE)
    out = tmp_path / "atoms16.s"
    cmd = [HIPCC if os.path.exists(HIPCC) else "hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-Wno-unused-command-line-argument", "--cuda-device-only", "-S", str(src), "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    listing = out.read_text()
    assert listing.count("v_mfma_f32_16x16x32_f16") > 300 and "v_mfma_i32_16x16x64_i8" in listing and "v_mfma_f32_16x16x32_bf16" in listing
    assert listing.count("v_mfma_f32_16x16x128_f8f6f4") >= 64 * 7 and "scratch_" not in listing  # seven tile bodies, no spills
    bad = hazards(listing)
    assert not bad, "\n".join("%s: %s  ->  %s" % (n[:60], a, b) for n, a, b in bad[:10])
    assert listing.count("global_load_lds_dwordx4") > 100 and foreign_m0_uses(listing) == []


@pytest.mark.skipif(not (os.path.exists(HIPCC) or shutil.which("hipcc")), reason="needs hipcc to produce the ISA listing")
def test_attention_kernel_has_no_use_of_m0_besides_its_transfers(tmp_path):
    """the attention kernel stages K and V with the same transfers (csrc/attention.hip: SK / SV issue_one): M0 is written by inline
    assembly without a clobber, so the compiler must have no use of M0 of its own in that kernel either"""
    out = tmp_path / "attention.s"
    cmd = [HIPCC if os.path.exists(HIPCC) else "hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-Wno-unused-command-line-argument", "--cuda-device-only", "-S", os.path.join(CSRC, "attention.hip"), "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    listing = out.read_text()
    assert listing.count("global_load_lds_dwordx4") >= 4 * 16 and listing.count("v_mfma_f32_32x32x16") >= 4 * 32  # four kernels (f16 / bf16, two K layouts)
    assert foreign_m0_uses(listing) == [] and "scratch_" not in listing
