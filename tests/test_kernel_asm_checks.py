"""Checks on the compiler's assembly for the grouped GEMM source (no GPU needed: hipcc cross-compiles).

The GEMM issues its LDS-DMA transfers from inline asm with the 64-bit base in scalar registers. When that base was
produced by a vector instruction (v_readfirstlane, v_readlane, a compare), the hardware wants five wait states before
a vector-memory instruction reads it. The compiler inserts such waits for its own instructions but does not look
inside asm text, so the asm carries them itself; this test reads the generated assembly and counts them. It also holds
the kernels to zero spilled vector registers: a reload inside the K loop waits for the slabs in flight.
"""
import os
import re
import shutil
import subprocess

import pytest

from memfabric_hybrid_amd import build

HIPCC = os.path.join(build.ROCM, "bin", "hipcc")
REQUIRED_WAIT_STATES = 5


@pytest.fixture(scope="module")
def gemm_asm(tmp_path_factory):
    if not (os.path.exists(HIPCC) or shutil.which("hipcc")):
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("asm") / "gemm.s"
    src = os.path.join(build.CSRC, "kernels", "gemm.hip")
    cmd = [HIPCC] + build.HIP_FLAGS + build.INCLUDES + ["--cuda-device-only", "-S", src, "-o", str(out)]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    return out.read_text().split("\n")


def _is_instruction(line):
    t = line.strip()
    return bool(t) and not t.startswith(";") and not t.startswith(".") and not t.endswith(":")


def _short_waits(lines):
    """(line number, instruction, writer, wait states) for every vector-memory read of a too-fresh scalar base"""
    found, total = [], 0
    vmem = re.compile(r"(global_load_lds_dword(?:x4)?|global_load_dword(?:x[234])?)\s+(?:v\[?[\d:]+\]?,\s*)?v\d+,\s*s\[(\d+):(\d+)\]")
    for i, line in enumerate(lines):
        m = vmem.match(line.strip())
        if not m:
            continue
        total += 1
        base = {int(m.group(2)), int(m.group(3))}
        states, j = 0, i - 1
        while j >= 0 and states < REQUIRED_WAIT_STATES:
            u = lines[j].strip()
            if _is_instruction(u):
                w = re.match(r"v_\S+\s+s(\d+)\b", u)
                wr = re.match(r"v_\S+\s+s\[(\d+):(\d+)\]", u)
                written = set()
                if w:
                    written = {int(w.group(1))}
                elif wr:
                    written = set(range(int(wr.group(1)), int(wr.group(2)) + 1))
                if written & base:
                    found.append((i + 1, line.strip(), u, states))
                    break
                nop = re.match(r"s_nop\s+(\d+)", u)
                states += int(nop.group(1)) + 1 if nop else 1
            j -= 1
    return found, total


def test_scanner_sees_a_short_wait():
    lines = ["\tv_readfirstlane_b32 s9, v3", "\tv_readfirstlane_b32 s8, v2", "\ts_mov_b32 m0, s28", "\ts_nop 0",
             "\tglobal_load_lds_dwordx4 v25, s[8:9]"]
    found, total = _short_waits(lines)
    assert total == 1 and len(found) == 1 and found[0][3] == 2
    lines[3] = "\ts_nop 3"
    assert _short_waits(lines) == ([], 1)


def test_dma_transfers_wait_for_their_scalar_base(gemm_asm):
    found, total = _short_waits(gemm_asm)
    assert total > 1000, "the scan did not find the kernels' LDS-DMA transfers (%d)" % total
    assert not found, "scalar base read too early by %d of %d transfers, e.g. %r" % (len(found), total, found[:3])


def test_gemm_kernels_spill_no_vector_registers(gemm_asm):
    counts = [int(m.group(1)) for m in (re.search(r"\.vgpr_spill_count:\s+(\d+)", l) for l in gemm_asm) if m]
    assert len(counts) >= 20, counts
    assert all(c == 0 for c in counts), counts
