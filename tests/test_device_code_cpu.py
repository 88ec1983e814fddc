"""What the compiler made of the kernels, read from its assembly output for
gfx950 (the device pass alone, a few seconds per file; nothing is launched).

Rules that the sources are written to keep, and that a later edit could break
without any test on a quiet GPU noticing:

* A buffer store of more than 8 bytes per lane takes its row offset in the
  lane's offset register, never in the scalar offset field.  With a scalar
  register in that field the compiler takes such a store to need no distance
  from an instruction that overwrites its data registers, and schedules the
  next arithmetic right behind it.  On MI355X the store then wrote, now and
  then and only with many wavefronts resident, what that arithmetic had just
  put into the registers (in the linear-domain sweeps: the lower 8 bytes of
  the last four lanes of a row of 16).  With a constant in the field the
  compiler keeps the distance itself; the second test checks that it does.
* No packed single-precision arithmetic: the build switches the feature off,
  and no source asks for it by hand.
* The lattice kernels stay within the registers that their occupancy rests on.
"""
import glob
import os
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "warp-ctct_amd")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
WIDE_STORE = re.compile(r"(buffer_store_dwordx[34]|buffer_store_format_xyzw?|buffer_store_format_d16_xyzw?)\s+"
                        r"(\S+)\s+(\S+)\s+(\S+)\s+(\S+)")


def _assemble(src, out_dir):
    out = os.path.join(out_dir, os.path.basename(src)[:-4] + ".s")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-I" + os.path.join(PKG, "csrc"), "-I" + os.path.join(ROOT, "include"),
           "-Wno-unused-command-line-argument", "-S", "--cuda-device-only", "-o", out, src]
    done = subprocess.run(cmd, capture_output=True, text=True, timeout=900)
    assert done.returncode == 0, done.stderr[-4000:]
    return out


@pytest.fixture(scope="module")
def listings(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    out_dir = str(tmp_path_factory.mktemp("device_asm"))
    sources = sorted(glob.glob(os.path.join(PKG, "csrc", "*.hip")))
    assert sources
    with ThreadPoolExecutor(max_workers=4) as pool:
        files = list(pool.map(lambda s: _assemble(s, out_dir), sources))
    return {os.path.basename(f): open(f).read().split("\n") for f in files}


def _instructions(lines):
    """(line number, text) of every instruction, labels, directives and comments left out."""
    for i, raw in enumerate(lines):
        text = raw.split(";")[0].strip()
        if text and not text.startswith(".") and not text.endswith(":"):
            yield i + 1, text


def _registers(operand):
    operand = operand.rstrip(",")
    m = re.match(r"[va]\[(\d+):(\d+)\]$", operand)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"[va](\d+)$", operand)
    return {int(m.group(1))} if m else set()


def test_wide_buffer_stores_take_no_scalar_register_as_their_offset(listings):
    found, stores = [], 0
    for name, lines in listings.items():
        for at, text in _instructions(lines):
            m = WIDE_STORE.match(text)
            if not m:
                continue
            stores += 1
            offset = m.group(5).rstrip(",")
            if not re.fullmatch(r"-?\d+|0x[0-9a-fA-F]+", offset):
                found.append("%s:%d: %s" % (name, at, text))
    assert stores > 0   # the sweeps do store 16 bytes per lane
    assert not found, "\n".join(found[:20])


def test_nothing_overwrites_the_data_of_a_wide_store_within_two_instructions(listings):
    found = []
    for name, lines in listings.items():
        code = list(_instructions(lines))
        for k, (at, text) in enumerate(code):
            m = re.match(r"(buffer|global|flat|scratch)_store_(dwordx[34]|format_xyzw?)\s+(.*)", text)
            if not m:
                continue
            operands = m.group(3).split()
            # the data: the first operand of a buffer store, the second of the others
            data = _registers(operands[0]) if m.group(1) == "buffer" else _registers(operands[1])
            slots, j = 0, k + 1
            while slots < 2 and j < len(code):
                op = code[j][1].split()
                j += 1
                if op[0] == "s_nop":
                    slots += 1 + int(op[1], 0)
                    continue
                slots += 1
                writes = op[0].startswith("v_") and not op[0].startswith(("v_cmp", "v_readlane", "v_readfirstlane"))
                if writes and len(op) > 1 and _registers(op[1]) & data:
                    found.append("%s:%d: %s  <-  %s" % (name, at, text, " ".join(op)))
    assert not found, "\n".join(found[:20])


def test_no_packed_single_precision_arithmetic(listings):
    found = []
    for name, lines in listings.items():
        for at, text in _instructions(lines):
            if re.match(r"v_pk_(add|mul|fma)_f32\b", text):
                found.append("%s:%d: %s" % (name, at, text))
    assert not found, "\n".join(found[:20])


def test_register_budgets_that_the_occupancy_rests_on(listings):
    """lattice_fill_kernel's clearing workgroups carry the sweeps' register
    allocation: up to 168 registers per lane three workgroups of 256 threads share
    a compute unit, with more only two, and the clear that the typical batch's
    step consists of takes 3 % longer.  The sweeping kernels must leave room for
    two wavefronts per SIMD (256), and none of the three may spill to scratch
    memory."""
    budgets = {"lattice_fill_kernel": 168, "lattice_kernelE": 256, "lattice_lin_kernel": 256}
    seen = {}
    for name, lines in listings.items():
        text = "\n".join(lines)
        for block in text.split("  - .agpr_count")[1:]:
            kernel = re.search(r"\.name:\s+(\S+)", block).group(1)
            vgprs = int(re.search(r"\.vgpr_count:\s+(\d+)", block).group(1))
            spilled = int(re.search(r"\.vgpr_spill_count:\s+(\d+)", block).group(1))
            for key, most in budgets.items():
                if key in kernel:
                    seen[key] = vgprs
                    assert vgprs <= most, (kernel, vgprs, most)
                    assert spilled == 0, (kernel, spilled)
    assert set(seen) == set(budgets), seen
