"""A property of the compiled forward kernels that no run-time test can see reliably.

The forward requests its tile-map words with scalar loads in one inline-assembly statement and waits
for them in another, much later, so that the address arithmetic in between hides their latency.
The compiler does not know that the registers are still in flight in between: if it ever read,
copied or redefined them there, the kernel would use stale words once in a while.  This test
compiles `attn_fwd.hip` to assembly (no GPU needed) and checks, for every kernel in it, that no
instruction between the two statements names those registers."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "sparse-mask-attention_amd", "csrc")


def _registers(line):
    regs = set(re.findall(r"\bs(\d+)\b", line))
    for a, b in re.findall(r"s\[(\d+):(\d+)\]", line):
        regs |= {str(k) for k in range(int(a), int(b) + 1)}
    return regs


def test_tile_map_words_are_not_touched_while_in_flight(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    out = tmp_path / "attn_fwd.s"
    subprocess.run([hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fno-finite-math-only",
                    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-inline-asm",
                    f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}", "-S", "--cuda-device-only",
                    os.path.join(CSRC, "attn_fwd.hip"), "-o", str(out)],
                   check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    lines = out.read_text().split("\n")
    kernel, pending, sites, i = None, None, 0, 0
    while i < len(lines):
        line = lines[i]
        m = re.match(r"^(_ZN3sma\S+):", line)
        if m:
            kernel, pending = m.group(1), None
        if "ASMSTART" in line:
            j, block = i + 1, []
            while "ASMEND" not in lines[j]:
                block.append(lines[j].strip())
                j += 1
            loads = [b for b in block if b.startswith("s_load_dword")]
            waits = [b for b in block if b.startswith("s_waitcnt lgkmcnt(0)")]
            if loads and not waits:                      # the requesting statement
                pending = set()
                for b in loads:
                    pending |= _registers(b.split(",")[0])
                sites += 1
            elif waits and not loads:                    # the awaiting statement
                pending = None
            i = j + 1
            continue
        if pending and not line.strip().startswith(";") and not line.strip().startswith("."):
            assert not (_registers(line) & pending), f"{kernel}: '{line.strip()}' touches a map word in flight"
        i += 1
    assert sites >= 24, "the scalar loads of the tile map were not found: has the prologue changed?"
