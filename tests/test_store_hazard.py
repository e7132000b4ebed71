"""A check on the generated code, not on results: no kernel of the library may contain a buffer store of more
than 64 bits whose scalar offset is a register.

On gfx950 a vector write to the first data register of such a store, issued directly behind it, corrupted the
stored dword in lanes 12-15 of every 16 (seen in the Winograd forward kernel's store loop).  The compiler
inserts the wait state between a wide store and a write to its data registers only when the store's scalar
offset is an immediate, so the kernels add run-time offsets to the vector offset instead; this test compiles
every source file to assembly (device side only, a few seconds each) and looks for the pattern."""
import glob
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "pipedream_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
WIDE_STORE_WITH_REGISTER_OFFSET = re.compile(
    r"buffer_store_(dwordx[34]|format_xyzw?)\s+v\[\d+:\d+\],\s*[^,]+,\s*s\[\d+:\d+\],\s*(s\d+|m0|ttmp\d+)\b")


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc")
@pytest.mark.parametrize("source", sorted(os.path.basename(p) for p in glob.glob(os.path.join(CSRC, "*.hip"))))
def test_no_wide_buffer_store_with_a_register_scalar_offset(source, tmp_path):
    out = tmp_path / (source + ".s")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"),
           "-I" + CSRC, "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only",
           os.path.join(CSRC, source), "-o", str(out)]
    done = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, universal_newlines=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    bad = [line.strip() for line in out.read_text().splitlines() if WIDE_STORE_WITH_REGISTER_OFFSET.search(line)]
    assert not bad, bad[:5]
