#!/usr/bin/env python3
"""Writes tests/golden/abi_layout.txt: sizes, member offsets and enumerator values of the marmot types the HIP
backend touches, printed by abi_probe.c compiled against the reference's own headers (run where the reference tree
is present). tests/test_backend_abi.py compares the mirror in include/marmot_hip_backend.h with this file."""
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
REF = os.environ.get("MARMOT_REFERENCE", "/root/reference")
CLANG = "/opt/rocm/llvm/bin/clang"


def reference_layout() -> str:
    with tempfile.TemporaryDirectory() as tmp:
        exe = os.path.join(tmp, "abi_ref")
        subprocess.run(
            [CLANG, "-std=c2x", "-D_GNU_SOURCE", "-DABI_PROBE_REFERENCE", f"-I{REF}/include", f"-I{REF}/src",
             f"-I{REF}", "-o", exe, os.path.join(HERE, "abi_probe.c")], check=True)
        return subprocess.run([exe], check=True, capture_output=True, text=True).stdout


if __name__ == "__main__":
    if not os.path.isdir(REF):
        sys.exit(f"reference tree not found at {REF}")
    out = os.path.join(HERE, "abi_layout.txt")
    with open(out, "w") as f:
        f.write(reference_layout())
    print("wrote", out)
