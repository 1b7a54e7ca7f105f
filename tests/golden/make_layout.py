#!/usr/bin/env python3
"""Writes tests/golden/layout.json: sizes and field offsets of the reference's boundary structs.

Compiles tests/golden/layout_probe.cpp against the reference's own headers
(/root/reference/include, or $ASX_REFERENCE/include) with hipcc (host pass; the headers carry
device code that a plain host compiler rejects) and runs the resulting host program, which calls
no HIP function.  Only the numbers are committed; run in the build container, where the
reference sources are mounted.
"""
import json
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
REF = os.environ.get("ASX_REFERENCE", "/root/reference")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def main():
    inc = os.path.join(REF, "include")
    if not os.path.isdir(inc):
        sys.exit(f"{inc} not found: the layout fixture can only be regenerated where the reference is mounted")
    with tempfile.TemporaryDirectory() as tmp:
        exe = os.path.join(tmp, "layout_probe")
        subprocess.run([HIPCC, "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-w", "-D__HIP__", "-I" + inc,
                        os.path.join(HERE, "layout_probe.cpp"), "-o", exe], check=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    data = json.loads(out)
    data.pop("end", None)
    with open(os.path.join(HERE, "layout.json"), "w") as f:
        json.dump(data, f, indent=1, sort_keys=True)
        f.write("\n")
    print(f"wrote {len(data)} entries")


if __name__ == "__main__":
    main()
