"""Build recipe: compiles the HIP library, the workload generator and (through oracle/Makefile)
the test oracle.  Everything is built in-tree so the shared objects travel with the source tree.

    python -m library_amd.build            # build everything
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libalphasparse_amd.so")
WORKLOADS = os.path.join(HERE, "libasx_workloads.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

HIP_SOURCES = ["asx_analysis.hip", "asx_spmv.hip", "asx_spmm.hip", "asx_capi.hip", "asx_blocked.hip", "asx_coo.hip", "asx_convert.hip", "asx_sliced.hip", "asx_window.hip"]
CXX_SOURCES = ["asx_rowblocks.cpp", "alphasparse_generic.cpp", "asx_mtx.cpp"]

# packed-fp32 code generation is switched off for all device code
HIP_FLAGS = ["--offload-arch=gfx950", "-std=c++17", "-O3", "-fPIC", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Rpass-analysis=kernel-resource-usage"]  # registers, LDS and scratch of every kernel, read below
CXX_FLAGS = ["-std=c++17", "-O2", "-fPIC", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include"]


def _run(cmd, **kw):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True, **kw)


def kernel_resources(compiler_output):
    """Per kernel of this library (asx::...), from the compiler's kernel-resource-usage remarks:
    {mangled name: {"VGPRs": .., "TotalSGPRs": .., "ScratchSize": .., "LDS Size": .., "Occupancy": ..}}."""
    table, cur = {}, None
    for line in compiler_output.splitlines():
        if "remark:" not in line:
            continue
        body = line.split("remark:", 1)[1].replace("[-Rpass-analysis=kernel-resource-usage]", "").strip()
        if body.startswith("Function Name:"):
            name = body.split(":", 1)[1].strip()
            cur = table.setdefault(name, {}) if "3asx" in name else None
        elif cur is not None and ":" in body:
            key, value = body.rsplit(":", 1)
            key = key.split("[")[0].strip()
            try:
                cur[key] = int(value)
            except ValueError:
                cur[key] = value.strip()
    return table


def build_library(verbose=False):
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    procs = []
    for src in HIP_SOURCES:
        obj = os.path.join(objdir, src + ".o")
        cmd = [HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    for src in CXX_SOURCES:
        obj = os.path.join(objdir, src + ".o")
        cmd = ["g++", *CXX_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    failed = False
    resources = {}
    for cmd, p in procs:
        out = p.communicate()[0].decode(errors="replace")
        resources.update(kernel_resources(out))
        lines, skip = [], 0
        for l in out.splitlines():  # drop the resource remarks (and the two source lines echoed after each)
            if skip:
                skip -= 1
            elif "kernel-resource-usage" in l:
                skip = 2 if "Function Name" in l else 0
            elif "packed-fp32-ops" not in l:
                lines.append(l)
        if p.returncode != 0 or verbose:
            print("\n".join(lines))
        elif lines:
            print("\n".join(l for l in lines if "warning" in l or "error" in l))
        failed |= p.returncode != 0
    if failed:
        raise RuntimeError("compilation failed")
    # A kernel that spills registers to scratch memory pays for it with memory traffic in its inner
    # loop (measured: 0.44 GB a call in one variant of the window kernel): not accepted silently.
    with open(os.path.join(objdir, "kernel_resources.txt"), "w") as f:
        for name in sorted(resources):
            r = resources[name]
            f.write(f"{name} vgpr={r.get('VGPRs')} sgpr={r.get('TotalSGPRs')} scratch={r.get('ScratchSize')} "
                    f"lds={r.get('LDS Size')} occupancy={r.get('Occupancy')}\n")
    spilling = sorted(n for n, r in resources.items() if r.get("ScratchSize", 0))
    if spilling:
        raise RuntimeError("kernels that spill registers to scratch memory: " + ", ".join(spilling))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,--version-script=" + os.path.join(CSRC, "exports.map"),
          "-o", LIB, *objs])
    return LIB


def build_workloads():
    _run(["gcc", "-O2", "-ffp-contract=off", "-fopenmp", "-fPIC", "-shared", "-Wall", "-o", WORKLOADS,
          os.path.join(CSRC, "workload_gen.c"), "-lm"])
    return WORKLOADS


def build_oracle():
    targets = ["oracle"]
    if os.path.isdir(os.environ.get("ASX_REFERENCE", "/root/reference")):
        targets.append("ref")  # only where the reference sources are mounted
    _run(["make", "-C", os.path.join(ROOT, "oracle"), "-j8", *targets])


def build_cxx_example():
    """A caller of the generic C++ API, written like the reference's GPU tests; used by tests/."""
    src = os.path.join(ROOT, "tests", "cxx", "generic_api_caller.cpp")
    exe = os.path.join(ROOT, "tests", "cxx", "generic_api_caller")
    _run([HIPCC, "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-O2", "-Wall",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-I" + os.path.join(ROOT, "include"), src, "-o", exe,
          "-L" + HERE, "-lalphasparse_amd", "-Wl,-rpath," + HERE, "-Wl,-rpath,$ORIGIN/../../library_amd"])
    return exe


def build_cli():
    """The command-line driver (MatrixMarket file -> SpMV / SpMM timings), library_amd/bin/."""
    src = os.path.join(HERE, "cli", "alphasparse_amd_cli.cpp")
    bindir = os.path.join(HERE, "bin")
    os.makedirs(bindir, exist_ok=True)
    exe = os.path.join(bindir, "alphasparse_amd_cli")
    _run([HIPCC, "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-O2", "-Wall",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-I" + os.path.join(ROOT, "include"), src, "-o", exe,
          "-L" + HERE, "-lalphasparse_amd", "-Wl,-rpath," + HERE, "-Wl,-rpath,$ORIGIN/.."])
    return exe


def build_all():
    build_workloads()
    build_library()
    build_cli()
    build_oracle()


if __name__ == "__main__":
    build_all()
    build_cxx_example()
    sys.exit(0)
