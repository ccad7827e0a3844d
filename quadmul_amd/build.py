"""Build recipe for the gfx950 library and the PyTorch-ROCm extension, in-tree.

    python -m quadmul_amd.build            # both
    python -m quadmul_amd.build --lib      # libqm_hip.so only (hipcc, no torch needed)

Outputs (git-ignored, but they travel with the tree):
    quadmul_amd/lib/libqm_hip.so                      hand-written HIP kernels + C ABI
    quadmul.cpython-<abi>.so  (repo root)             module `quadmul`, host-only C++

The kernels are compiled by hipcc for gfx950 only; the extension is compiled by
the host compiler against torch's headers and calls the library through
include/qm_abi.h.  Takes the place of the reference's setup.py:1-17 (nvcc +
CUDAExtension), without torch's source-translation step.
"""
from __future__ import annotations

import argparse
import glob
import os
import re
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(PKG, "build")
LIB_PATH = os.path.join(LIBDIR, "libqm_hip.so")
PROBE_PATH = os.path.join(LIBDIR, "libqm_probe.so")
N_TILE_TUS = 14

HIPCC = os.environ.get("HIPCC", shutil.which("hipcc") or "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm", "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def ext_path() -> str:
    return os.path.join(ROOT, "quadmul" + sysconfig.get_config_var("EXT_SUFFIX"))


# The compilers the full GPU suite has passed with.  The kernels order matrix-core
# instructions and their hazards by hand inside asm statements; another compiler may schedule
# the code around them differently, so a build with one is refused unless
# QM_ALLOW_UNVALIDATED_COMPILER=1 says to go ahead (tests/ -m gpu is the gate for adding one).
VALIDATED_COMPILERS = ("HIP version: 7.2",)


def compiler_version() -> str:
    try:
        out = subprocess.run([HIPCC, "--version"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True).stdout
    except OSError:
        return "unknown compiler"
    lines = [l.strip() for l in out.splitlines() if l.strip()]
    hip = next((l for l in lines if l.startswith("HIP version")), "")
    clang = next((l for l in lines if "clang version" in l), "")
    clang = clang.split("(")[0].strip()
    return "; ".join(x for x in (hip, clang) if x) or "unknown compiler"


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    return out


# A memory instruction must not read a scalar register within five wait states of a vector
# instruction that wrote it (v_readlane, v_readfirstlane, a comparison into a register pair).
# The compiler inserts the wait states for its own memory instructions and cannot for the
# ones inside asm statements -- the ring's loads and the stores of tiles that stick out of C
# take a base pointer in scalar registers -- so the generated code is scanned for it.
_ASM_VMEM = re.compile(r"global_(?:store_dwordx[24]|load_lds_dwordx4)\s.*\bs\[(\d+):(\d+)\]")


def scalar_operand_hazards(isa_path: str):
    """(line number, writer, reader) for every load/store with a scalar base in the device
    assembly at ``isa_path`` whose base a vector instruction wrote fewer than five wait
    states before."""
    lines = open(isa_path).read().split("\n")
    found = []
    for i, line in enumerate(lines):
        m = _ASM_VMEM.search(line)
        if not m:
            continue
        lo, hi = int(m[1]), int(m[2])
        waited, j = 0, i - 1
        while j >= 0 and waited < 5:
            t = lines[j].strip()
            j -= 1
            if not t or t[0] in ";." or t.endswith(":"):
                continue
            if re.match(r"v_(?:readlane|readfirstlane)_b32 s(?:%d|%d)\b" % (lo, hi), t) or re.match(r"v_cmp\S* s\[%d:%d\]" % (lo, hi), t):
                found.append((i + 1, t, line.strip()))
                break
            nop = re.match(r"s_nop (\d+)", t)
            waited += int(nop[1]) + 1 if nop else 1
    return found


def build_lib(jobs: int = 8, verbose: bool = False) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    ver = compiler_version()
    if not any(ver.startswith(v) for v in VALIDATED_COMPILERS):
        msg = (f"building with {ver!r}, which the GPU test-suite has not been run with "
               f"(validated: {', '.join(VALIDATED_COMPILERS)})")
        if os.environ.get("QM_ALLOW_UNVALIDATED_COMPILER") != "1":
            raise RuntimeError(f"quadmul_amd.build: refusing: {msg}.  The kernels order matrix-core instructions and their "
                               "hazards by hand; set QM_ALLOW_UNVALIDATED_COMPILER=1 to build anyway, then run "
                               "`pytest tests -m gpu` before trusting any result and add the compiler to VALIDATED_COMPILERS")
        print(f"quadmul_amd.build: WARNING: {msg}; run `pytest tests -m gpu` before trusting results", file=sys.stderr)
    units = [("qm_dispatch.o", [f'-DQM_COMPILER_VERSION="{ver}"', "-mllvm", "-amdgpu-kernarg-preload-count=16", "-c", os.path.join(CSRC, "qm_dispatch.hip")]),
             ("qm_scratch.o", ["-c", os.path.join(CSRC, "qm_scratch.hip")])]
    # (the units with the scaled-output kernels, 6 and up, take longest: they go first)
    units = [(f"qm_tile_inst_{tu}.o", [f"-DQM_TU={tu}", "-c", os.path.join(CSRC, "qm_tile_inst.hip")])
             for tu in sorted(range(N_TILE_TUS), key=lambda t: (t < 6, t))] + units
    # (a directory per unit: the compiler's intermediate files, kept for the scan below, are
    # named after the source file, which the tile units share)
    objs = [os.path.join(OBJDIR, name[:-2], name) for name, _ in units]

    def compile_one(item):
        (name, args), obj = item
        shutil.rmtree(os.path.dirname(obj), ignore_errors=True)
        os.makedirs(os.path.dirname(obj))
        return _run([HIPCC] + HIP_FLAGS + ["-save-temps=obj"] + args + ["-o", obj])

    with ThreadPoolExecutor(max_workers=max(1, min(jobs, 16))) as pool:
        for out in pool.map(compile_one, zip(units, objs)):
            if verbose and out.strip():
                print(out)
    hazards = []
    for obj in objs:
        for isa in glob.glob(os.path.join(os.path.dirname(obj), "*-amdgcn-amd-amdhsa-gfx950.s")):
            hazards += [(os.path.basename(os.path.dirname(obj)),) + h for h in scalar_operand_hazards(isa)]
        for junk in glob.glob(os.path.join(os.path.dirname(obj), "*")):
            if junk != obj:
                os.remove(junk)
    if hazards:
        raise RuntimeError("quadmul_amd.build: a load or store inside an asm statement reads a scalar register that a vector "
                           "instruction wrote fewer than five wait states before (unit, line, writer, reader):\n  " +
                           "\n  ".join(str(h) for h in hazards[:20]) + f"\n  ({len(hazards)} in all)")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs)
    return LIB_PATH


def build_probe(verbose: bool = False) -> str:
    """The measurement probes of bench.py (MFMA issue rate, launch floor, read floor): a
    library of their own, not linked into libqm_hip.so."""
    os.makedirs(LIBDIR, exist_ok=True)
    out = _run([HIPCC] + HIP_FLAGS + ["-shared", os.path.join(CSRC, "qm_probe.hip"), "-o", PROBE_PATH])
    if verbose and out.strip():
        print(out)
    return PROBE_PATH


def build_ext(verbose: bool = False) -> str:
    import torch
    from torch.utils import cpp_extension

    if not os.path.exists(LIB_PATH):
        raise RuntimeError("build libqm_hip.so first")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    incs = cpp_extension.include_paths() + [os.path.join(rocm, "include"), os.path.join(ROOT, "include"), sysconfig.get_paths()["include"]]
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=quadmul", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-deprecated-declarations"]
    for i in incs:
        cmd += ["-isystem", i]
    cmd += [os.path.join(CSRC, "ext.cpp"), "-o", ext_path(),
            "-L", LIBDIR, "-lqm_hip", "-L", torch_lib, "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip",
            "-Wl,-rpath,$ORIGIN/quadmul_amd/lib", "-Wl,-rpath," + torch_lib]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return ext_path()


def build_all(jobs: int = 8, verbose: bool = False):
    return build_lib(jobs, verbose), build_probe(verbose), build_ext(verbose)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--lib", action="store_true", help="build only libqm_hip.so")
    ap.add_argument("--ext", action="store_true", help="build only the torch extension")
    ap.add_argument("-j", "--jobs", type=int, default=8)
    ap.add_argument("-v", "--verbose", action="store_true")
    a = ap.parse_args(argv)
    if a.lib or not a.ext:
        print("built", build_lib(a.jobs, a.verbose))
        print("built", build_probe(a.verbose))
    if a.ext or not a.lib:
        print("built", build_ext(a.verbose))
    return 0


if __name__ == "__main__":
    sys.exit(main())
