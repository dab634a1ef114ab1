"""Compiles the HIP library for gfx950 in-tree: lib/libaccelgcn.so.

hipcc cross-compiles without a GPU.  Packed-FP32 instruction selection is
switched off for the device code (scalar fp32 FMAs are used instead).
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB = LIB_DIR / "libaccelgcn.so"
BIN_DIR = PKG / "bin"
SOURCES = ["capi.hip", "preprocess.hip", "spmm.hip", "state.hip", "dense.hip", "spmm_accel.cpp"]
ARCH = "gfx950"


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; the library cannot be built")
    return exe


def compile_flags():
    return ["-x", "hip", f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-Wall", "-Wno-unused-command-line-argument",
            f"-I{ROOT / 'include'}", f"-I{CSRC}"]


def build(verbose: bool = False) -> Path:
    """Compile every source and link lib/libaccelgcn.so, then the two programs in bin/
    and the comparison-baselines library."""
    LIB_DIR.mkdir(exist_ok=True)
    out = LIB
    objs = []
    procs = []
    for src in SOURCES:
        obj = out.parent / (out.stem + "." + src + ".o")
        cmd = [hipcc(), *compile_flags(), "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(str(obj))
    failed = []
    for src, p in procs:
        text, _ = p.communicate()
        if p.returncode != 0:
            failed.append((src, text))
        elif verbose and text.strip():
            print(text)
    if failed:
        raise RuntimeError("hipcc failed:\n" + "\n".join(f"--- {s}\n{o}" for s, o in failed))
    tmp = out.with_suffix(".so.tmp")
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", str(tmp)]
    subprocess.run(cmd, check=True)
    os.replace(tmp, out)
    for o in objs:
        os.unlink(o)
    build_cli(verbose)
    build_baselines(verbose)
    return out


def build_baselines(verbose: bool = False) -> Path:
    """lib/libaccelgcn_baselines.so: comparison baselines (rocSPARSE SpMM, a
    neighbour-partition kernel, rocBLAS SGEMM) and the pure-gather measurement probe.  Kept in its own library: the product library does
    not link any sparse library and holds no comparison code."""
    out = LIB_DIR / "libaccelgcn_baselines.so"
    cmd = [hipcc(), *compile_flags(), "-shared", str(PKG / "baselines" / "rocsparse_spmm.cpp"),
           str(PKG / "baselines" / "neighbor_partition_spmm.cpp"),
           str(PKG / "baselines" / "gather_probe.cpp"), str(PKG / "baselines" / "rocblas_gemm.cpp"),
           "-o", str(out), "-lrocsparse", "-lrocblas"]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for baselines/*.cpp:\n" + r.stdout)
    return out


def build_cli(verbose: bool = False) -> Path:
    """bin/spmm_test: the command-line harness (counterpart of upstream's main.cu);
    bin/operator_check: error paths of the C++ operator, run by the tests."""
    BIN_DIR.mkdir(exist_ok=True)
    for name in ("spmm_test", "operator_check"):
        exe = BIN_DIR / name
        cmd = [hipcc(), *compile_flags(), str(CSRC / f"{name}.cpp"), "-o", str(exe),
               f"-L{LIB_DIR}", "-laccelgcn", "-Wl,-rpath,$ORIGIN/../lib"]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {name}.cpp:\n" + r.stdout)
    # a driver written the way upstream's main.cu is, against include/ alone (run by the tests)
    caller = ROOT / "tests" / "cases" / "upstream_shaped_caller.cpp"
    if caller.exists():
        cmd = [hipcc(), "-x", "hip", f"--offload-arch={ARCH}", "-O2", "-std=c++17", "-Wno-unused-value",
               f"-I{ROOT / 'include'}", str(caller), "-o", str(BIN_DIR / "upstream_shaped_caller"),
               f"-L{LIB_DIR}", "-laccelgcn", "-Wl,-rpath,$ORIGIN/../lib"]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for upstream_shaped_caller.cpp:\n" + r.stdout)
    return BIN_DIR / "spmm_test"


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
