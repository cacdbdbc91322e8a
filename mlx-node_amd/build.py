"""Compiles the HIP kernels and the C ABI into mlx-node_amd/libmxopt.so for gfx950.

hipcc cross-compiles without a GPU.  Flags that matter for parity with the reference's
float32 op chain: -ffp-contract=off (no fused multiply-add), no fast-math, correctly
rounded float32 divide and square root (hipcc's default).  Packed float32 instructions are
switched off for the device pass.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmxopt.so")

SOURCES = ["mxopt_kernels.hip", "mxopt_reduce_kernels.hip", "mxopt_list_kernels.hip", "mxopt_list_kernels_sgd_rmsprop.hip", "mxopt_hbm_pool.hip",
           "mxopt_api.cpp", "mxopt_region_scan.cpp",
           "mxopt_optimizers.cpp", "mxopt_engine.cpp", "mxopt_checkpoint.cpp"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-fno-fast-math", "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]
OBJ_DIR = os.path.join(HERE, "bin", "obj")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature and says so; that is harmless
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        sys.stderr.write(err + "\n")
        raise RuntimeError("hipcc failed: " + os.path.basename(cmd[-1]))
    if verbose and err.strip():
        print(err)


def _headers_mtime() -> float:
    dirs = [CSRC, os.path.join(ROOT, "include")]
    return max(os.path.getmtime(os.path.join(d, f)) for d in dirs for f in os.listdir(d) if f.endswith(".h"))


def build_variant(out: str, defines, verbose: bool = False) -> str:
    """The library alone, compiled with extra -D definitions into `out` (for A/B measurements of one build
    against another on the same machine); objects go to a directory of their own."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    obj_dir = os.path.join(HERE, "bin", "obj_" + os.path.basename(out))
    os.makedirs(obj_dir, exist_ok=True)
    jobs = []
    for s in SOURCES:
        obj = os.path.join(obj_dir, os.path.splitext(s)[0] + ".o")
        jobs.append(([hipcc] + FLAGS + ["-D" + d for d in defines] + ["-x", "hip", "-c", os.path.join(CSRC, s), "-o", obj], obj))
    with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1, 8)) as pool:
        list(pool.map(lambda j: _run(j[0], verbose), jobs))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + [obj for _, obj in jobs] + ["-o", out], verbose)
    return out


def build(verbose: bool = False, incremental: bool = False) -> str:
    """Every translation unit is compiled by its own hipcc process (they are independent and the three
    kernel files take about as long as each other), then linked.  incremental: a unit whose object file is
    newer than its source and than every header is not compiled again (for edit-compile loops; the default
    compiles everything)."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs, objs = [], []
    newest_header = _headers_mtime() if incremental else 0.0
    for s in SOURCES:
        obj = os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o")
        objs.append(obj)
        src = os.path.join(CSRC, s)
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header):
            continue
        jobs.append(([hipcc] + FLAGS + ["-x", "hip", "-c", src, "-o", obj], obj))
    with ThreadPoolExecutor(max_workers=min(max(len(jobs), 1), os.cpu_count() or 1, 8)) as pool:
        list(pool.map(lambda j: _run(j[0], verbose), jobs))
    jobs = [(None, o) for o in objs]
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + [obj for _, obj in jobs] + ["-o", LIB + ".tmp"], verbose)
    os.replace(LIB + ".tmp", LIB)
    build_demo(verbose)
    build_napi(verbose)
    return LIB


DEMO = os.path.join(HERE, "bin", "cabi_demo")


def build_demo(verbose: bool = False) -> str:
    """examples/cabi_demo.c as plain C11 against the public headers: a host without Python, and the
    proof that the headers are C."""
    os.makedirs(os.path.dirname(DEMO), exist_ok=True)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["gcc", "-std=c11", "-O2", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(rocm, "include"), os.path.join(HERE, "examples", "cabi_demo.c"), "-o", DEMO,
           "-L", HERE, "-lmxopt", "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-lm",
           "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return DEMO


NAPI = os.path.join(HERE, "bin", "mxopt.node")


def build_napi(verbose: bool = False):
    """napi/mxopt_napi.c -> bin/mxopt.node (the JavaScript surface), when node's headers are installed."""
    include = next((d for d in ("/usr/include/node", "/usr/local/include/node") if os.path.exists(os.path.join(d, "node_api.h"))),
                   None)
    if include is None:
        if verbose:
            print("node_api.h not found: the N-API binding is not built")
        return None
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["gcc", "-std=c11", "-O2", "-Wall", "-Werror", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(ROOT, "include"), "-I", os.path.join(rocm, "include"), "-I", include,
           os.path.join(HERE, "napi", "mxopt_napi.c"), "-o", NAPI, "-L", HERE, "-lmxopt",
           "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-lm", "-Wl,-rpath,$ORIGIN/..",
           "-Wl,-rpath," + os.path.join(rocm, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return NAPI


SANITY = os.path.join(HERE, "bin", "host_sanity_asan")


def build_sanitized(verbose: bool = False) -> str:
    """examples/host_sanity.cpp + the whole host layer under AddressSanitizer and UBSan (host code only;
    the device pass is not instrumented).  Not part of the default build: it takes a couple of minutes.
    Run with ASAN_OPTIONS=detect_leaks=0 (the HIP runtime keeps its own allocations)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(os.path.dirname(SANITY), exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in SOURCES] + [os.path.join(HERE, "examples", "host_sanity.cpp")]
    cmd = [hipcc, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-ffp-contract=off",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=undefined",
           "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-x", "hip"] + srcs + ["-o", SANITY]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write("\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l) + "\n")
        raise RuntimeError("sanitized build failed")
    return SANITY


if __name__ == "__main__":
    if "--variant" in sys.argv:   # --variant OUT.so [NAME=VALUE ...]
        i = sys.argv.index("--variant")
        print(build_variant(os.path.abspath(sys.argv[i + 1]), [a for a in sys.argv[i + 2:] if "=" in a]))
    elif "--sanitize" in sys.argv:
        print(build_sanitized(verbose=True))
    else:
        print(build(verbose=True, incremental="--incremental" in sys.argv))
