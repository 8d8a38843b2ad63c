"""Builds libvsparse.so (the C-ABI HIP library) in-tree with hipcc for gfx950.

    python -m vectorsparse_amd.build
"""
import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libvsparse.so")
OBJ_DIR = os.path.join(_HERE, "build")
SOURCES = ["vsparse_api.hip", "spmm_mfma.hip", "spmm_mfma_flat.hip", "spmm_mfma_slab.hip", "spmm_valu.hip", "sddmm_mfma.hip", "sddmm_valu.hip",
           "sparse_softmax.hip", "sparse_attention.hip",
           "sparse_attention_union.hip"]
# VS_RETIRED_VARIANTS=1 in the environment also compiles the two SpMM variants that measured slower on every shape
# and are therefore not part of the default library: the LDS-DMA gather (spmm_mfma_dma.hip, option spmm_gather = 2)
# and four 32-vector steps in flight (option spmm_steps = 4)
RETIRED = os.environ.get("VS_RETIRED_VARIANTS") == "1"
if RETIRED:
    SOURCES.append("spmm_mfma_dma.hip")
PROBE_PATH = os.path.join(_HERE, "libvsprobe.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    # only the C ABI of include/vsparse.h leaves the library (csrc/vsparse_api.hip exports it explicitly)
    "-fvisibility=hidden",
    # the device code objects are stored compressed (the HIP runtime unpacks them when the library is loaded)
    "--offload-compress",
    # packed-fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first sixteen dwords of kernel arguments arrive in registers with the wave instead of through a load
    # (0.04-0.09 us per launch on the latency-bound SpMM shapes)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature and says so; that is harmless
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in proc.stdout.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)


def _stale(src, obj):
    if not os.path.exists(obj):
        return True
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    newest = max(os.path.getmtime(p) for p in [src, os.path.join(os.path.dirname(_HERE), "include", "vsparse.h")] + headers)
    return os.path.getmtime(obj) < newest


def build(verbose=False, jobs=None, incremental=False):
    """Compile every source to an object (in parallel: the translation units are independent) and link.
    incremental: recompile only the sources that are newer than their objects (or whose shared headers are)."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(OBJ_DIR, exist_ok=True)
    compile_flags = [f for f in FLAGS if f != "-shared"] + (["-DVS_RETIRED_VARIANTS"] if RETIRED else [])
    objects = [os.path.join(OBJ_DIR, s.replace(".hip", ".o")) for s in SOURCES]
    cmds = [[HIPCC] + compile_flags + ["-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(SOURCES, objects)
            if not incremental or _stale(os.path.join(CSRC, s), o)]
    jobs = jobs or max(1, min(len(cmds), os.cpu_count() or 1, 16))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    _run([HIPCC, "--offload-arch=gfx950", "-fPIC", "-shared", "-Wl,--version-script=" + os.path.join(CSRC, "exports.map"),
          "-o", LIB_PATH] + objects, verbose)
    return LIB_PATH


def build_probe(verbose=False):
    """Compile csrc/launch_probe.hip (an empty kernel on a grid of the caller's choice) to libvsprobe.so, the
    measurement aid bench.py prices the dispatch floor with; not part of libvsparse.so."""
    _run([HIPCC, "-O2", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
          os.path.join(CSRC, "launch_probe.hip"), "-o", PROBE_PATH], verbose)
    return PROBE_PATH


def build_cxx_caller(verbose=False):
    """Compile tests/cxx/reference_call_sites.cpp (a C++ program that calls the operators the way the
    reference's benchmarks do, through include/vsparse_shim.hpp) and link it with libvsparse.so."""
    root = os.path.dirname(_HERE)
    src = os.path.join(root, "tests", "cxx", "reference_call_sites.cpp")
    exe = os.path.join(root, "tests", "cxx", "reference_call_sites")
    cmd = [HIPCC, "-O2", "--offload-arch=gfx950", "-std=c++17", "-I", os.path.join(root, "include"), src,
           "-L", _HERE, "-lvsparse", "-Wl,-rpath,$ORIGIN/../../vectorsparse_amd", "-o", exe]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout)
    return exe


if __name__ == "__main__":
    print(build(verbose=True, incremental="--incremental" in sys.argv))
    print(build_probe(verbose=True))
    print(build_cxx_caller(verbose=True))
    sys.exit(0)
