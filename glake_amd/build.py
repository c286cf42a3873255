"""Compile the HIP sources of the vtkv library for gfx950 into ``glake_amd/lib/libvtkv.so``.

Usage: ``python -m glake_amd.build`` (hipcc cross-compiles, no GPU needed).
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libvtkv.so")
SOURCES = ["vtkv_vmm.cpp", "vtkv_cache.hip", "vtkv_attention.hip", "vtkv_attention_f32.hip", "vtkv_prefill.hip"]

# Packed-FP32 instruction selection is switched off for all device code of this library.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # keep MFMA accumulators in ordinary VGPRs: the softmax rescale multiplies them on the VALU and
    # the AGPR form would copy all of them back and forth every tile
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    # only the C ABI of include/vtkv.h (declared with default visibility there) leaves the shared object
    "-fvisibility=hidden", "-fvisibility-inlines-hidden",
    "-Wall", "-Wno-unused-function",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the vtkv library cannot be built")
    return exe


def build_library(verbose: bool = False, out_path: str = LIB_PATH, extra_flags=()) -> str:
    os.makedirs(os.path.dirname(out_path), exist_ok=True)
    obj_dir = os.path.join(_HERE, "build", os.path.basename(out_path) + ".o")
    os.makedirs(obj_dir, exist_ok=True)
    hipcc = _hipcc()

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc, *HIP_FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        res = subprocess.run(cmd, capture_output=True, text=True)
        # the host pass does not know the device-only feature flag and says so: not an error
        err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    tmp = out_path + ".tmp"
    res = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs, "-lpthread",
                          "-Wl,--version-script=" + os.path.join(CSRC, "vtkv.map")],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("linking libvtkv.so failed:\n" + res.stderr)
    os.replace(tmp, out_path)
    return out_path


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser(description="compile libvtkv.so for gfx950")
    ap.add_argument("--define", action="append", default=[], metavar="NAME[=VALUE]",
                    help="a tuning build: -DNAME[=VALUE] for every source (e.g. VTKV_ATTN_TRACE: the decode kernel "
                         "records when each of its workgroups starts and ends, for bench.py --workgroup-trace)")
    ap.add_argument("--out", default=LIB_PATH, help="where the shared object goes (VTKV_LIBRARY_PATH selects it at run time)")
    cli = ap.parse_args()
    print(build_library(verbose=True, out_path=os.path.abspath(cli.out), extra_flags=["-D" + d for d in cli.define]))
