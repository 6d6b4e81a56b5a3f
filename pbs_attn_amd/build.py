"""Builds libpbs_hip.so (the gfx950 kernels + C ABI) in-tree with hipcc."""
from __future__ import annotations

import os
import shutil
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libpbs_hip.so")

SOURCES = ["pbs_abi.hip", "pbs_score.hip", "pbs_sort.hip", "pbs_gather.hip", "pbs_estimate.hip",
           "pbs_select.hip", "pbs_attn.hip", "pbs_pipeline.hip", "pbs_rope.hip"]
# measurement kernels for bench.py, in a library of their own: not part of the operator's ABI
PROBE_SOURCES = ["pbs_probe.hip"]
PROBE_LIB_PATH = os.path.join(LIB_DIR, "libpbs_probe.so")

DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unused-command-line-argument", "-Wno-unused-value"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the PBS HIP kernels cannot be built")
    return exe


def build_library(verbose: bool = False) -> str:
    """Compiles every .hip source for gfx950 and links the shared library."""
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = _hipcc()
    with tempfile.TemporaryDirectory() as tmp:
        objs = []
        procs = []
        for src in SOURCES + PROBE_SOURCES:
            obj = os.path.join(tmp, src.replace(".hip", ".o"))
            cmd = [hipcc, *DEVICE_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
            procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)))
            objs.append(obj)
        for src, p in procs:
            out, err = p.communicate()
            if p.returncode != 0:
                raise RuntimeError(f"hipcc failed on {src}:\n{err}")
            if verbose and err.strip():
                print(err)
        probe_objs = objs[len(SOURCES):]
        tmp_lib = os.path.join(tmp, "libpbs_hip.so")
        subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-o", tmp_lib, *objs[:len(SOURCES)]], check=True)
        shutil.move(tmp_lib, LIB_PATH)
        tmp_probe = os.path.join(tmp, "libpbs_probe.so")
        subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-o", tmp_probe, *probe_objs, "-L" + LIB_DIR, "-lpbs_hip",
                        "-Wl,-rpath,$ORIGIN"], check=True)
        shutil.move(tmp_probe, PROBE_LIB_PATH)
    return LIB_PATH


C_SMOKE_SRC = os.path.join(os.path.dirname(HERE), "tests", "c_abi", "smoke.c")
C_SMOKE_BIN = os.path.join(os.path.dirname(HERE), "tests", "c_abi", "smoke")


def build_c_smoke() -> str:
    """Compiles tests/c_abi/smoke.c with gcc as plain C99 against include/pbs_hip.h and links it to the
    library and the HIP runtime: the check that the C ABI is usable without Python or torch."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["gcc", "-std=c99", "-O2", C_SMOKE_SRC, "-I" + os.path.join(os.path.dirname(HERE), "include"),
           "-I" + os.path.join(rocm, "include"), "-D__HIP_PLATFORM_AMD__", "-o", C_SMOKE_BIN, "-L" + LIB_DIR, "-lpbs_hip",
           "-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-lm", "-Wl,-rpath,$ORIGIN/../../pbs_attn_amd/lib",
           "-Wl,-rpath," + os.path.join(rocm, "lib")]
    subprocess.run(cmd, check=True)
    return C_SMOKE_BIN


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_c_smoke())
