"""Build libmongoose_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m mongoose_amd.build

The library is written next to this file so that it travels with the tree.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmongoose_hip.so")

SOURCES = ["kernels.hip", "flow.hip", "prefill.hip", "q4_dp4a.hip", "abi.hip", "fused_infer.hip", "stream_infer.hip", "host_quant.cpp"]

# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 from float code on this target.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
                "-D__HIP_PLATFORM_AMD__"]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build(verbose=True):
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            continue
        obj = os.path.join(objdir, src.rsplit(".", 1)[0] + ".o")
        cmd = [hipcc()] + COMMON_FLAGS + DEVICE_FLAGS + ["-c", path, "-o", obj]
        if src.endswith(".cpp"):
            cmd = [hipcc()] + COMMON_FLAGS + ["-x", "hip"] + DEVICE_FLAGS + ["-c", path, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l or "error" in l]
        if lines and verbose:
            print("\n".join(lines), flush=True)
        if p.returncode != 0:
            failed = True
            print(f"FAILED: {src}", file=sys.stderr)
    if failed:
        raise RuntimeError("hipcc compile failed")
    link = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs + ["-lpthread"]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.check_call(link)
    return LIB


if __name__ == "__main__":
    build()
