"""Build recipe for the HIP library (gfx950 only).

    python ornith-rs_amd/build.py          # compile csrc/*.hip, *.cpp -> libornith_hip.so

hipcc cross-compiles without a GPU. Every translation unit is compiled with
-ffp-contract=off (the only fused multiply-adds are the explicit ones, so results
do not depend on what the optimiser chooses to contract), with packed-fp32
instruction selection disabled, and with kernel-argument preloading on.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libornith_hip.so")

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fno-fast-math", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first 14 dwords of a kernel's flat (non-struct) arguments arrive in scalar registers
    # with the wavefront instead of through a scalar load (gfx950 kernel-argument preloading)
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument", "-Wno-pass-failed",
]


# extra compiler flags for one-off builds (e.g. -DORN_TIMING: per-workgroup time stamps)
FLAGS += os.environ.get("ORN_EXTRA_FLAGS", "").split()


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def _compile(src):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the packed-fp32 feature and says so; drop that line
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    return src, obj, r.returncode, err


def build(verbose=True, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, obj, rc, err in ex.map(_compile, sources()):
            if verbose and err.strip():
                print(f"[{src}]\n{err}", file=sys.stderr)
            if rc != 0:
                raise RuntimeError(f"hipcc failed on {src}")
            objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        print(r.stderr, file=sys.stderr)
        raise RuntimeError("link failed")
    return LIB


if __name__ == "__main__":
    print(build())
