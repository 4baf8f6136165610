"""Builds libboxconv_hip.so (the gfx950 kernels behind include/boxconv.h) with hipcc.

    python box-convolutions_amd/build.py            # compile what changed, link
    python box-convolutions_amd/build.py --force    # recompile everything

hipcc cross-compiles for gfx950 without a GPU. The library depends on the HIP runtime only
(libamdhip64), never on torch; inside a Python process that has imported torch first, the runtime
torch already loaded is the one that gets bound (same soname).
"""
import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "box_convolution", "libboxconv_hip.so")

SOURCES = ["box_sampling.hip", "box_forward.hip", "integral_image.hip", "box_misc.hip", "boxconv_c_abi.hip"]
HEADERS = ["boxconv_device.hpp", "boxconv_host.hpp", "box_sampling_common.hpp", os.path.join("..", "..", "include", "boxconv.h")]

ARCH = os.environ.get("BOXCONV_OFFLOAD_ARCH", "gfx950")
# packed-fp32 instructions stay disabled: scalar float code only.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=" + ARCH,
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libboxconv_hip.so cannot be built")
    return exe


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = _hipcc()
    header_paths = [os.path.normpath(os.path.join(CSRC, h)) for h in HEADERS] + [os.path.abspath(__file__)]
    jobs = []
    objs = []
    for src in SOURCES:
        src_path = os.path.join(CSRC, src)
        obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        objs.append(obj)
        if force or _stale(obj, [src_path] + header_paths):
            jobs.append([hipcc] + HIPCC_FLAGS + ["-c", src_path, "-o", obj])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)

    with ThreadPoolExecutor(max_workers=min(5, max(1, len(jobs)))) as pool:
        list(pool.map(run, jobs))

    if force or jobs or _stale(LIB_PATH, objs):
        run([hipcc, "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o", LIB_PATH] + objs)
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    args = ap.parse_args()
    print(build(force=args.force))
    sys.exit(0)
