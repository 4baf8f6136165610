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

# (source, object name, extra defines). box_sampling_inst.hip holds the explicit instantiations of
# the backward kernels and is compiled once per element-type pair and part, so that they build in
# parallel (one translation unit with all of them takes six minutes).
def _inst(tag, t, tg, part, same):
    defs = ["-DBOXCONV_INST_T=" + t, "-DBOXCONV_INST_TG=" + tg, "-DBOXCONV_INST_PART=%d" % part]
    if same:
        defs.append("-DBOXCONV_INST_SAME_TYPE=1")
    return ("box_sampling_inst.hip", "box_sampling_inst_%s_%d.o" % (tag, part), defs)


SOURCES = [(s, s.replace(".hip", ".o"), []) for s in
           ("box_sampling.hip", "box_forward.hip", "integral_image.hip", "integral_image_int.hip", "box_misc.hip",
            "boxconv_c_abi.hip")]
for _tag, _t, _tg in (("f32", "float", "float"), ("f64", "double", "double"),
                      ("f16", "float", "f16_t"), ("bf16", "float", "bf16_t")):
    for _part in (1, 2) + ((3, 4) if _t == "float" else ()):
        SOURCES.append(_inst(_tag, _t, _tg, _part, _t == _tg))
HEADERS = ["boxconv_device.hpp", "boxconv_host.hpp", "box_sampling_common.hpp", "box_sampling_impl.hpp",
           os.path.join("..", "..", "include", "boxconv.h")]

ARCH = "gfx950"      # the only target: the kernels assume its 160 KiB of LDS per workgroup and its ISA
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


GLUE_SRC = os.path.join(CSRC, "torch_glue.cpp")
GLUE_PATH = os.path.join(HERE, "box_convolution", "_boxconv_glue.so")


def build_glue(force=False, verbose=True):
    """The C++ autograd node of the training step (csrc/torch_glue.cpp): a Python extension module
    compiled with g++ against the installed torch's headers. It holds no kernels and does not link
    to libboxconv_hip.so (it is handed that library's entry points as addresses at start-up)."""
    if not (force or _stale(GLUE_PATH, [GLUE_SRC, os.path.abspath(__file__)])):
        return GLUE_PATH
    import sysconfig
    import torch
    from torch.utils import cpp_extension
    cxx = shutil.which("g++") or "g++"
    tdir = os.path.dirname(torch.__file__)
    cmd = [cxx, "-O2", "-fPIC", "-std=c++17", "-shared", "-w",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-DTORCH_EXTENSION_NAME=_boxconv_glue", "-DTORCH_API_INCLUDE_EXTENSION_H"]
    cmd += ["-I" + d for d in cpp_extension.include_paths()]
    cmd += ["-I" + sysconfig.get_paths()["include"], GLUE_SRC, "-o", GLUE_PATH,
            "-L" + os.path.join(tdir, "lib"), "-lc10", "-ltorch_cpu", "-ltorch", "-ltorch_python",
            "-Wl,-rpath," + os.path.join(tdir, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return GLUE_PATH


def build(force=False, verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = _hipcc()
    header_paths = [os.path.normpath(os.path.join(CSRC, h)) for h in HEADERS] + [os.path.abspath(__file__)]
    jobs = []
    objs = []
    for src, obj_name, defines in SOURCES:
        src_path = os.path.join(CSRC, src)
        obj = os.path.join(OBJ_DIR, obj_name)
        objs.append(obj)
        if force or _stale(obj, [src_path] + header_paths):
            jobs.append([hipcc] + HIPCC_FLAGS + defines + ["-c", src_path, "-o", obj])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)

    workers = min(os.cpu_count() or 4, 8, max(1, len(jobs)))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        list(pool.map(run, jobs))

    if force or jobs or _stale(LIB_PATH, objs):
        run([hipcc, "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o", LIB_PATH] + objs)
    build_glue(force=force, verbose=verbose)
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    args = ap.parse_args()
    print(build(force=args.force))
    sys.exit(0)
