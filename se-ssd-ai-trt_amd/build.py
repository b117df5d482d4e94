"""Build libsessd3d.so (HIP, gfx950 only) in-tree: se-ssd-ai-trt_amd/lib/libsessd3d.so.

    python se-ssd-ai-trt_amd/build.py            # compile every source and link
    python se-ssd-ai-trt_amd/build.py --if-stale # skip when the library is newer than all sources

hipcc cross-compiles for gfx950 without a GPU.  Packed-FP32 VALU instructions are disabled for all
device code; fast-math is never enabled (voxel coordinates need IEEE FP32 division).
"""
import concurrent.futures as cf
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "lib", "libsessd3d.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-fast-math", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources():
    return sorted(glob.glob(os.path.join(SRC_DIR, "*.hip")))


def headers():
    return (sorted(glob.glob(os.path.join(SRC_DIR, "*.h"))) + [os.path.join(HERE, "..", "include", "sessd3d.h")] +
            [os.path.join(HERE, "examples", "run_frame.c"), os.path.join(HERE, "examples", "gather_order.hip")])


def is_stale():
    if not os.path.exists(LIB) or not os.path.exists(os.path.join(HERE, "lib", "run_frame")) or not os.path.exists(GATHER_ORDER):
        return True
    t = os.path.getmtime(LIB)
    return any(os.path.getmtime(p) > t for p in sources() + headers())


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return src, obj, r.returncode, r.stdout


def build(force=True, jobs=8, verbose=False):
    if not force and not is_stale():
        return LIB
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    objs = []
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, obj, rc, out in ex.map(_compile, sources()):
            # the host pass warns that it does not know the packed-fp32 feature: harmless
            text = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
            if rc != 0:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
            if verbose and text:
                print(text)
            objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    build_example()
    build_gather_order()
    return LIB


EXAMPLE_SRC = os.path.join(HERE, "examples", "run_frame.c")
EXAMPLE = os.path.join(HERE, "lib", "run_frame")


def build_example():
    """The C host of the library (examples/run_frame.c): plain C99 with gcc against include/sessd3d.h and the
    HIP runtime API, linked to the library beside it."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [os.environ.get("CC", "gcc"), "-std=c99", "-O2", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(HERE, "..", "include"), "-I", os.path.join(rocm, "include"), EXAMPLE_SRC, "-o", EXAMPLE,
           "-L", os.path.dirname(LIB), "-lsessd3d", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the C example failed:\n" + r.stdout)
    return EXAMPLE


GATHER_ORDER_SRC = os.path.join(HERE, "examples", "gather_order.hip")
GATHER_ORDER = os.path.join(HERE, "lib", "gather_order")


def build_gather_order():
    """The stand-alone measurement behind the order of conv_wide.hip's row requests (examples/gather_order.hip)."""
    cmd = [HIPCC] + [f for f in FLAGS if f != "-fPIC"] + [GATHER_ORDER_SRC, "-o", GATHER_ORDER]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("building examples/gather_order.hip failed:\n" + r.stdout)
    return GATHER_ORDER


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv, verbose=True))
