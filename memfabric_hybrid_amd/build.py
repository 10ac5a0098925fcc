"""Builds libzbal.so (HIP kernels for gfx950 + the C++ host layer) in-tree.

    python -m memfabric_hybrid_amd.build            # incremental
    python -m memfabric_hybrid_amd.build --force    # recompile everything

hipcc cross-compiles for gfx950 without a GPU present. Device code is built
with -ffp-contract=off (products and sums round separately unless written as
fmaf) and with packed fp32 instructions disabled.
"""
import concurrent.futures
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(CSRC, "_obj")
LIB_DIR = os.path.join(PKG, "lib")
LIB = os.path.join(LIB_DIR, "libzbal.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

KERNELS = ["layout", "dispatch", "combine", "reduce", "prepack", "gemm"]
HOST = ["zbal_runtime", "zbal_registry", "zbal_gpu_communicator", "zbal_c_api", "zbal_amd_operators"]

HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__"]
INCLUDES = ["-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(CSRC, "kernels"), "-I" + os.path.join(CSRC, "host"),
            "-I" + os.path.join(ROCM, "include")]


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def _headers():
    hs = []
    for d in (os.path.join(ROOT, "include"), os.path.join(CSRC, "kernels"), os.path.join(CSRC, "host")):
        hs += [os.path.join(d, f) for f in os.listdir(d) if f.endswith(".h")]
    return hs


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), r.stdout))
    return r.stdout


def build_library(force=False, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    hdrs = _headers()
    jobs = []
    objs = []
    for k in KERNELS:
        src = os.path.join(CSRC, "kernels", k + ".hip")
        obj = os.path.join(OBJ, k + ".o")
        objs.append(obj)
        if force or not _newer(obj, [src] + hdrs):
            jobs.append([os.path.join(ROCM, "bin", "hipcc")] + HIP_FLAGS + INCLUDES + ["-c", src, "-o", obj])
    for h in HOST:
        src = os.path.join(CSRC, "host", h + ".cpp")
        obj = os.path.join(OBJ, h + ".o")
        objs.append(obj)
        if force or not _newer(obj, [src] + hdrs):
            jobs.append(["g++"] + HOST_FLAGS + INCLUDES + ["-c", src, "-o", obj])
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for out in ex.map(_run, jobs):
            if verbose and out.strip():
                print(out)
    if jobs or force or not os.path.exists(LIB):
        _run([os.path.join(ROCM, "bin", "hipcc"), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs +
             ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    return LIB


def build_asan_library():
    """The C++ host layer under AddressSanitizer and UndefinedBehaviorSanitizer (as the reference builds its unit
    tests, CMakeLists.txt:73-80), linked with the library's ordinary kernel objects, into lib/libzbal_asan.so. For the
    host-side tests on a machine without a GPU (the kernels are never launched there):

        make -C oracle asan && python -m memfabric_hybrid_amd.build --asan
        LD_PRELOAD=$(gcc -print-file-name=libasan.so) ASAN_OPTIONS=detect_leaks=0 \
            ZBAL_LIB=memfabric_hybrid_amd/lib/libzbal_asan.so ZBAL_ORACLE_LIB=oracle/_build/libzbal_oracle_asan.so \
            python -m pytest tests/test_capi_host.py tests/test_oracle_pins.py -q
    """
    build_library()
    san = ["-fsanitize=address,undefined", "-fno-omit-frame-pointer", "-fno-sanitize-recover=undefined", "-g", "-O1"]
    objs = [os.path.join(OBJ, k + ".o") for k in KERNELS]
    for h in HOST:
        obj = os.path.join(OBJ, h + ".asan.o")
        _run(["g++"] + [f for f in HOST_FLAGS if f != "-O2"] + san + INCLUDES + ["-c", os.path.join(CSRC, "host", h + ".cpp"), "-o", obj])
        objs.append(obj)
    out = os.path.join(LIB_DIR, "libzbal_asan.so")
    _run(["g++", "-shared", "-fPIC"] + san + ["-o", out] + objs + ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-lpthread",
                                                                     "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    return out


if __name__ == "__main__":
    if "--asan" in sys.argv:
        print(build_asan_library())
    else:
        print(build_library(force="--force" in sys.argv, verbose=True))
