"""Builds the two in-tree shared objects of this package for gfx950.

    libot_transducer.so        HIP kernels + C ABI (include/ot_transducer.h), no torch
    _optimized_transducer.so   torch extension (argument checks, allocation, stream)

``python -m optimized_transducer_amd.build`` compiles both with hipcc / g++.
hipcc cross-compiles, so no GPU is needed to build.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
KERNEL_LIB = os.path.join(HERE, "libot_transducer.so")
EXT_LIB = os.path.join(HERE, "_optimized_transducer.so")

# -packed-fp32-ops off: scalar float code must not be fused into v_pk_*_f32.
# No fast-math, no FP contraction: the float expressions keep their written order.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=off", "-fno-fast-math", "-Wall",
]
KERNEL_SOURCES = ("ot_kernels.hip", "ot_joiner.hip", "ot_half.hip", "ot_project.hip",
                  "ot_project_grad.hip")
OBJ_DIR = os.path.join(HERE, "build")  # objects only; ignored by git


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(x) <= t for x in sources)


def build_kernels(incremental=False):
    """One object per source file, compiled side by side, then one shared library.
    incremental: keep the objects whose source and headers have not changed since."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE) if f.endswith(".h")]
    jobs = []
    for f in KERNEL_SOURCES:
        src, obj = os.path.join(CSRC, f), os.path.join(OBJ_DIR, f + ".o")
        if not (incremental and _newer(obj, [src] + headers)):
            jobs.append([hipcc] + HIPCC_FLAGS + ["-I", INCLUDE, "-I", CSRC, "-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=4) as pool:
        list(pool.map(_run, jobs))
    objs = [os.path.join(OBJ_DIR, f + ".o") for f in KERNEL_SOURCES]
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", KERNEL_LIB])
    return KERNEL_LIB


def build_extension():
    import pybind11
    import torch
    tdir = os.path.dirname(torch.__file__)
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
        "-DTORCH_EXTENSION_NAME=_optimized_transducer",
        '-DOT_BUILT_WITH_TORCH="%s"' % torch.__version__,
        "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi,
        "-I", INCLUDE,
        "-I", os.path.join(tdir, "include"),
        "-I", os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
        "-I", sysconfig.get_paths()["include"],
        "-I", pybind11.get_include(),
        "-I", os.path.join(ROCM, "include"),
        os.path.join(CSRC, "binding.cpp"), "-o", EXT_LIB,
        "-L", HERE, "-l:libot_transducer.so",
        "-L", os.path.join(tdir, "lib"),
        "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-ltorch_python",
        "-L", os.path.join(ROCM, "lib"), "-lamdhip64",
        "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(tdir, "lib"),
        "-Wl,-rpath," + os.path.join(ROCM, "lib"),
    ]
    _run(cmd)
    return EXT_LIB


def build_all(incremental=False):
    build_kernels(incremental)
    if not (incremental and _newer(EXT_LIB, [os.path.join(CSRC, "binding.cpp"),
                                            os.path.join(INCLUDE, "ot_transducer.h")])):
        build_extension()


if __name__ == "__main__":
    build_all(incremental="--incremental" in sys.argv[1:])
    sys.exit(0)
