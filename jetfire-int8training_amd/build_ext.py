"""Builds the native parts in-tree (no JIT cache, so the artefacts travel with the source tree):

  libjetfire_hip.so        hipcc, gfx950 only: the HIP kernels behind the C ABI of include/jetfire_hip.h
  libjetfire_prof.so       hipcc, gfx950 only: measurement aids (include/jetfire_prof.h): the phase-recording build of
                           the GEMM kernel (the same source, -DJF_PROF_LIB) and register-only calibration loops;
                           used by the benchmark, not by the operators
  BlockQuantizeCUDA*.so    host C++ (g++): the PyTorch extension with the reference's module name and
                           function signatures (JetfireGEMMKernel/setup.py:13, bindings.cpp:6-35), plus the
                           submodule BlockQuantizeCUDA.jetfire with every other operator of the path; it is
                           compiled as plain C++ (no device code, nothing for hipify to rewrite) and
                           calls the HIP side only through the C ABI.

Usage:  python build_ext.py [hip] [torch]      (default: both)
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HIP_LIB = os.path.join(HERE, "libjetfire_hip.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIP_SOURCES = ["jf_gemm.hip", "jf_blockops.hip"]
PROF_LIB = os.path.join(HERE, "libjetfire_prof.so")
PROF_SOURCES = [("jf_gemm.hip", ["-DJF_PROF_LIB"], "jf_gemm_prof.o"), ("jf_calib.hip", [], "jf_calib.o")]
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",                                         # roundings are exactly the ones written
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",  # no packed-fp32 VALU forms
    "-Wall", "-Wno-unused-function",
]


def torch_ext_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(HERE, "BlockQuantizeCUDA" + suffix)


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_hip():
    """One hipcc process per source file, side by side (the GEMM file alone takes a minute), then one link."""
    flags = [f for f in HIP_FLAGS if f != "-shared"]
    if os.environ.get("JF_PHILOX_ROUNDS"):                       # 7 (default) to 10 rounds of the rounding-noise generator
        flags.append("-DJF_PHILOX_ROUNDS=%d" % int(os.environ["JF_PHILOX_ROUNDS"]))
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    jobs, prof_jobs = [], []
    for src in HIP_SOURCES:
        obj = os.path.join(objdir, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc] + flags + ["-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        jobs.append((cmd, obj, subprocess.Popen(cmd)))
    for src, extra, name in PROF_SOURCES:
        obj = os.path.join(objdir, name)
        cmd = [hipcc] + flags + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        prof_jobs.append((cmd, obj, subprocess.Popen(cmd)))
    for cmd, obj, proc in jobs + prof_jobs:
        if proc.wait() != 0:
            raise subprocess.CalledProcessError(proc.returncode, cmd)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB] + [obj for _, obj, _ in jobs])
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROF_LIB] + [obj for _, obj, _ in prof_jobs])
    return HIP_LIB


TORCH_SOURCES = ["bqc_ext.cpp", "jf_ops_ext.cpp"]


def build_torch():
    import torch
    from torch.utils import cpp_extension as ce

    out = torch_ext_path()
    inc = []
    for p in ce.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", os.path.join(ROCM, "include"), "-I", sysconfig.get_paths()["include"]]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cflags = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-variable",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=BlockQuantizeCUDA",
        "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
    ] + inc
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    jobs = []
    for src in TORCH_SOURCES:                                    # side by side: each takes most of a minute in the torch headers
        obj = os.path.join(objdir, os.path.splitext(src)[0] + ".o")
        cmd = cflags + ["-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        jobs.append((cmd, obj, subprocess.Popen(cmd)))
    for cmd, obj, proc in jobs:
        if proc.wait() != 0:
            raise subprocess.CalledProcessError(proc.returncode, cmd)
    _run(["g++", "-shared", "-o", out] + [obj for _, obj, _ in jobs] + [
        "-L" + torch_lib, "-L" + HERE, "-L" + os.path.join(ROCM, "lib"),
        "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip", "-ltorch_python", "-ljetfire_hip", "-lamdhip64",
        "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib, "-Wl,-rpath," + os.path.join(ROCM, "lib"),
    ])
    return out


def main(argv):
    what = argv or ["hip", "torch"]
    if "hip" in what:
        build_hip()
    if "torch" in what:
        build_torch()


if __name__ == "__main__":
    main(sys.argv[1:])
