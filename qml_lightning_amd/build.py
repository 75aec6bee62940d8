"""Build, in-tree: libqmll.so (the C-ABI HIP library, hipcc for gfx950) and
libqmll_torch.so (the TORCH_LIBRARY operator registrations over that C ABI, host C++ only).

    python -m qml_lightning_amd.build        # or: from qml_lightning_amd.build import build; build()
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libqmll.so")
TORCH_LIB = os.path.join(HERE, "libqmll_torch.so")
SOURCES = ["qmll_core.cpp", "neighbours.hip", "fchl19.hip", "sorf.hip", "project.hip", "rff.hip", "gram.hip", "solve.hip", "probe.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-value"]


def build(verbose=True, jobs=8):
    """Compile every source to an object (in parallel) and link libqmll.so."""
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        cmd = [HIPCC] + FLAGS + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    build_torch_ops(verbose)
    build_host_check(verbose)
    return LIB


def build_torch_ops(verbose=True):
    """Compile csrc/torch_ops.cpp against the installed libtorch and link it to libqmll.so
    (found next to it at run time through an $ORIGIN run path)."""
    import torch
    tdir = os.path.dirname(torch.__file__)
    abi = int(torch.compiled_with_cxx11_abi())
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1",
           "-DUSE_ROCM=1", "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi,
           "-I" + os.path.join(tdir, "include"), "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           "-I/opt/rocm/include", os.path.join(CSRC, "torch_ops.cpp"), "-o", TORCH_LIB,
           "-L" + os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
           "-L" + HERE, "-lqmll", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return TORCH_LIB


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            sys.stderr.write(out + "\n")
            raise RuntimeError("hipcc failed on %s" % src)
        if out.strip():
            print(out)




def build_host_check(verbose=True):
    """tests/cpp/run_scripted: a C++ program (libtorch only, no Python) that loads a saved model
    through libqmll_torch.so; the GPU tests run it as a child process."""
    import torch
    tdir = os.path.dirname(torch.__file__)
    src = os.path.join(os.path.dirname(HERE), "tests", "cpp", "run_scripted.cpp")
    if not os.path.exists(src):
        return None
    out = os.path.splitext(src)[0]
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O1", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch.compiled_with_cxx11_abi()),
           "-I" + os.path.join(tdir, "include"), "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           src, "-o", out, "-L" + os.path.join(tdir, "lib"), "-Wl,--no-as-needed", "-ltorch", "-ltorch_cpu", "-lc10",
           "-ltorch_hip", "-lc10_hip", "-ldl", "-Wl,-rpath," + os.path.join(tdir, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


if __name__ == "__main__":
    build()
