"""Build recipe for the native libraries of this package.

``libgs_hip.so``  HIP kernels + C ABI (``include/gs_hip.h``); hipcc, gfx950 only,
                  no torch dependency.
``libgs.so``      C++ host layer (``gs::Graph``, ``graph_ops``, TORCH_LIBRARY
                  registration) on top of the C ABI; built by
                  :func:`build_host` when its sources are present.

Both are built in-tree, next to this file.  Run ``python -m graph_sampling_amd.build``.
"""
import glob
import os
import subprocess
import sys

_PKG = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_PKG, "csrc")
_ROOT = os.path.dirname(_PKG)

KERNEL_LIB = os.path.join(_PKG, "libgs_hip.so")
HOST_LIB = os.path.join(_PKG, "libgs.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
HIP_FLAGS = [
    "--offload-arch=" + ARCH,
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def kernel_sources():
    return sorted(glob.glob(os.path.join(_CSRC, "*.hip"))) + [os.path.join(_CSRC, "gs_api.cpp")]


STAMPS_LIB = os.path.join(_PKG, "libgs_hip_stamps.so")


def build_stamps(verbose=False):
    """The measuring build of the kernel library: the same sources with -DGS_PHASE_STAMPS, which
    compiles wall-clock marks into the minibatch kernels (graph_sampling_amd/phase_stamps.py
    reads them).  Never loaded by the package itself."""
    return build_kernels(verbose, extra_flags=("-DGS_PHASE_STAMPS",), out=STAMPS_LIB,
                         objdir=os.path.join(_PKG, "build", "stamps"))


def build_kernels(verbose=False, extra_flags=(), out=None, objdir=None):
    """Compile every HIP translation unit for gfx950 and link libgs_hip.so."""
    out = out or KERNEL_LIB
    objdir = objdir or os.path.join(_PKG, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    procs = []
    for src in kernel_sources():
        obj = os.path.join(objdir, os.path.basename(src) + ".o")
        objs.append(obj)
        cmd = [HIPCC] + HIP_FLAGS + list(extra_flags) + ["-x", "hip", "-c", src, "-o", obj]
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                                            text=True)))
    for cmd, p in procs:
        log, _ = p.communicate()
        log = "\n".join(l for l in log.splitlines()
                        if "is not a recognized feature for this target" not in l)
        if p.returncode != 0:
            raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), log))
        if verbose and log.strip():
            print(log)
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", out] + objs)
    return out


def host_sources():
    return sorted(glob.glob(os.path.join(_CSRC, "host", "*.cc")))


def build_host(verbose=False):
    """Compile the C++ host layer against libtorch and link it to libgs_hip.so."""
    srcs = host_sources()
    if not srcs:
        return None
    import torch
    from torch.utils import cpp_extension as ce
    objdir = os.path.join(_PKG, "build")
    os.makedirs(objdir, exist_ok=True)
    inc = []
    for p in ce.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", "/opt/rocm/include", "-I", os.path.join(_ROOT, "include")]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    flags = ["-O2", "-std=c++17", "-fPIC", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
             "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi, "-Wno-deprecated-declarations"]
    flags += os.environ.get("GS_HOST_CXXFLAGS", "").split()
    objs, procs = [], []
    for src in srcs:
        obj = os.path.join(objdir, "host_" + os.path.basename(src) + ".o")
        objs.append(obj)
        cmd = ["g++"] + flags + inc + ["-c", src, "-o", obj]
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                                            text=True)))
    for cmd, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
        if verbose and out.strip():
            print(out)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    link = ["g++", "-shared", "-o", HOST_LIB] + objs + [
        "-L" + _PKG, "-lgs_hip", "-Wl,-rpath,$ORIGIN",
        "-L" + torch_lib, "-lc10", "-ltorch_cpu", "-ltorch", "-lc10_hip",
        # libtorch_hip registers the GPU backend from its static initialisers; nothing here
        # refers to a symbol of it, so the linker would drop it and a C++ program that loads
        # only this library would find no GPU
        "-Wl,--no-as-needed", "-ltorch_hip", "-Wl,--as-needed",
        "-Wl,-rpath," + torch_lib,
        "-L/opt/rocm/lib", "-lamdhip64", "-lrocprofiler-sdk-roctx", "-Wl,-rpath,/opt/rocm/lib",
    ]
    _run(link)
    return HOST_LIB


CPP_CHECK_SRC = os.path.join(_ROOT, "tests", "cpp", "host_api_check.cc")
CPP_CHECK_BIN = os.path.join(_ROOT, "tests", "cpp", "host_api_check")


def build_cpp_check(verbose=False):
    """Compile the C++ caller of the host layer (tests/cpp) against the public headers and
    link it to libgs.so: proof that gs::Graph and the free functions can be used from C++."""
    if not os.path.exists(CPP_CHECK_SRC):
        return None
    import torch
    from torch.utils import cpp_extension as ce
    inc = []
    for p in ce.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", "/opt/rocm/include", "-I", os.path.join(_CSRC, "host")]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O1", "-std=c++17", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi, "-Wno-deprecated-declarations"] + inc + [
        CPP_CHECK_SRC, "-o", CPP_CHECK_BIN,
        "-L" + _PKG, "-lgs", "-lgs_hip", "-Wl,-rpath,$ORIGIN/../../graph_sampling_amd",
        "-L" + torch_lib, "-lc10", "-ltorch_cpu", "-ltorch", "-lc10_hip", "-ltorch_hip",
        "-Wl,-rpath," + torch_lib,
        "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return CPP_CHECK_BIN


STAMP = os.path.join(_PKG, "libgs.stamp")


def source_hash():
    """sha256 over every source the two libraries are built from (csrc/, include/)."""
    import hashlib
    h = hashlib.sha256()
    files = sorted(glob.glob(os.path.join(_CSRC, "**", "*"), recursive=True) +
                   glob.glob(os.path.join(_ROOT, "include", "*.h")))
    for path in files:
        if os.path.isfile(path):
            h.update(os.path.relpath(path, _ROOT).encode())
            with open(path, "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def built_from_current_sources():
    """Whether both libraries exist and were built from the sources as they are now (the
    build leaves the hash of its sources beside the libraries)."""
    if not (os.path.exists(KERNEL_LIB) and os.path.exists(HOST_LIB) and os.path.exists(STAMP)):
        return False
    with open(STAMP) as f:
        return f.read().strip() == source_hash()


def build_all(verbose=False):
    digest = source_hash()
    libs = [build_kernels(verbose)]
    host = build_host(verbose)
    if host:
        libs.append(host)
        check = build_cpp_check(verbose)
        if check:
            libs.append(check)
    with open(STAMP, "w") as f:
        f.write(digest + "\n")
    return libs


if __name__ == "__main__":
    if "--stamps" in sys.argv:
        print("built", build_stamps(verbose="-v" in sys.argv))
    else:
        for lib in build_all(verbose="-v" in sys.argv):
            print("built", lib)
