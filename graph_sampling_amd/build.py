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
    if out == KERNEL_LIB and not extra_flags:
        _stamp("kernels")
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
    _stamp("host")
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


def _hash_of(paths):
    import hashlib
    h = hashlib.sha256()
    for path in sorted(paths):
        if os.path.isfile(path):
            h.update(os.path.relpath(path, _ROOT).encode())
            with open(path, "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def _headers():
    return glob.glob(os.path.join(_ROOT, "include", "*.h"))


def source_hashes():
    """sha256 over what each library is built from: {"kernels": ..., "host": ...}."""
    kernels = [p for p in glob.glob(os.path.join(_CSRC, "*")) if os.path.isfile(p)]
    host = glob.glob(os.path.join(_CSRC, "host", "*"))
    return {"kernels": _hash_of(kernels + _headers()), "host": _hash_of(host + _headers())}


def source_hash():
    h = source_hashes()
    return h["kernels"][:8] + h["host"][:8]


def _read_stamp():
    try:
        with open(STAMP) as f:
            return dict(line.split() for line in f if len(line.split()) == 2)
    except OSError:
        return None


def _stamp(which):
    """Records that library `which` has just been built from the sources as they are."""
    have = _read_stamp() or {}
    have[which] = source_hashes()[which]
    with open(STAMP, "w") as f:
        for k in sorted(have):
            f.write("%s %s\n" % (k, have[k]))


def build_state():
    """"current": both libraries exist and were built from the sources as they are now (each
    build leaves the hash of its sources beside the libraries); "stale": one was built from
    other sources; "unknown": libraries without hashes beside them; "missing"."""
    if not (os.path.exists(KERNEL_LIB) and os.path.exists(HOST_LIB)):
        return "missing"
    have = _read_stamp()
    if not have:
        return "unknown"
    return "current" if have == source_hashes() else "stale"


def build_all(verbose=False):
    libs = [build_kernels(verbose)]
    host = build_host(verbose)
    if host:
        libs.append(host)
        check = build_cpp_check(verbose)
        if check:
            libs.append(check)
    return libs


if __name__ == "__main__":
    if "--stamps" in sys.argv:
        print("built", build_stamps(verbose="-v" in sys.argv))
    else:
        for lib in build_all(verbose="-v" in sys.argv):
            print("built", lib)
