"""Build libkvcomp_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m kvcomp_amd.build            # compile every csrc/*.hip, link kvcomp_amd/lib/libkvcomp_hip.so,
                                          # then the compiled `kvcomp_cuda` module over it (kvcomp_amd/ext/)

Objects are compiled in parallel (one hipcc process per source file) and linked into one shared
library that exports the C ABI declared in include/kvcomp_hip.h.  The Python extension module
(csrc/kvcomp_cuda_module.cpp, host C++ only) is compiled with g++ against the installed libtorch and
linked to that library.
"""
import json
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBPATH = os.path.join(LIBDIR, "libkvcomp_hip.so")
EXTDIR = os.path.join(HERE, "ext")
MODULE_SRC = os.path.join(CSRC, "kvcomp_cuda_module.cpp")
MODULE_PATH = os.path.join(EXTDIR, "kvcomp_cuda.so")         # `import kvcomp_cuda` with EXTDIR on sys.path
ARCH = "gfx950"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++20", "-fPIC", "--offload-arch=" + ARCH,
    # packed-fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
    # the code generator's own account of every kernel (registers, spills, scratch, LDS), kept beside the objects
    "-Rpass-analysis=kernel-resource-usage",
]
RESOURCES = os.path.join(HERE, "build", "kernel_resources.json")
_REMARK = re.compile(r"remark:\s+([A-Za-z][A-Za-z /\[\]]*?):\s+(\S+) \[-Rpass-analysis=kernel-resource-usage\]")


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src, objdir, verbose):
    obj = os.path.join(objdir, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    kernels, name, keep, skip = {}, None, [], 0
    for line in r.stdout.splitlines():
        if "packed-fp32-ops" in line:                   # the host pass does not know the device feature: harmless
            continue
        m = _REMARK.search(line)
        if m:
            skip = 2                                    # the remark's two lines of source context
            if m.group(1) == "Function Name":
                name = m.group(2)
                kernels[name] = {}
            elif name is not None:
                v = m.group(2)
                kernels[name][m.group(1).strip()] = int(v) if v.isdigit() else v
        elif skip:
            skip -= 1
        else:
            keep.append(line)
    out = "\n".join(keep)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    if verbose and out.strip():
        print(out, flush=True)
    return obj, kernels


def build(verbose=True, jobs=None):
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, (os.cpu_count() or 2) - 1), 8)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        done = list(pool.map(lambda s: _compile(s, objdir, verbose), srcs))
    objs = [o for o, _ in done]
    with open(RESOURCES, "w") as f:
        json.dump({os.path.basename(s): k for s, (_, k) in zip(srcs, done)}, f, indent=1, sort_keys=True)
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o", LIBPATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIBPATH


def build_module(verbose=True):
    """The reference's `kvcomp_cuda` extension module (kvcomp_cuda_extension/export_kvcomp.cpp:8-26) over the C ABI."""
    import sysconfig
    import torch
    from torch.utils.cpp_extension import include_paths
    os.makedirs(EXTDIR, exist_ok=True)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(os.path.dirname(HERE), "include"), "-I" + os.path.join(rocm, "include"),
           "-I" + sysconfig.get_paths()["include"]]
    cmd += ["-I" + p for p in include_paths()]
    cmd += ["-o", MODULE_PATH, MODULE_SRC, "-L" + LIBDIR, "-lkvcomp_hip", "-Wl,-rpath,$ORIGIN/../lib",
            "-L" + torch_lib, "-Wl,-rpath," + torch_lib, "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_python"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return MODULE_PATH


if __name__ == "__main__":
    build(verbose="-q" not in sys.argv)
    print("built", LIBPATH)
    build_module(verbose="-q" not in sys.argv)
    print("built", MODULE_PATH)
