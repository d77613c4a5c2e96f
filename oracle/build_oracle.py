"""Build recipe for the CPU oracle (test infrastructure, never the product).

  python oracle/build_oracle.py          # libkvc_oracle.so, and oracle/_ref/ when the reference is mounted

* oracle/libkvc_oracle.so  <- oracle/kvc_oracle.c   (gcc, plain C, optional OpenMP)
* oracle/_ref/libkvc_ref.so <- the reference's own src/huffman.cpp + src/compute.cpp compiled where they
  lie in the reference checkout (never copied), plus oracle/ref_shim.cpp.  Needs only g++ and the
  libtorch that ships with the installed PyTorch.  Skipped when the checkout is absent (GPU box).
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REF = os.environ.get("KVCOMP_REFERENCE", "/root/reference")


def build_oracle(verbose=True):
    out = os.path.join(HERE, "libkvc_oracle.so")
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp", "-ffp-contract=off",
           "-o", out, os.path.join(HERE, "kvc_oracle.c"), "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


def build_ref(verbose=True):
    ext = os.path.join(REF, "kvcomp_cuda_extension")
    srcs = [os.path.join(ext, "src", "huffman.cpp"), os.path.join(ext, "src", "compute.cpp")]
    if not all(os.path.exists(s) for s in srcs):
        if verbose:
            print("reference checkout not present: oracle/_ref not built", flush=True)
        return None
    import torch
    from torch.utils.cpp_extension import include_paths
    os.makedirs(os.path.join(HERE, "_ref"), exist_ok=True)
    out = os.path.join(HERE, "_ref", "libkvc_ref.so")
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O1", "-std=c++17", "-fPIC", "-shared", "-w",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(ext, "include")]
    cmd += ["-I" + p for p in include_paths()]
    cmd += ["-o", out, os.path.join(HERE, "ref_shim.cpp")] + srcs
    cmd += ["-L" + libdir, "-Wl,-rpath," + libdir, "-ltorch", "-ltorch_cpu", "-lc10"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


if __name__ == "__main__":
    build_oracle()
    if "--no-ref" not in sys.argv:
        build_ref()
