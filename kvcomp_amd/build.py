"""Build libkvcomp_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m kvcomp_amd.build            # compile every csrc/*.hip, link kvcomp_amd/lib/libkvcomp_hip.so

Objects are compiled in parallel (one hipcc process per source file) and linked into one shared
library that exports the C ABI declared in include/kvcomp_hip.h.
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


if __name__ == "__main__":
    build(verbose="-q" not in sys.argv)
    print("built", LIBPATH)
