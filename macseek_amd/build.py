"""Build libmsq.so (hipcc, gfx950 only) in-tree. `python -m macseek_amd.build` or `build()`."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libmsq.so")
OBJDIR = os.path.join(HERE, "csrc", "build")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-I" + os.path.join(HERE, "..", "include")]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


# Per-file additions. The one-token MoE kernels take the expert address table as their first argument and have it
# delivered in scalar registers with the wave (kernel-argument preload): the table can be read while the rest of the
# arguments is still on its way from memory.
# The token matvec kernel takes what its first loads need (activations, then weight rows) as twelve leading words in the
# same way.
EXTRA = {"msq_moe.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=2"],
         "msq_matvec.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=12"]}


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.basename(src)[:-4] + ".o")
    r = subprocess.run([HIPCC] + FLAGS + EXTRA.get(os.path.basename(src), []) + ["-c", src, "-o", obj],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj


def build(verbose=True):
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs +
                       ["-L/opt/rocm/lib", "-lrocblas", "-Wl,-rpath,/opt/rocm/lib"],  # rocBLAS: the dense fp16 GEMM of msq_matmul for many tokens
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    if verbose:
        print("built", OUT, "from", [os.path.basename(s) for s in srcs])
    return OUT


def build_shim_test(verbose=True):
    """tests/cpp/shim_test: the C++ operator shim exercised like the reference's own test programs."""
    root = os.path.join(HERE, "..")
    src = os.path.join(root, "tests", "cpp", "shim_test.cpp")
    out = os.path.join(root, "tests", "cpp", "shim_test")
    r = subprocess.run([HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++20", "-Wno-unused-command-line-argument",
                        "-I" + os.path.join(root, "include"), src, "-o", out, "-L" + HERE, "-lmsq", "-Wl,-rpath," + os.path.abspath(HERE)],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("shim_test build failed:\n" + r.stdout)
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    build()
    build_shim_test()
    sys.exit(0)
