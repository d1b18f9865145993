"""Build libmsq.so (hipcc, gfx950 only) in-tree. `python -m macseek_amd.build` or `build()`."""
import json
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libmsq.so")
# the benchmark's instruction-issue probe: a shared object of its own, no part of the library
PROBE_SRC = [os.path.join(CSRC, "probe", f) for f in ("issue_probe.hip", "handover_probe.hip", "lds_bank_probe.hip")]
PROBE_OUT = os.path.join(HERE, "libmsq_probe.so")
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
         "msq_matvec.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=12"],
         "msq_router.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=6"],  # x, W, dim, n_exp of the fused router: 11.1 -> 10.8 us
         "msq_matmul.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=14"]}  # the fused matmul's arguments: 2-3 % at 64 / 128 tokens


# What the compiler reports per kernel (-Rpass-analysis=kernel-resource-usage) is kept beside the library: registers, LDS
# and, above all, scratch bytes per lane -- a kernel that starts to keep an array or spilled registers in scratch memory
# still computes the right thing, several times slower, and tests/test_kernel_resources.py reads this file to notice.
REPORT = os.path.join(HERE, "libmsq.kernels.json")
_FIELDS = {"VGPRs": "vgprs", "AGPRs": "agprs", "TotalSGPRs": "sgprs", "ScratchSize [bytes/lane]": "scratch",
           "VGPRs Spill": "vgpr_spill", "LDS Size [bytes/block]": "lds", "Occupancy [waves/SIMD]": "occupancy"}


def _resources(text):
    kernels, cur = {}, None
    for l in text.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", l)
        if m:
            cur = kernels.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z][A-Za-z \[\]/]*?): (\d+)", l)
        if m and cur is not None and m.group(1) in _FIELDS:
            cur[_FIELDS[m.group(1)]] = int(m.group(2))
    return kernels


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.basename(src)[:-4] + ".o")
    r = subprocess.run([HIPCC] + FLAGS + EXTRA.get(os.path.basename(src), []) +
                       ["-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", obj],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l and "remark:" not in l)
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, _resources(r.stdout)


def build(verbose=True):
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        done = list(ex.map(_compile, srcs))
    objs = [o for o, _ in done]
    report = {}
    for (_, k), src in zip(done, srcs):
        report[os.path.basename(src)] = k
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs +
                       ["-L/opt/rocm/lib", "-lrocblas", "-Wl,-rpath,/opt/rocm/lib"],  # rocBLAS: the dense fp16 GEMM of msq_matmul for many tokens
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    with open(REPORT, "w") as f:
        json.dump(report, f, indent=1, sort_keys=True)
    r = subprocess.run([HIPCC] + FLAGS + ["-shared"] + PROBE_SRC + ["-o", PROBE_OUT], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (PROBE_SRC, r.stdout))
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
