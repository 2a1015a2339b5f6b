"""In-tree build recipes: hipcc for the HIP kernels + C-ABI library, g++ for the ATen extension.

Everything is built for gfx950 only and lands in torch_mlu_amd/lib/ so that the shared objects travel
with the source tree.  No JIT, no caches outside the tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_HERE)
CSRC = os.path.join(_HERE, "csrc")
LIBDIR = os.path.join(_HERE, "lib")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed-fp32 VALU forms are switched off for all device code.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wno-inline-asm",
    "-Wno-unused-command-line-argument",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


KERNEL_SOURCES = ("fa_fwd_kernels.hip", "fa_bwd_kernels.hip")


def _run(cmd, **kw):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    out = "\n".join(l for l in r.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if r.returncode != 0:
        raise RuntimeError("build step failed: " + " ".join(cmd) + "\n" + out)
    return out


def check_bwd256_scratch(remarks: str) -> None:
    """The head_dim-256 backward kernels run one wavefront per SIMD with their MFMA-only operands pinned to the
    accumulation registers; without the pins the compiler spilled up to 91 vector registers in them and they ran 1.5 x
    slower.  `remarks` is what hipcc -Rpass-analysis=kernel-resource-usage printed for fa_bwd_kernels.hip; a build in
    which one of those kernels uses scratch memory again is refused."""
    import re

    name = None
    seen = 0
    for line in remarks.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            continue
        m = re.search(r"remark:\s+ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and name and re.search(r"fa_bwd_(dq|dkv)_kernelIDF16[b_]Li256E", name):
            seen += 1
            if int(m.group(1)) != 0:
                raise RuntimeError(f"fa_bwd_kernels: {name} spills {m.group(1)} bytes per lane to scratch memory")
    if seen == 0:
        raise RuntimeError("fa_bwd_kernels: no resource remarks for the head_dim-256 kernels (check not run)")


def build_kernels(verbose: bool = False) -> str:
    """hipcc: csrc/fa_fwd_kernels.hip + csrc/fa_bwd_kernels.hip -> lib/libfa_fwd.so (the C ABI of
    include/fa_fwd.h and include/fa_bwd.h)."""
    os.makedirs(LIBDIR, exist_ok=True)
    out = os.path.join(LIBDIR, "libfa_fwd.so")
    tmp = out + ".tmp"
    srcs = [os.path.join(CSRC, f) for f in KERNEL_SOURCES]
    objs = [os.path.join(LIBDIR, os.path.splitext(f)[0] + ".o") for f in KERNEL_SOURCES]
    # one hipcc process per translation unit, side by side
    def extra(src):  # the backward file reports its kernels' registers and scratch (checked below)
        return ["-Rpass-analysis=kernel-resource-usage"] if src.endswith("fa_bwd_kernels.hip") else []

    procs = [(src, subprocess.Popen([HIPCC, *HIP_FLAGS, *extra(src), "-c", f"-I{INCLUDE}", f"-I{CSRC}", src, "-o", obj],
                                    stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
             for src, obj in zip(srcs, objs)]
    log = ""
    for src, pr in procs:
        o, _ = pr.communicate()
        o = "\n".join(l for l in o.splitlines() if "is not a recognized feature for this target" not in l)
        if pr.returncode != 0:
            raise RuntimeError("build step failed: hipcc -c " + src + "\n" + o)
        if extra(src):
            check_bwd256_scratch(o)
            kept, skip = [], 0  # a remark is three lines: the message, the source line, the caret
            for l in o.splitlines():
                if "-Rpass-analysis=kernel-resource-usage" in l:
                    skip = 2
                elif skip:
                    skip -= 1
                else:
                    kept.append(l)
            o = "\n".join(kept)
        log += o
    # the export list is the C ABI and nothing else (hidden visibility covers the C++ internals, the version script
    # the per-translation-unit marker symbols that hipcc emits)
    vs = os.path.join(LIBDIR, "exports.map")
    with open(vs, "w") as f:
        f.write("{ global: fa_fwd_*; fa_bwd_*; local: *; };\n")
    log += _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", f"-Wl,--version-script={vs}", *objs, "-o", tmp])
    os.replace(tmp, out)
    os.remove(vs)
    for obj in objs:
        os.remove(obj)
    if verbose and log.strip():
        print(log)
    return out


def build_aten(verbose: bool = False, out: str = None, extra_flags=()) -> str:
    """g++: csrc/fa_aten.cpp + csrc/fa_sdp_choice.cpp -> lib/libfa_aten.so (registers the forward and backward aten ops
    and the SDPA backend selector; links libfa_fwd.so by $ORIGIN).  `out` / `extra_flags`: an instrumented build next
    to the real one (the sanitizer test), which finds libfa_fwd.so through an rpath to lib/."""
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(LIBDIR, exist_ok=True)
    out = out or os.path.join(LIBDIR, "libfa_aten.so")
    tmp = out + ".tmp"
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = [f"-I{p}" for p in ce.include_paths("cuda")] + [f"-I{INCLUDE}"]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
        *inc, os.path.join(CSRC, "fa_aten.cpp"), os.path.join(CSRC, "fa_sdp_choice.cpp"), "-o", tmp,
        f"-L{LIBDIR}", "-lfa_fwd", f"-L{tlib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
        "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{LIBDIR}", f"-Wl,-rpath,{tlib}", "-Wl,--no-as-needed", *extra_flags,
    ]
    log = _run(cmd)
    os.replace(tmp, out)
    if verbose and log.strip():
        print(log)
    return out


def build_all(verbose: bool = False) -> None:
    build_kernels(verbose)
    build_aten(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built:", sorted(os.listdir(LIBDIR)))
