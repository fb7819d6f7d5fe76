"""Builds libfta.so (HIP kernels + C ABI) in-tree for gfx950 with hipcc.

    python flash-triangle-attention_amd/build.py [--force]

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB = os.path.join(HERE, "libfta.so")
SOURCES = ["fta_api.hip", "fta_fwd.hip", "fta_fwd1.hip", "fta_fwd2.hip", "fta_fwd_feat.hip", "fta_bwd.hip", "fta_bwd_feat.hip", "fta_bwd_dq1.hip",
           "fta_bwd_dkdv1.hip"]

DEMO_SOURCE = "fta_c_demo.cpp"
DEMO = os.path.join(HERE, "fta_c_demo")

OBJDIR = os.path.join(HERE, "build")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms are kept off for every device translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
]


def needs_build() -> bool:
    if not os.path.exists(LIB) or not os.path.exists(DEMO):
        return True
    t = os.path.getmtime(LIB)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [os.path.join(INCLUDE, "fta.h")]
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = True, verbose: bool = False) -> str:
    if not force and not needs_build():
        return LIB
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    # one object per source, compiled side by side (each is an independent hipcc run), then one link
    os.makedirs(OBJDIR, exist_ok=True)
    objs = [os.path.join(OBJDIR, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    cmds = [[hipcc] + FLAGS + ["-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(SOURCES, objs)]
    if verbose:
        for c in cmds:
            print(" ".join(c))
    procs = [subprocess.Popen(c, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True) for c in cmds]
    failed = False
    for pr in procs:
        out, _ = pr.communicate()
        if pr.returncode != 0:
            sys.stderr.write(out)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed compiling libfta.so")
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(link))
    res = subprocess.run(link, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed linking libfta.so")
    # the C-ABI demo: a plain C++ program (HIP runtime only) linked against the library next to it
    demo = [hipcc, "--offload-arch=gfx950", "-O2", "-std=c++17", "-Wno-unused-command-line-argument", "-I", INCLUDE,
            os.path.join(CSRC, DEMO_SOURCE), "-o", DEMO, "-L", HERE, "-lfta", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(demo))
    res = subprocess.run(demo, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed building fta_c_demo")
    return LIB


if __name__ == "__main__":
    print(build(force=True, verbose=True))
