"""Builds libksimhip.so for gfx950 with hipcc (in-tree, no JIT cache).

Usage: python -m ksim_amd.csrc.build [--force] [--profile]

--profile builds libksimhip_prof.so instead: the same sources with -DKS_PROFILE, whose step kernel writes the clock cycles
it spends in each phase into the `dbg_M` debug buffer (and whose fused MLP kernel stamps its phases).  A tuning aid that
nothing loads by default.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(os.path.dirname(HERE), "libksimhip.so")
PROFILE_LIB = os.path.join(os.path.dirname(HERE), "libksimhip_prof.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared", "-fno-gpu-rdc",
    # packed-FP32 VALU forms are disabled on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-attributes",
]
# The physics kernels divide and take square roots by reciprocal and product (within 2.5 ulp) instead of the correctly
# rounded sequences, a tenth of the instructions each; their results are held to the float64 oracle within 1e-4, far
# above that.  The other sources keep IEEE division: the reward / termination known answers are compared bit for bit.
SOURCE_FLAGS = {"ks_dynamics.hip": ["-fno-hip-fp32-correctly-rounded-divide-sqrt"]}


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(HERE, "*.hip")))


def headers() -> list[str]:
    return sorted(glob.glob(os.path.join(HERE, "*.h"))) + [os.path.join(HERE, "..", "..", "include", "ksim_hip.h")]


def is_stale() -> bool:
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    return any(os.path.getmtime(p) > t for p in sources() + headers())


def build(force: bool = True, verbose: bool = True, profile: bool = False) -> str:
    if not force and not profile and not is_stale():
        return LIB
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    extra = ["-DKS_PROFILE"] if profile else []
    target = PROFILE_LIB if profile else LIB
    for src in sources():
        obj = os.path.join(HERE, "build", os.path.basename(src) + (".prof.o" if profile else ".o"))
        objs.append(obj)
        cmd = ([HIPCC] + [f for f in FLAGS if f != "-shared"] + SOURCE_FLAGS.get(os.path.basename(src), []) + extra +
               ["-c", src, "-o", obj])
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out:
            print(out)
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-rdc", "-o", target] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return target


if __name__ == "__main__":
    print("built", build(force=True, profile="--profile" in sys.argv))
