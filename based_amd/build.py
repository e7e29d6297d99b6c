"""Compiles the HIP sources under based_amd/csrc into based_amd/libbased_hip.so for gfx950.

Usage:  python -m based_amd.build          (cross-compiles; no GPU needed)
"""
from __future__ import annotations

import concurrent.futures as cf
import glob
import json
import os
import re
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OBJDIR = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libbased_hip.so")

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-command-line-argument",
    # packed-fp32 VALU forms are disabled for all device code built here
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", INCLUDE,
    "-I", CSRC,
]


RESOURCES = os.path.join(OBJDIR, "resource_usage.json")
_REMARK = re.compile(r"remark:\s+(Function Name|VGPRs|AGPRs|VGPRs Spill|SGPRs Spill|ScratchSize \[bytes/lane\]|"
                     r"Occupancy \[waves/SIMD\]|LDS Size \[bytes/block\]):\s+(\S+)")


_SNIPPET = re.compile(r"^\s*\d*\s*\|")   # the source lines clang shows under a remark


def _compile(src: str):
    """Compiles one source; returns (object file, {kernel: resource figures the compiler reports})."""
    obj = os.path.join(OBJDIR, os.path.basename(src).rsplit(".", 1)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    noise = "unknown target-feature"  # host pass does not know the gfx feature name; harmless
    usage, cur, other = {}, None, []
    for line in r.stderr.splitlines():
        m = _REMARK.search(line)
        if m:
            if m.group(1) == "Function Name":
                cur = usage.setdefault(m.group(2), {})
            elif cur is not None:
                cur[m.group(1)] = int(m.group(2))
        elif ("-Rpass-analysis" not in line and line.strip() and noise not in line and "packed-fp32-ops" not in line
              and not _SNIPPET.match(line)):
            other.append(line)
    if other:
        sys.stderr.write("\n".join(other) + "\n")
    return obj, usage


def build(verbose: bool = False) -> str:
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError("no HIP sources found")
    with cf.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        done = list(ex.map(_compile, srcs))
    objs = [o for o, _ in done]
    # what the compiler says each kernel needs (registers, spills, LDS): kept beside the objects; a
    # kernel that spills vector registers is named, because a few spilled registers in a loop have
    # cost a hot kernel 5 % here without any other sign
    usage = {os.path.basename(src): u for src, (_, u) in zip(srcs, done)}
    with open(RESOURCES, "w") as f:
        json.dump(usage, f, indent=1, sort_keys=True)
    for src, kernels in usage.items():
        for name, u in kernels.items():
            if u.get("VGPRs Spill", 0) > 0:
                sys.stderr.write(f"note: {src}: {name} spills {u['VGPRs Spill']} vector registers\n")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


if __name__ == "__main__":
    build(verbose=True)
