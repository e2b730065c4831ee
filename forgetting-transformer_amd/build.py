"""Build libfox_attn.so (gfx950 HIP kernels + flat C ABI) in-tree with hipcc.

    python forgetting-transformer_amd/build.py [--jobs N] [--force]

Each csrc/*.hip is compiled to an object under build/ and the objects are linked
into forgetting_transformer/_lib/libfox_attn.so.  hipcc cross-compiles for
gfx950, so no GPU is needed to build.
"""
from __future__ import annotations

import argparse
import concurrent.futures
import json
import os
import re
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
OBJ_DIR = ROOT / "build"
LIB_PATH = ROOT / "forgetting_transformer" / "_lib" / "libfox_attn.so"
USAGE_PATH = LIB_PATH.with_name("kernel_resources.json")   # registers, spills, LDS of every kernel, from the compiler
SOURCES = ["fox_fwd.hip", "fox_decode.hip", "fox_bwd.hip", "fox_scan.hip", "fox_shift.hip", "fox_norm_gate.hip", "fox_probe.hip", "fox_capi.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU ops are not to be generated for this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Rpass-analysis=kernel-resource-usage",   # parsed into kernel_resources.json: the MFMA kernels must not spill
]


_REMARK = re.compile(r"remark: (?:\s*)([A-Za-z ]+?)(?: \[bytes/(?:lane|block)\]| \[waves/SIMD\])?: (\S+) \[-Rpass-analysis")


def _parse_usage(stderr: str) -> dict:
    """{mangled kernel name: {"VGPRs": .., "AGPRs": .., "ScratchSize": .., "VGPRs Spill": .., "Occupancy": .., "LDS Size": ..}}"""
    usage, cur = {}, None
    for line in stderr.splitlines():
        m = _REMARK.search(line)
        if not m:
            continue
        key, val = m.group(1).strip(), m.group(2)
        if key == "Function Name":
            cur = usage.setdefault(val, {})
        elif cur is not None and val.lstrip("-").isdigit():
            cur[key] = int(val)
    return usage


def _compile(src: str):
    obj = OBJ_DIR / (Path(src).stem + ".o")
    cmd = [HIPCC, *FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = ("is not a recognized feature for this target", "-Rpass-analysis=kernel-resource-usage")
    excerpt = re.compile(r"^\s*\d*\s*\|")   # the source excerpt clang prints under every remark
    err = "\n".join(l for l in proc.stderr.splitlines() if not any(n in l for n in noise) and not excerpt.match(l))
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj, _parse_usage(proc.stderr)


def build(jobs: int = 4, force: bool = True) -> Path:
    """Compile and link the library; returns its path."""
    OBJ_DIR.mkdir(exist_ok=True)
    LIB_PATH.parent.mkdir(parents=True, exist_ok=True)
    if not force and LIB_PATH.exists():
        newest = max(p.stat().st_mtime for p in list(CSRC.iterdir()) + [ROOT.parent / "include" / "fox_attn.h"])
        if LIB_PATH.stat().st_mtime >= newest:
            return LIB_PATH
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [obj for obj, _ in results]
    usage = {name: u for _, per_file in results for name, u in per_file.items()}
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,--no-undefined", *map(str, objs), "-o", str(LIB_PATH)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    import ctypes
    ctypes.CDLL(str(LIB_PATH), mode=ctypes.RTLD_GLOBAL | getattr(os, "RTLD_NOW", 2))  # every symbol must resolve
    USAGE_PATH.write_text(json.dumps(usage, indent=1, sort_keys=True))
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=4)
    ap.add_argument("--force", action="store_true", default=False)
    ns = ap.parse_args()
    print(build(ns.jobs, force=True if ns.force else False))
