"""Builds libtract_rocm.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: ``python -m tract_amd.build [--force]``.  The shared library is written next
to this file (``tract_amd/libtract_rocm.so``); objects go to ``tract_amd/csrc/build``.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libtract_rocm.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
COMMON = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
    "-Rpass-analysis=kernel-resource-usage",   # per-kernel registers / spills / LDS, kept beside the objects
]
# per-file extra flags: the quantiser must not contract a*b+c into an fma
EXTRA = {"kv_quant.hip": ["-ffp-contract=off"], "elementwise.hip": ["-ffp-contract=off"], "kivi.hip": ["-ffp-contract=off"]}
SOURCES = ["abi.hip", "copy.hip", "kv_quant.hip", "sdpa_generic.hip", "sdpa_decode.hip", "sdpa_decode_quant.hip",
           "sdpa_prefill.hip", "sdpa_prefill_pp.hip", "elementwise.hip", "dat_format.hip", "q4_matvec.hip", "q4_matvec_mfma.hip", "q4_matmul.hip", "q4_tiled.hip", "sdpa_decode_mfma.hip", "kivi.hip"]


def _newer(target: str, deps: list[str]) -> bool:
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def _run(cmd: list[str]) -> None:
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    lines = [l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l]
    remarks = [l.split("remark: ", 1)[1].split(" [-Rpass", 1)[0].strip() for l in lines if "[-Rpass-analysis=kernel-resource-usage]" in l]
    kept, pending, in_remark = [], [], False
    for l in lines:   # drop the remarks together with their source-context and include-stack lines
        if "-Rpass-analysis=kernel-resource-usage" in l:
            pending, in_remark = [], True
        elif l.startswith("In file included from"):
            pending.append(l)
        elif in_remark and re.match(r"^\s*(\d+\s*)?\|", l):
            pass
        else:
            kept += pending + [l]
            pending, in_remark = [], False
    out = "\n".join(kept)
    if p.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    if "-c" in cmd:
        with open(cmd[cmd.index("-o") + 1] + ".usage.txt", "w") as f:
            f.write("\n".join(remarks) + "\n")
    if out.strip():
        print(out)


def resource_usage() -> dict:
    """{kernel symbol: {"VGPRs": n, "VGPRs Spill": n, "ScratchSize [bytes/lane]": n, ...}} of the last
    build (hipcc's kernel-resource-usage remarks), building first if an object is stale."""
    build(verbose=False)
    res = {}
    for src in SOURCES:
        path = os.path.join(OBJ, src.replace(".hip", ".o")) + ".usage.txt"
        cur = None
        for line in open(path):
            key, _, val = line.strip().partition(": ")
            if key == "Function Name":
                cur = res.setdefault(val, {"source": src})
            elif cur is not None and val.strip().lstrip("-").isdigit():
                cur[key] = int(val)
    return res


def build(force: bool = False, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    headers = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")) + [os.path.join(HERE, "..", "include", "tract_rocm.h"), __file__]
    jobs = []
    objs = []
    for src in SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ, src.replace(".hip", ".o"))
        objs.append(o)
        if force or not _newer(o, [s] + headers) or not os.path.exists(o + ".usage.txt"):
            jobs.append([HIPCC] + COMMON + EXTRA.get(src, []) + ["-c", s, "-o", o])
    if jobs:
        if verbose:
            print(f"[tract_amd.build] compiling {len(jobs)} file(s) for {ARCH}", flush=True)
        with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
            list(ex.map(_run, jobs))
    if jobs or not os.path.exists(LIB):
        _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB] + objs)
        if verbose:
            print(f"[tract_amd.build] linked {LIB}", flush=True)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
