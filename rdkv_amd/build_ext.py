"""Build librdkv_hip.so (gfx950) in-tree with hipcc.  Used by ``__graft_entry__.build()``
and runnable directly: ``python -m rdkv_amd.build_ext``."""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "librdkv_hip.so")

COMMON = [
    "-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-fvisibility=hidden",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    # packed-fp32 VALU forms are kept off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Wno-unused-command-line-argument",
]
# bit-exact quantizer code must not contract a*b+c into fma
# (select.hip: an unroll request on the candidate loop of the shared-row knapsack is honoured at some of
# its inlined call sites only - measured 3 % faster with it - and the optimizer says so for the others)
PER_FILE = {"quantize.hip": ["-ffp-contract=off"], "select.hip": ["-ffp-contract=off", "-Wno-pass-failed"]}


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; cannot build librdkv_hip.so")


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def build(verbose: bool = True) -> str:
    hipcc = _hipcc()
    objdir = os.path.join(PKG, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *COMMON, *PER_FILE.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        objs = list(ex.map(compile_one, sources()))
    tmp = LIB + ".tmp"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    os.replace(tmp, LIB)
    if verbose:
        print(f"built {LIB} from {len(objs)} sources")
    return LIB


if __name__ == "__main__":
    build()
