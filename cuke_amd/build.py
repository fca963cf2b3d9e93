"""Builds libkge_mi355.so from cuke_amd/csrc/*.hip with hipcc for gfx950.

The library is built in-tree (cuke_amd/libkge_mi355.so) so that it travels
with the source tree; nothing is compiled at import time.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "libkge_mi355.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
] + os.environ.get("KGE_EXTRA_HIPCC_FLAGS", "").split()


def sources() -> list[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, src[:-4] + ".o")
    deps = [os.path.join(CSRC, src), os.path.join(HERE, "..", "include", "kge_mi355.h")] + \
        [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) > os.path.getmtime(d) for d in deps):
        return obj
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    msgs = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                     if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{msgs}")
    if msgs:
        print(msgs, file=sys.stderr)
    return obj


def build(force: bool = True, jobs: int = 8) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(force="--incremental" not in sys.argv))
