"""Build liblandmark_hip.so for gfx950 with plain hipcc (cross-compiles without a GPU).

    python landmark-attention_amd/build.py [--force]

One object per translation unit in csrc/, linked into
landmark_hip/liblandmark_hip.so next to the Python shim that loads it.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "landmark_hip", "liblandmark_hip.so")
OBJ = os.path.join(HERE, "build")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-math-errno", "-ffp-contract=fast",
    # packed fp32 VALU ops are switched off for every device compile of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes", "-Wno-ignored-optimization-argument",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, src[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err:
        print(err, file=sys.stderr)
    return obj


def build(force: bool = True, jobs: int = 4) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    if not force and os.path.exists(OUT):
        newest = max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC))
        if os.path.getmtime(OUT) >= newest:
            return OUT
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return OUT


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or True))
