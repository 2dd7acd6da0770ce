"""Compiles the HIP sources in ``csrc/`` for gfx950 into ``libveloxquant_hip.so``.

Run as ``python -m veloxquant_mlx_amd.build`` (cross-compiles; no GPU needed).
"""

from __future__ import annotations

import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "_obj")
LIB = os.path.join(HERE, "libveloxquant_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # bit-exact quantisation needs separately rounded mul/add and IEEE division
    "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def sources() -> list[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


# Kernels that account for their own global-to-LDS copies with the outstanding-load counter: a
# register spilled to scratch memory would be reloaded with a vector load the accounting does
# not know, so these sources must compile without scratch.
NO_SCRATCH = ("attend_mfma_packed_",)


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, src[:-4] + ".o")
    check_scratch = src.startswith(NO_SCRATCH)
    extra = ["-Rpass-analysis=kernel-resource-usage"] if check_scratch else []
    cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    lines = r.stderr.splitlines()
    kept, in_remark = [], False
    for l in lines:
        if "packed-fp32-ops" in l:
            continue
        if "[-Rpass-analysis=kernel-resource-usage]" in l:
            in_remark = True            # followed by a source excerpt
            continue
        if in_remark and re.match(r"^\s*\d*\s*\|", l):
            continue
        in_remark = False
        kept.append(l)
    # "In file included from" lines that introduced nothing but remarks
    kept = [l for i, l in enumerate(kept)
            if not (l.startswith("In file included from") and
                    (i + 1 == len(kept) or kept[i + 1].startswith("In file included from")))]
    err = "\n".join(kept)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if check_scratch:
        name = "?"
        for l in lines:
            if "Function Name:" in l:
                name = l.split("Function Name:")[1].split()[0]
            elif "ScratchSize [bytes/lane]:" in l and int(l.split("ScratchSize [bytes/lane]:")[1].split()[0]) != 0:
                raise RuntimeError(f"{src}: kernel {name} uses scratch memory ({l.strip()}); "
                                   "its copy accounting needs a build without spills")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(jobs: int = 4) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, sources()))
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build())
