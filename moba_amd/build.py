"""Builds the HIP kernels into ``moba_amd/libmoba_hip.so`` with hipcc for gfx950.

Run as ``python -m moba_amd.build``.  hipcc cross-compiles without a GPU.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libmoba_hip.so")
SOURCES = ["chunk_mean.hip", "gate_topk.hip", "lists.hip", "fwd.hip", "bwd.hip", "decode.hip", "plan.hip", "probe.hip", "capi.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 instructions stay off: scalar fp32 code only
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", "-Wno-inline-asm",
]


# per-source extra flags: the attention kernels never produce NaN from finite inputs, and
# telling the compiler so removes the canonicalisation of every MFMA result before a max
EXTRA = {"fwd.hip": ["-fno-honor-nans"]}


def _compile(src: str, force: bool) -> str:
    path = os.path.join(CSRC, src)
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    deps = [path, os.path.join(CSRC, "common.h"), os.path.join(CSRC, "attn_common.h"), os.path.abspath(__file__)]
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) > os.path.getmtime(d) for d in deps):
        return obj
    cmd = [HIPCC, *FLAGS, *EXTRA.get(src, []), "-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr[-8000:]}")
    errs = [l for l in r.stderr.splitlines() if "warning" in l and "packed-fp32-ops" not in l]
    if errs:
        sys.stderr.write("\n".join(errs[:20]) + "\n")
    return obj


def build(force: bool = True, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    # the hand-issued MFMAs of the dK/dV kernel: nothing touches their results too early in the generated code
    from . import asm_check
    report = asm_check.check_dkv_kernel(asm_check.device_assembly(HIPCC, FLAGS, os.path.join(CSRC, "bwd.hip")))
    if verbose:
        print(report)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {LIB} from {len(objs)} objects")
    return LIB


if __name__ == "__main__":
    build(force="--incremental" not in sys.argv)
