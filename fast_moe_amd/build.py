"""Builds libfastmoe_hip.so (gfx950) from fast_moe_amd/csrc with hipcc, in-tree.

    python -m fast_moe_amd.build            # compile every translation unit and link
    python -m fast_moe_amd.build --out fast_moe_amd/libfastmoe_hip_trace.so -DFMOE_TRACE
                                            # a second library beside it (here: the debug build whose
                                            # ring kernel records per-tile time stamps; load it with
                                            # FMOE_LIB_PATH=<that file>, see bench.py --tile-trace)
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libfastmoe_hip.so")
OBJ_DIR = os.path.join(CSRC, "build")

SOURCES = ["core.hip", "routing.hip", "quant.hip", "combine.hip", "gemm_api.hip", "gemm_bf16.hip",
           "gemm_fp8.hip", "gemm_f32.hip", "backward.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # keep the compiler from forming packed fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str, extra, obj_dir: str = OBJ_DIR) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    return obj


def build(extra_flags=(), jobs: int = 8, verbose: bool = True, out: str = LIB_PATH) -> str:
    # (a library under another name keeps its objects apart from the product's)
    obj_dir = OBJ_DIR if os.path.abspath(out) == LIB_PATH else os.path.join(OBJ_DIR, os.path.splitext(os.path.basename(out))[0])
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(SOURCES)))) as pool:
        objs = list(pool.map(lambda s: _compile(s, list(extra_flags), obj_dir), SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {out} ({os.path.getsize(out) / 1e6:.1f} MB)")
    return out


if __name__ == "__main__":
    args = sys.argv[1:]
    target = LIB_PATH
    if "--out" in args:
        i = args.index("--out")
        target = os.path.abspath(args[i + 1])
        del args[i:i + 2]
    build(extra_flags=args, out=target)
