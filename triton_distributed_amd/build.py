"""Build recipe of libfdk.so (hipcc, gfx950 only).

``python -m triton_distributed_amd.build`` compiles every translation unit under ``csrc/`` and links
them into ``triton_distributed_amd/lib/libfdk.so``.  The library is built in-tree, ahead of time; the
Python host only ever loads the finished file.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libfdk.so"
OBJ_DIR = PKG_DIR / "build"

SOURCES = [
    "fdk_api.hip", "fdk_combine.hip", "fdk_splitkv_valu.hip", "fdk_splitkv_mfma.hip",
    "fdk_splitkv_valu_bf16.hip", "fdk_splitkv_valu_bf16_fp8.hip", "fdk_splitkv_valu_fp16.hip",
    "fdk_splitkv_valu_fp16_fp8.hip", "fdk_splitkv_mfma_d64.hip", "fdk_splitkv_mfma_d128.hip", "fdk_splitkv_mfma_d256.hip", "fdk_kv_append.hip", "fdk_probe.hip",
]

# -packed-fp32-ops off: v_pk_*_f32 forms are not to be generated for this target.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-pass-failed",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm")


def _compile_one(hipcc: str, src: Path, obj: Path) -> None:
    cmd = [hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{res.stdout}\n{res.stderr}")


def build(verbose: bool = True, jobs: int = 8) -> Path:
    """Compile and link libfdk.so; always recompiles.  Returns the library path."""
    hipcc = hipcc_path()
    OBJ_DIR.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    pairs = [(CSRC / s, OBJ_DIR / (Path(s).stem + ".o")) for s in SOURCES]
    if verbose:
        print(f"[fdk build] hipcc={hipcc} -> {LIB_PATH}", flush=True)
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(pairs)))) as ex:
        list(ex.map(lambda so: _compile_one(hipcc, so[0], so[1]), pairs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(tmp), *[str(o) for _, o in pairs]]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[fdk build] ok: {LIB_PATH} ({LIB_PATH.stat().st_size} bytes)", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
