"""Build recipe of libfdk.so (hipcc, gfx950 only).

``python -m triton_distributed_amd.build`` compiles every translation unit under ``csrc/`` and links
them into ``triton_distributed_amd/lib/libfdk.so``.  The library is built in-tree, ahead of time; the
Python host only ever loads the finished file.

``--timeline`` builds ``lib/libfdk_timeline.so`` instead: the same sources with ``-DFDK_TIMELINE``, whose
matrix-core split kernel records when every wavefront started, issued its first loads and finished
(``fdk_measure_args.timeline``, include/fdk_measure.h).  A measurement aid (``bench.py --op timeline`` loads it
through the ``FDK_LIBRARY`` environment variable); nothing else uses it, and ``--all`` builds both.
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
TIMELINE_LIB_PATH = LIB_DIR / "libfdk_timeline.so"
OBJ_DIR = PKG_DIR / "build"

SOURCES = [
    "fdk_api.hip", "fdk_combine.hip", "fdk_splitkv_valu.hip", "fdk_splitkv_mfma.hip",
    "fdk_splitkv_valu_bf16.hip", "fdk_splitkv_valu_bf16_fp8.hip", "fdk_splitkv_valu_fp16.hip",
    "fdk_splitkv_valu_fp16_fp8.hip", "fdk_splitkv_mfma_d64.hip", "fdk_splitkv_mfma_d128.hip", "fdk_splitkv_mfma_d256.hip",
    "fdk_splitkv_mfma_d64_bal.hip", "fdk_splitkv_mfma_d128_bal.hip", "fdk_splitkv_mfma_d256_bal.hip",
    "fdk_splitkv_mfma_d64_queue.hip", "fdk_splitkv_mfma_d128_queue.hip", "fdk_splitkv_mfma_d256_queue.hip", "fdk_kv_append.hip", "fdk_probe.hip",
    # q / K rows of two segments (192 = 128 + 64, 576 = 512 + 64), V rows of their own length
    "fdk_splitkv_mfma_d192.hip", "fdk_splitkv_mfma_d192_queue.hip", "fdk_splitkv_mfma_d192_bal.hip",
    "fdk_splitkv_mfma_d192v128.hip", "fdk_splitkv_mfma_d192v128_queue.hip", "fdk_splitkv_mfma_d192v128_bal.hip",
    "fdk_splitkv_mfma_d576v512.hip", "fdk_splitkv_mfma_d576v512_queue.hip", "fdk_splitkv_mfma_d576v512_bal.hip",
    # ... large q-head groups on one kv head: the wavefronts of a workgroup share the staged tiles
    "fdk_splitkv_mfma_d576v512_shared.hip", "fdk_splitkv_mfma_d576v512_shared_queue.hip", "fdk_splitkv_mfma_d576v512_shared_bal.hip",
    # rows of 128 values with more than 16 q heads per kv head
    "fdk_splitkv_mfma_d128_tiled.hip", "fdk_splitkv_mfma_d128_tiled_queue.hip", "fdk_splitkv_mfma_d128_tiled_bal.hip",
]

# the translation units that contain the matrix-core split kernel: the only ones the timeline build compiles anew
TIMELINE_SOURCES = ("fdk_splitkv_mfma_d64.hip", "fdk_splitkv_mfma_d128.hip", "fdk_splitkv_mfma_d256.hip",
                    "fdk_splitkv_mfma_d64_bal.hip", "fdk_splitkv_mfma_d128_bal.hip", "fdk_splitkv_mfma_d256_bal.hip",
                    "fdk_splitkv_mfma_d64_queue.hip", "fdk_splitkv_mfma_d128_queue.hip", "fdk_splitkv_mfma_d256_queue.hip", "fdk_probe.hip")

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


def _compile_one(hipcc: str, src: Path, obj: Path, extra=()) -> None:
    cmd = [hipcc, *HIPCC_FLAGS, *extra, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{res.stdout}\n{res.stderr}")


def build(verbose: bool = True, jobs: int = 8, timeline: bool = False) -> Path:
    """Compile and link libfdk.so (``timeline``: libfdk_timeline.so, see above); always recompiles.  Returns the
    library path."""
    hipcc = hipcc_path()
    obj_dir = OBJ_DIR / "timeline" if timeline else OBJ_DIR
    lib_path = TIMELINE_LIB_PATH if timeline else LIB_PATH
    extra = ("-DFDK_TIMELINE",) if timeline else ()
    obj_dir.mkdir(parents=True, exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    pairs = [(CSRC / s, obj_dir / (Path(s).stem + ".o")) for s in SOURCES]
    todo = pairs
    if timeline:
        # every other translation unit is the product library's object, if that has been built
        shared = {s: OBJ_DIR / (Path(s).stem + ".o") for s in SOURCES if s not in TIMELINE_SOURCES}
        if all(o.exists() for o in shared.values()):
            pairs = [(src, shared.get(src.name, obj)) for src, obj in pairs]
            todo = [(src, obj) for src, obj in pairs if src.name in TIMELINE_SOURCES]
    if verbose:
        print(f"[fdk build] hipcc={hipcc} -> {lib_path}", flush=True)
    todo = sorted(todo, key=lambda so: so[0].name not in TIMELINE_SOURCES)       # the longest compilations first
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo)))) as ex:
        list(ex.map(lambda so: _compile_one(hipcc, so[0], so[1], extra), todo))
    tmp = lib_path.with_suffix(".so.tmp")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(tmp), *[str(o) for _, o in pairs]]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, lib_path)
    if verbose:
        print(f"[fdk build] ok: {lib_path} ({lib_path.stat().st_size} bytes)", flush=True)
    return lib_path


def build_all(verbose: bool = True, jobs: int = 8) -> None:
    """Both libraries, with the compilations of the two sharing one pool of workers."""
    hipcc = hipcc_path()
    OBJ_DIR.mkdir(exist_ok=True)
    (OBJ_DIR / "timeline").mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    product = [(CSRC / s, OBJ_DIR / (Path(s).stem + ".o"), ()) for s in SOURCES]
    measure = [(CSRC / s, OBJ_DIR / "timeline" / (Path(s).stem + ".o"), ("-DFDK_TIMELINE",)) for s in TIMELINE_SOURCES]
    if verbose:
        print(f"[fdk build] hipcc={hipcc} -> {LIB_PATH}, {TIMELINE_LIB_PATH}", flush=True)
    # the matrix-core kernels take longest: start them first
    jobs_list = sorted(product + measure, key=lambda j: j[0].name not in TIMELINE_SOURCES)
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        list(ex.map(lambda j: _compile_one(hipcc, j[0], j[1], j[2]), jobs_list))
    swapped = {src.name: obj for src, obj, _ in measure}
    for lib_path, objs in ((LIB_PATH, [o for _, o, _ in product]),
                           (TIMELINE_LIB_PATH, [swapped.get(src.name, o) for src, o, _ in product])):
        tmp = lib_path.with_suffix(".so.tmp")
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(tmp), *[str(o) for o in objs]]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
        os.replace(tmp, lib_path)
        if verbose:
            print(f"[fdk build] ok: {lib_path} ({lib_path.stat().st_size} bytes)", flush=True)


if __name__ == "__main__":
    if "--all" in sys.argv[1:]:
        build_all()
    else:
        build(timeline="--timeline" in sys.argv[1:])
    sys.exit(0)
