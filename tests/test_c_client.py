"""The C ABI from C: tests/c_abi/fdk_c_client.c is a C99 program that includes include/fdk.h, links libfdk.so and the
HIP runtime, and uses no Python, torch or C++.  Without a GPU it must compile and link; on the GPU it runs a small
paged decode through fdk_plan / fdk_workspace_bytes / fdk_decode and checks it against a naive double-precision
attention of its own (out 2e-2, lse 1e-3)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "c_abi", "fdk_c_client.c")
LIB_DIR = os.path.join(ROOT, "triton_distributed_amd", "lib")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def _build(tmp_path):
    if shutil.which("gcc") is None or not os.path.exists(os.path.join(ROCM, "lib", "libamdhip64.so")):
        pytest.skip("gcc or the HIP runtime library is not available")
    exe = tmp_path / "fdk_c_client"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", f"-I{ROCM}/include",
                    f"-I{ROOT}/include", SRC, f"-L{LIB_DIR}", "-lfdk", f"-L{ROCM}/lib", "-lamdhip64", "-lm",
                    f"-Wl,-rpath,{LIB_DIR}", f"-Wl,-rpath,{ROCM}/lib", "-o", str(exe)], check=True)
    return exe


def test_c_client_compiles_and_links_against_the_library(tmp_path):
    exe = _build(tmp_path)
    needed = subprocess.run(["readelf", "-d", str(exe)], capture_output=True, text=True, check=True).stdout
    assert "libfdk.so" in needed and "libamdhip64" in needed


@pytest.mark.gpu
def test_c_client_decodes_on_the_gpu(cuda_device, tmp_path):
    exe = _build(tmp_path)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    print(res.stdout, res.stderr, flush=True)
    assert res.returncode == 0, res.stderr
    assert res.stdout.strip().endswith("OK") and res.stdout.count("plan:") == 2
