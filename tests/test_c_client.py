"""The C ABI from C: tests/c_abi/fdk_c_client.c is a C99 program that includes include/fdk.h, links libfdk.so and the
HIP runtime, and uses no Python, torch or C++.  Without a GPU it must compile and link; on the GPU it runs a small
paged decode through fdk_plan / fdk_workspace_bytes / fdk_decode and checks it against a naive double-precision
attention of its own (out 2e-2, lse 1e-3).  The same program is also compiled against tests/c_abi/fdk_abi8_rev0.h, the
header as first released under this ABI version: a caller built then must run unchanged against today's library."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "c_abi", "fdk_c_client.c")
LIB_DIR = os.path.join(ROOT, "triton_distributed_amd", "lib")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


FROZEN = os.path.join(ROOT, "tests", "c_abi", "fdk_abi8_rev0.h")
HEADERS = ["current", "first_release"]


def _build(tmp_path, header="current"):
    if shutil.which("gcc") is None or not os.path.exists(os.path.join(ROCM, "lib", "libamdhip64.so")):
        pytest.skip("gcc or the HIP runtime library is not available")
    inc = f"{ROOT}/include"
    if header == "first_release":              # the program's #include "fdk.h" finds the frozen header
        inc = tmp_path / "include_first_release"
        inc.mkdir()
        shutil.copy(FROZEN, inc / "fdk.h")
    exe = tmp_path / f"fdk_c_client_{header}"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", f"-I{ROCM}/include",
                    f"-I{inc}", SRC, f"-L{LIB_DIR}", "-lfdk", f"-L{ROCM}/lib", "-lamdhip64", "-lm",
                    f"-Wl,-rpath,{LIB_DIR}", f"-Wl,-rpath,{ROCM}/lib", "-o", str(exe)], check=True)
    return exe


@pytest.mark.parametrize("header", HEADERS)
def test_c_client_compiles_and_links_against_the_library(tmp_path, header):
    exe = _build(tmp_path, header)
    needed = subprocess.run(["readelf", "-d", str(exe)], capture_output=True, text=True, check=True).stdout
    assert "libfdk.so" in needed and "libamdhip64" in needed


@pytest.mark.gpu
@pytest.mark.parametrize("header", HEADERS)
def test_c_client_decodes_on_the_gpu(cuda_device, tmp_path, header):
    exe = _build(tmp_path, header)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    print(res.stdout, res.stderr, flush=True)
    assert res.returncode == 0, res.stderr
    assert res.stdout.strip().endswith("OK") and res.stdout.count("plan:") == 2
