"""The C ABI from plain C on the GPU: tests/c_abi_gpu_client.c allocates device buffers with the HIP runtime's C API, calls
omni_router_select through include/omni_moe_hip.h and checks ids and scores against a scalar loop; it then calls omni_init()
and captures, without any eager call before, a GEMM whose kernel needs 128 KiB of dynamic LDS and the two schedule entry
points into HIP graphs, and checks three replays of each."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_program_runs_router_select_on_device_buffers(tmp_path, device):
    from omni_moe.ops.hip import _lib
    lib = _lib.LIB_PATH
    assert os.path.exists(lib)
    exe = str(tmp_path / "c_abi_gpu_client")
    r = subprocess.run(["gcc", "-std=c99", "-O1", "-Wall", "-Wno-unused-function", "-I", os.path.join(ROOT, "include"), "-I", "/opt/rocm/include",
                        os.path.join(ROOT, "tests", "c_abi_gpu_client.c"), lib, "-L/opt/rocm/lib", "-lamdhip64",
                        "-Wl,-rpath," + os.path.dirname(lib), "-Wl,-rpath,/opt/rocm/lib", "-o", exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    print("running the C client", flush=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "c abi gpu ok" in r.stdout
