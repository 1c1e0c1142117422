"""pllmTensor's slicing helpers (nanoflow_amd/csrc/host/tensor.h) against hand-derived cases;
host only: the check program is compiled with g++ and run here."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_pllm_tensor_slicing(tmp_path):
    exe = str(tmp_path / "tensor_check")
    subprocess.check_call(["g++", "-std=c++20", "-O1", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
                           "-I" + os.path.join(ROOT, "nanoflow_amd", "csrc", "host"),
                           os.path.join(ROOT, "tests", "host", "tensor_check.cpp"), "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout + out.stderr
