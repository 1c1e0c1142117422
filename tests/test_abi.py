"""The C-ABI libraries load without a GPU and export every symbol their headers declare."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:nf|pllm)_\w+)\s*\(", text)))


@pytest.mark.parametrize("header,libname", [
    ("nanoflow_kernels.h", "libnf_kernels.so"),
    ("nanoflow_pllm.h", "libnf_pipeline.so"),
])
def test_library_exports_every_declared_symbol(header, libname):
    path = os.path.join(ROOT, "nanoflow_amd", libname)
    if not os.path.exists(os.path.join(ROOT, "include", header)):
        pytest.skip(f"{header} not present")
    assert os.path.exists(path), f"{path} missing: run __graft_entry__.build()"
    lib = ctypes.CDLL(path)
    names = _declared(header)
    assert len(names) >= 5
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_kernel_binding_lists_the_header_symbols():
    from nanoflow_amd import kernels
    assert sorted(kernels.SYMBOLS) == _declared("nanoflow_kernels.h")
    assert kernels.lib().nf_abi_version() >= 1


def test_argument_errors_are_reported_without_a_gpu():
    # shape validation happens on the host before any launch
    from nanoflow_amd import kernels
    l = kernels.lib()
    rc = l.nf_rmsnorm_f16(None, None, None, 4, 30, 1e-5, None)   # hidden not a multiple of 8
    assert rc == -1 and b"multiple of 8" in l.nf_last_error()
    rc = l.nf_rope_append_f16(*([None] * 7), 3, 8, 2, 64, 16, 1.0, 1e4, 0.0, 0.0, None)
    assert rc == -1 and b"head_dim" in l.nf_last_error()
    rc = l.nf_attention_paged_f16(*([None] * 7), 3, 3, 12, 4, 128, 16, 0, 0, None, 0, None)
    assert rc == -1   # null pointers
    rc = l.nf_gemm_f16(None, None, None, None, 0, 64, 64, 1.0, 0.0, 0, None)  # M == 0 is a no-op
    assert rc == 0
