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


def test_split_over_k_plan_without_a_gpu():
    """Which GEMM launches are split over K, and into how many shares, is host arithmetic (the CU count
    defaults to the MI355X's 256 without a device): at most 512 rows, at least 1024 deep, as many
    shares as fill the chip (tiles of 64 x 256 up to 64 rows, 128 x 128 up to 256, 320 x 128 up to 320, else
    256 x 256),
    each at least 512 deep, at most 16."""
    from nanoflow_amd import kernels
    l = kernels.lib()
    shares = lambda M, N, K: l.nf_gemm_workspace_bytes(M, N, K) // (M * N * 4)
    assert shares(64, 6144, 4096) == 8            # 24 tiles -> 10 would fit, K / 512 = 8
    assert shares(64, 4096, 14336) == 16          # 16 tiles, capped at 16 shares
    assert shares(128, 4096, 4096) == 8           # 32 tiles of 128 x 128
    assert shares(200, 6144, 4096) == 2           # 96 tiles
    assert shares(257, 4096, 4096) == 8           # 257 .. 320 rows: one 320-row tile per 128 columns, 32 tiles
    assert shares(267, 8192, 28672) == 4          # the down projection in the KV-bound 70B regime: 64 tiles
    assert shares(321, 4096, 4096) == 0           # above 320 rows only long contractions are split
    assert shares(400, 4096, 14336) == 8          # two 256-row tiles per 256 columns: 32 tiles
    assert shares(513, 4096, 4096) == 0           # more than 512 rows
    assert shares(2048, 4096, 14336) == 2         # dense rows, 128 tiles of 256 x 256 against a long contraction: two shares
    assert shares(1500, 4096, 14336) == 2 and shares(1024, 4096, 14336) == 0    # 96 tiles; 64 tiles: a quarter of the CUs
    assert shares(2048, 4096, 4096) == 0 and shares(2048, 8192, 28672) == 0     # too shallow; tiles enough
    assert shares(64, 128256, 4096) == 0          # the LM head has tiles enough
    assert shares(64, 4096, 512) == 0             # too shallow
    assert l.nf_gemm_workspace_bytes_upto(2048, 6144, 4096) == max(l.nf_gemm_workspace_bytes(m, 6144, 4096)
                                                                   for m in range(1, 513))
    assert l.nf_gemm_workspace_bytes_upto(2048, 4096, 14336) == 2 * 2048 * 4096 * 4
    assert l.nf_gemm_workspace_bytes_upto(1400, 4096, 14336) == max(l.nf_gemm_workspace_bytes(m, 4096, 14336)
                                                                    for m in range(1, 1401))
    dual = lambda M, N, K: l.nf_dual_swiglu_workspace_bytes(M, N, K) // (2 * M * N * 4)
    assert dual(64, 14336, 4096) == 2 and dual(64, 28672, 8192) == 0 and dual(256, 14336, 4096) == 0
    assert l.nf_gemm_f8w_workspace_bytes(2048, 4096) == 2048 * 4096 + 2048 * 4


def test_extension_module_imports_without_a_gpu_and_has_the_reference_names():
    """nanoflow_amd/ext/pllm_python.*.so (pybind11 over the control-plane C ABI): the reference's
    module surface (pipeline/src/pybind.cu:189-284), importable with no device present."""
    import importlib.util
    ext = os.path.join(ROOT, "nanoflow_amd", "ext")
    files = [f for f in os.listdir(ext) if f.startswith("pllm_python.") and f.endswith(".so")] if os.path.isdir(ext) else []
    assert files, "extension module missing: run __graft_entry__.build()"
    spec = importlib.util.spec_from_file_location("pllm_python", os.path.join(ext, files[0]))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    for name in ("init", "config", "update", "run", "run_async", "run_async_wait", "finalize", "getPipelineOutput",
                 "setRank", "setModelConfig", "createModelWeight", "createInitData", "VortexInitData",
                 "VortexUpdateData", "VortexConfigData", "VortexWeight", "VortexLayerWeight", "VortexModelWeight",
                 "VortexOutputData", "PipelineType"):
        assert hasattr(mod, name), name
    u = mod.VortexUpdateData()
    u.decodePrefillBorder = 7
    u.setKVIndices(0)
    u.setGemvBatchSize(__import__("numpy").array([1, 2, 3, 4], dtype="int32"))
    assert u.decodePrefillBorder == 7
    c = mod.VortexConfigData()
    c.setGemmOpTag(["a", "b"])
    assert c.gemmOpTag == ["a", "b"]
    with pytest.raises(RuntimeError):
        mod.setRank(2, 2)              # one rank only


def test_nanobatch_split_and_attention_groups_are_checked_on_the_host():
    """What pllm_config / pllm_update reject before anything is built or written, through the two
    stateless checkers they call: a QKV cut outside its nano-batch, and decode-attention groups that
    reach past the QKV pieces finished when the group's launch starts (four-way schedule)."""
    lib = ctypes.CDLL(os.path.join(ROOT, "nanoflow_amd", "libnf_pipeline.so"))
    lib.pllm_last_error.restype = ctypes.c_char_p
    PLLM, NONOVERLAP, NANOBATCH, OFFLOAD, LOCAL, SEQ = 0, 1, 2, 3, 7, 8
    cfg = lib.pllm_check_nanobatch_split
    assert cfg(PLLM, 2048, 2048, 640, 256, 768) == 0
    assert cfg(PLLM, 2048, 2048, 640, 0, 1408) == 0              # cuts on the borders are allowed
    for bad in ((PLLM, 2048, 2048, 640, 641, 768), (NANOBATCH, 2048, 2048, 640, 256, 1409),
                (OFFLOAD, 2048, 2048, 640, -1, 10), (PLLM, 2048, 2048, 2048, 1, 1), (PLLM, 1024, 2048, 640, 1, 1),
                (LOCAL, 2048, 2048, 0, 0, 0), (42, 2048, 2048, 640, 1, 1)):
        assert cfg(*bad) == -1, bad
    assert b"kqv3_size" in (cfg(NANOBATCH, 2048, 2048, 640, 256, 1409), lib.pllm_last_error())[1]
    assert cfg(LOCAL, 2048, 2048, 640, 9999, -5) == 0            # two-way schedules never read the QKV cuts
    assert cfg(SEQ, 2048, 2048, 0, 0, 0) == 0 and cfg(NONOVERLAP, 2048, 2048, 0, 0, 0) == 0
    grp = lib.pllm_check_gemv_split
    g = lambda *v: (ctypes.c_int32 * 4)(*v)
    # 1000 decode rows on 640 | 1408 with QKV pieces 256 | 384 | 768 | 640
    assert grp(PLLM, 640, 256, 768, 1000, g(256, 384, 360, 0)) == 0
    assert grp(PLLM, 640, 256, 768, 1000, g(200, 440, 360, 0)) == 0      # group 1 inside pieces 1..2
    assert grp(PLLM, 640, 256, 768, 1000, g(300, 340, 360, 0)) == -1     # group 0 past QKV piece 1
    assert b"group 0" in lib.pllm_last_error()
    assert grp(PLLM, 640, 256, 768, 1800, g(256, 384, 800, 360)) == -1   # groups 0..2 past piece 3
    assert grp(PLLM, 640, 256, 768, 1800, g(256, 384, 768, 392)) == 0
    assert grp(PLLM, 640, 256, 768, 1000, g(256, 300, 444, 0)) == -1     # groups 0+1 != decode rows of nano-batch 1
    assert grp(PLLM, 640, 256, 768, 1000, g(256, 384, 300, 0)) == -1     # does not sum to the decode rows
    assert grp(LOCAL, 640, 256, 768, 1000, g(300, 340, 360, 0)) == 0     # two-way: only the 0+1 rule
    assert grp(SEQ, 0, 0, 0, 1000, g(1000, 0, 0, 0)) == 0
    assert grp(PLLM, 640, 256, 768, 1000, None) == -1
