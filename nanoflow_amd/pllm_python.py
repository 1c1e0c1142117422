"""Python face of the pipeline control plane (C ABI: include/nanoflow_pllm.h).

Keeps the names of the reference's pybind11 module ``pllm_python``
(pipeline/src/pybind.cu:189-284): ``setRank``, ``setModelConfig``, ``init``, ``config``,
``update``, ``run``, ``run_async``, ``run_async_wait``, ``getPipelineOutput``, ``finalize``,
the ``Vortex*`` data classes and ``PipelineType``.  Raw addresses are passed as integers, as
in the reference (``setPtr``, ``setKVIndices`` ...).

There is no fallback: a missing ``libnf_pipeline.so`` raises.
"""
from __future__ import annotations

import ctypes as C
import enum
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnf_pipeline.so")

_u16p = C.POINTER(C.c_uint16)
_i32p = C.POINTER(C.c_int32)


class NanoflowPipelineError(RuntimeError):
    pass


class PipelineType(enum.IntEnum):
    PLLM = 0
    NONOVERLAP = 1
    NANOBATCH = 2
    PLLMOFFLOAD = 3
    KQVBIAS = 4
    NONOVERLAP_KQVBIAS = 5
    NANOBATCH_KQVBIAS = 6
    LOCAL = 7
    NON_OVERLAP_LOCAL = 8
    NANOBATCH_LOCAL = 9


class VortexWeight(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("N", C.c_int), ("K", C.c_int)]

    def setPtr(self, ptr: int):
        self.ptr = ptr


class VortexLayerWeight(C.Structure):
    _fields_ = [(n, VortexWeight) for n in ("W_O1", "W_O2", "W_U", "W_G", "W_D", "W_KQV", "B_KQV",
                                            "W_LN_Attention", "W_LN_FFN", "W_ROT")]


class _CModelWeight(C.Structure):
    _fields_ = [("lm_head", VortexWeight), ("embedding", VortexWeight),
                ("model_layernorm", VortexWeight), ("layer_weight", C.POINTER(VortexLayerWeight)),
                ("num_layers", C.c_int)]


class VortexModelWeight:
    def __init__(self):
        self.lm_head = VortexWeight()
        self.embedding = VortexWeight()
        self.model_layernorm = VortexWeight()
        self.layer_weight: list[VortexLayerWeight] = []

    def _to_c(self):
        arr = (VortexLayerWeight * max(len(self.layer_weight), 1))(*self.layer_weight)
        c = _CModelWeight(self.lm_head, self.embedding, self.model_layernorm, arr,
                          len(self.layer_weight))
        return c, arr


class _CInitData(C.Structure):
    _fields_ = [("kv_data", C.POINTER(C.c_void_p)), ("weight", _CModelWeight),
                ("weight_size", C.c_size_t), ("tmp_buffer", C.c_void_p),
                ("tmp_buffer_size", C.c_size_t)]


class VortexInitData:
    def __init__(self):
        self.kv_data: list[int] = []
        self.weight = VortexModelWeight()
        self.weight_size = 0
        self.tmp_buffer = 0
        self.tmp_buffer_size = 0

    def setKVdata(self, kv_data):
        self.kv_data = [int(p) for p in kv_data]

    def setWeight(self, weight: VortexModelWeight, weight_size: int = 0):
        self.weight = weight
        self.weight_size = weight_size

    def setTmpBuffer(self, tmp_buffer: int, tmp_buffer_size: int):
        self.tmp_buffer = tmp_buffer
        self.tmp_buffer_size = tmp_buffer_size


class _CUpdateData(C.Structure):
    _fields_ = [("decodePrefillBorder", C.c_int), ("prefillNum", C.c_int),
                ("prefillTokensNum", C.c_int), ("keepTokenListLength", C.c_int),
                ("input_tokens", C.c_void_p), ("input_indptr", C.c_void_p),
                ("rev_input_indptr", C.c_void_p), ("keep_token_list", C.c_void_p),
                ("kv_indptr", C.c_void_p), ("kv_indices", C.c_void_p),
                ("kv_last_page_len", C.c_void_p), ("per_token_offset", C.c_void_p),
                ("gemv_batch_size", C.c_void_p), ("gemv_num_blocks", C.c_void_p)]


class VortexUpdateData:
    """Host addresses of this iteration's arrays (int32)."""

    def __init__(self):
        self.decodePrefillBorder = 0
        self.prefillNum = 0
        self.prefillTokensNum = 0
        self.keepTokenListLength = 0
        self._p = {}
        self._keep = []

    def _set(self, name, addr):
        self._p[name] = int(addr)

    def setInputEmbedding(self, a): self._set("input_tokens", a)
    def setInputIndptr(self, a): self._set("input_indptr", a)
    def setRevInputIndptr(self, a): self._set("rev_input_indptr", a)
    def setKeepTokenList(self, a): self._set("keep_token_list", a)
    def setKVIndptr(self, a): self._set("kv_indptr", a)
    def setKVIndices(self, a): self._set("kv_indices", a)
    def setKVLastPageLen(self, a): self._set("kv_last_page_len", a)
    def setPerTokenOffset(self, a): self._set("per_token_offset", a)

    def setGemvBatchSize(self, arr):
        a = np.ascontiguousarray(arr, dtype=np.int32)
        self._keep.append(a)
        self._set("gemv_batch_size", a.ctypes.data)

    def setGemvNumBlocks(self, arr):
        a = np.ascontiguousarray(arr, dtype=np.int32)
        self._keep.append(a)
        self._set("gemv_num_blocks", a.ctypes.data)

    def _to_c(self):
        c = _CUpdateData(self.decodePrefillBorder, self.prefillNum, self.prefillTokensNum,
                         self.keepTokenListLength)
        for k, v in self._p.items():
            setattr(c, k, v)
        return c


class _CConfigData(C.Structure):
    _fields_ = [("gemm_op_tag", C.POINTER(C.c_char_p)), ("num_gemm_op_tag", C.c_int),
                ("global_batch_size", C.c_int), ("nanobatch_1_size", C.c_int),
                ("kqv1_size", C.c_int), ("kqv3_size", C.c_int)]


class VortexConfigData:
    def __init__(self):
        self.gemmOpTag: list[str] = []
        self.globalBatchSize = 0
        self.nanobatch1Size = 0
        self.kqv1Size = 0
        self.kqv3Size = 0

    def setGemmOpTag(self, tags):
        self.gemmOpTag = [str(t) for t in tags]


class PipelineTimings(C.Structure):
    _fields_ = [("iter_ms", C.c_double), ("decode_attn_ms", C.c_double),
                ("decode_attn_launches", C.c_long), ("prefill_attn_ms", C.c_double),
                ("prefill_attn_launches", C.c_long)]


SYMBOLS = [
    "pllm_last_error", "pllm_set_model_config", "pllm_set_rank", "pllm_tmp_buffer_halves",
    "pllm_max_page_num", "pllm_init", "pllm_model_weight_to_gpu", "pllm_config", "pllm_update",
    "pllm_run", "pllm_run_async", "pllm_run_async_wait", "pllm_get_pipeline_output",
    "pllm_finalize", "pllm_build_input_tokens", "pllm_set_profiling", "pllm_get_timings",
    "pllm_reset_timings", "pllm_debug_buffer",
]

_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NanoflowPipelineError(
                f"{LIB_PATH} is missing: build it with `make -C nanoflow_amd/csrc` (no fallback)")
        # the host library resolves libnf_kernels.so through its $ORIGIN rpath
        l = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        l.pllm_last_error.restype = C.c_char_p
        l.pllm_set_model_config.argtypes = [C.c_char_p]
        l.pllm_set_rank.argtypes = [C.c_int, C.c_int]
        l.pllm_tmp_buffer_halves.restype = C.c_size_t
        l.pllm_max_page_num.restype = C.c_size_t
        l.pllm_init.argtypes = [C.POINTER(_CInitData), C.c_int]
        l.pllm_model_weight_to_gpu.argtypes = [C.POINTER(_CModelWeight), C.POINTER(_CModelWeight),
                                               C.POINTER(VortexLayerWeight)]
        l.pllm_config.argtypes = [C.POINTER(_CConfigData)]
        l.pllm_update.argtypes = [C.POINTER(_CUpdateData)]
        l.pllm_get_pipeline_output.argtypes = [C.POINTER(_i32p), C.POINTER(C.c_int)]
        l.pllm_build_input_tokens.argtypes = [_i32p, C.c_int, _i32p, C.c_int, _i32p, C.c_int, _i32p]
        l.pllm_set_profiling.argtypes = [C.c_int]
        l.pllm_get_timings.argtypes = [C.POINTER(PipelineTimings)]
        l.pllm_debug_buffer.argtypes = [C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_int),
                                        C.POINTER(C.c_int)]
        _lib = l
    return _lib


def _check(rc, what):
    if rc != 0:
        raise NanoflowPipelineError(f"{what} failed ({rc}): {lib().pllm_last_error().decode()}")


_nranks = 1
_alive = []  # ctypes objects the C side keeps pointers into


def setRank(nranks: int, vnranks: int):
    global _nranks
    _check(lib().pllm_set_rank(nranks, vnranks), "setRank")
    _nranks = nranks


def setModelConfig(filename: str):
    _check(lib().pllm_set_model_config(filename.encode()), "setModelConfig")


def tmpBufferHalves() -> int:
    return lib().pllm_tmp_buffer_halves()


def maxPageNum() -> int:
    return lib().pllm_max_page_num()


def init(data_array, pipeTy):
    """data_array: [VortexInitData] with DEVICE weights (one rank)."""
    if len(data_array) != 1:
        raise NanoflowPipelineError("this build runs exactly one rank")
    d = data_array[0]
    cw, arr = d.weight._to_c()
    kv = (C.c_void_p * max(len(d.kv_data), 1))(*d.kv_data)
    ci = _CInitData(kv, cw, d.weight_size, d.tmp_buffer, d.tmp_buffer_size)
    _alive.extend([cw, arr, kv, ci])
    _check(lib().pllm_init(C.byref(ci), int(pipeTy)), "init")


def config(config_array):
    c = config_array[0]
    tags = (C.c_char_p * max(len(c.gemmOpTag), 1))(*[t.encode() for t in c.gemmOpTag])
    cc = _CConfigData(tags, len(c.gemmOpTag), c.globalBatchSize, c.nanobatch1Size, c.kqv1Size,
                      c.kqv3Size)
    _check(lib().pllm_config(C.byref(cc)), "config")


def update(update_array):
    cu = update_array[0]._to_c()
    _check(lib().pllm_update(C.byref(cu)), "update")


def run():
    _check(lib().pllm_run(), "run")


def run_async():
    _check(lib().pllm_run_async(), "run_async")


def run_async_wait():
    _check(lib().pllm_run_async_wait(), "run_async_wait")


def getPipelineOutput() -> np.ndarray:
    """Copy of the sampled token ids of the last completed run (int32)."""
    p = _i32p()
    n = C.c_int()
    _check(lib().pllm_get_pipeline_output(C.byref(p), C.byref(n)), "getPipelineOutput")
    if n.value == 0:
        return np.zeros(0, np.int32)
    return np.ctypeslib.as_array(p, shape=(n.value,)).copy()


def finalize():
    _check(lib().pllm_finalize(), "finalize")
    _alive.clear()


def buildInputTokens(prev_output, keep_token_list, prefill_tokens) -> np.ndarray:
    prev = np.ascontiguousarray(prev_output, dtype=np.int32)
    keep = np.ascontiguousarray(keep_token_list, dtype=np.int32)
    pre = np.ascontiguousarray(prefill_tokens, dtype=np.int32)
    out = np.empty(len(keep) + len(pre) + 1, np.int32)
    n = lib().pllm_build_input_tokens(prev.ctypes.data_as(_i32p), len(prev), keep.ctypes.data_as(_i32p),
                                      len(keep), pre.ctypes.data_as(_i32p), len(pre),
                                      out.ctypes.data_as(_i32p))
    if n < 0:
        _check(n, "buildInputTokens")
    return out[:n]


def setProfiling(on: bool):
    _check(lib().pllm_set_profiling(int(on)), "setProfiling")


def getTimings() -> PipelineTimings:
    t = PipelineTimings()
    _check(lib().pllm_get_timings(C.byref(t)), "getTimings")
    return t


def resetTimings():
    _check(lib().pllm_reset_timings(), "resetTimings")


def debugBuffer(name: str):
    p, r, c = C.c_void_p(), C.c_int(), C.c_int()
    _check(lib().pllm_debug_buffer(name.encode(), C.byref(p), C.byref(r), C.byref(c)), "debugBuffer")
    return p.value, r.value, c.value
