"""Python face of the pipeline control plane (C ABI: include/nanoflow_pllm.h).

Keeps the names of the reference's pybind11 module ``pllm_python``
(pipeline/src/pybind.cu:189-284): ``setRank``, ``setModelConfig``, ``init``, ``config``,
``update``, ``run``, ``run_async``, ``run_async_wait``, ``getPipelineOutput``, ``finalize``,
the ``Vortex*`` data classes and ``PipelineType``.  Raw addresses are passed as integers, as
in the reference (``setPtr``, ``setKVIndices`` ...).

There is no fallback: a missing ``libnf_pipeline.so`` raises.
"""
from __future__ import annotations

import atexit
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

    @property
    def has_kqv_bias(self) -> bool:
        """The three bias types (pipeline/src/computeBound.cu:234-242): B_KQV is added by the QKV GEMMs."""
        return self in (PipelineType.KQVBIAS, PipelineType.NONOVERLAP_KQVBIAS, PipelineType.NANOBATCH_KQVBIAS)

    @property
    def is_sequential(self) -> bool:
        """One stream, no nano-batch split: four GEMM tags, one decode-attention group."""
        return self in (PipelineType.NON_OVERLAP_LOCAL, PipelineType.NONOVERLAP_KQVBIAS, PipelineType.NONOVERLAP)

    @property
    def is_four_way(self) -> bool:
        """The reference's main Pipeline: QKV / RoPE-append / decode attention as four nano-batches, nine
        GEMM tags (O1, O2, D1, D2, KQV1-4, LOGITS)."""
        return self in (PipelineType.PLLM, PipelineType.NANOBATCH, PipelineType.PLLMOFFLOAD, PipelineType.KQVBIAS,
                        PipelineType.NANOBATCH_KQVBIAS)

    @property
    def gemm_tags(self) -> int:
        return 4 if self.is_sequential else 9 if self.is_four_way else 7


# serve_configs.pipeline_type of the reference's pipeline files (pipeline/utils/serve_8B.py:48-59).
# PLLM, NANOBATCH, PLLM_OFFLOAD and the nano-batched bias types run the reference's main schedule (four
# QKV / attention nano-batches) without its exchange steps; NON_OVERLAP runs as NON_OVERLAP_LOCAL.
pipeline_map = {
    "LOCAL": PipelineType.LOCAL,
    "PLLM": PipelineType.PLLM,
    "NON_OVERLAP": PipelineType.NONOVERLAP,
    "NANOBATCH": PipelineType.NANOBATCH,
    "PLLM_OFFLOAD": PipelineType.PLLMOFFLOAD,
    "NON_OVERLAP_LOCAL": PipelineType.NON_OVERLAP_LOCAL,
    "NANOBATCH_LOCAL": PipelineType.NANOBATCH_LOCAL,
    "KQVBIAS": PipelineType.KQVBIAS,
    "NANOBATCH_KQVBIAS": PipelineType.NANOBATCH_KQVBIAS,
    "NONOVERLAP_KQVBIAS": PipelineType.NONOVERLAP_KQVBIAS,
}


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
                ("prefill_attn_launches", C.c_long), ("gemm_ms", C.c_double),
                ("gemm_launches", C.c_long), ("gemm_flop", C.c_double), ("layer_stride", C.c_int)]


SYMBOLS = [
    "pllm_last_error", "pllm_set_model_config", "pllm_set_rank", "pllm_tmp_buffer_halves",
    "pllm_max_page_num", "pllm_init", "pllm_model_weight_to_gpu", "pllm_create_model_weight",
    "pllm_create_init_data", "pllm_config", "pllm_update",
    "pllm_run", "pllm_run_async", "pllm_run_async_wait", "pllm_get_pipeline_output",
    "pllm_finalize", "pllm_build_input_tokens", "pllm_set_profiling", "pllm_set_profiling_stride", "pllm_get_timings",
    "pllm_reset_timings", "pllm_debug_buffer", "pllm_set_graph_mode", "pllm_get_graph_counters",
    "pllm_set_weight_format", "pllm_get_weight_format", "pllm_e4m3_weight_bytes", "pllm_e4m3_weight_scale_offset",
    "pllm_quantize_weight_e4m3",
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
        atexit.register(l.pllm_finalize)   # a pipeline left open must not keep the process alive
        l.pllm_last_error.restype = C.c_char_p
        l.pllm_set_model_config.argtypes = [C.c_char_p]
        l.pllm_set_rank.argtypes = [C.c_int, C.c_int]
        l.pllm_tmp_buffer_halves.restype = C.c_size_t
        l.pllm_max_page_num.restype = C.c_size_t
        l.pllm_init.argtypes = [C.POINTER(_CInitData), C.c_int]
        l.pllm_model_weight_to_gpu.argtypes = [C.POINTER(_CModelWeight), C.POINTER(_CModelWeight),
                                               C.POINTER(VortexLayerWeight)]
        l.pllm_create_model_weight.argtypes = [C.POINTER(_CModelWeight), C.POINTER(VortexLayerWeight), C.c_int]
        l.pllm_create_init_data.argtypes = [C.POINTER(_CInitData), C.POINTER(C.c_void_p), C.c_int,
                                            C.POINTER(_CModelWeight)]
        l.pllm_config.argtypes = [C.POINTER(_CConfigData)]
        l.pllm_update.argtypes = [C.POINTER(_CUpdateData)]
        l.pllm_get_pipeline_output.argtypes = [C.POINTER(_i32p), C.POINTER(C.c_int)]
        l.pllm_build_input_tokens.argtypes = [_i32p, C.c_int, _i32p, C.c_int, _i32p, C.c_int, _i32p]
        l.pllm_set_profiling.argtypes = [C.c_int]
        l.pllm_set_weight_format.argtypes = [C.c_int]
        l.pllm_e4m3_weight_bytes.restype = C.c_size_t
        l.pllm_e4m3_weight_bytes.argtypes = [C.c_int, C.c_int]
        l.pllm_e4m3_weight_scale_offset.restype = C.c_size_t
        l.pllm_e4m3_weight_scale_offset.argtypes = [C.c_int, C.c_int]
        l.pllm_quantize_weight_e4m3.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
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


_MAX_LAYERS = 1024


def createModelWeight(weight: VortexModelWeight, rank: int = 0):
    """pllm_python.createModelWeight (pybind.cu:228): device memory for every weight of the configured
    model; fills ``weight`` in place.  The memory lives until the process ends, as in the reference."""
    if rank != 0:
        raise NanoflowPipelineError("this build runs one rank")
    layers = (VortexLayerWeight * _MAX_LAYERS)()
    c = _CModelWeight()
    _check(lib().pllm_create_model_weight(C.byref(c), layers, _MAX_LAYERS), "createModelWeight")
    weight.lm_head, weight.embedding, weight.model_layernorm = c.lm_head, c.embedding, c.model_layernorm
    weight.layer_weight = [layers[i] for i in range(c.num_layers)]
    weight._keep = layers


def createInitData(data: "VortexInitData", weight: VortexModelWeight, rank: int = 0):
    """pllm_python.createInitData (pybind.cu:229): tmp buffer and zeroed per-layer KV pools for the
    configured model around ``weight``; fills ``data`` in place (never freed, as in the reference)."""
    if rank != 0:
        raise NanoflowPipelineError("this build runs one rank")
    cw, keep = weight._to_c()
    kv = (C.c_void_p * _MAX_LAYERS)()
    c = _CInitData()
    _check(lib().pllm_create_init_data(C.byref(c), kv, _MAX_LAYERS, C.byref(cw)), "createInitData")
    data.setKVdata([kv[i] for i in range(cw.num_layers)])
    data.setWeight(weight, c.weight_size)
    data.setTmpBuffer(c.tmp_buffer, c.tmp_buffer_size)
    data._keep = (keep, kv)


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


class WeightFormat(enum.IntEnum):
    """Storage of the five per-layer GEMM weights in the init data (include/nanoflow_pllm.h)."""
    F16 = 0
    E4M3 = 1


def setWeightFormat(fmt):
    """Call before init.  E4M3: VortexWeight.ptr of W_KQV, W_O1/W_O2, W_G, W_U, W_D points at N*K e4m3
    bytes [N][K] + N fp32 scales (e4m3WeightBytes / quantizeWeightE4M3)."""
    _check(lib().pllm_set_weight_format(int(fmt)), "setWeightFormat")


def getWeightFormat() -> WeightFormat:
    return WeightFormat(lib().pllm_get_weight_format())


def e4m3WeightBytes(N: int, K: int) -> int:
    return int(lib().pllm_e4m3_weight_bytes(N, K))


def e4m3WeightScaleOffset(N: int, K: int) -> int:
    return int(lib().pllm_e4m3_weight_scale_offset(N, K))


def quantizeWeightE4M3(w_f16_ptr: int, out_ptr: int, N: int, K: int, stream: int = 0):
    """Device fp16 [K][N] weight -> the E4M3 form at out_ptr (e4m3WeightBytes(N, K) bytes)."""
    _check(lib().pllm_quantize_weight_e4m3(w_f16_ptr, out_ptr, N, K, stream), "quantizeWeightE4M3")


def setProfilingStride(stride: int):
    """Time every stride-th launch of each operator (0 = automatic); call before setProfiling / init."""
    _check(lib().pllm_set_profiling_stride(int(stride)), "setProfilingStride")


def setProfiling(level):
    """0/False: off; 1/True: attention launches are timed; 2: dense GEMM launches as well."""
    _check(lib().pllm_set_profiling(int(level)), "setProfiling")


def setGraphMode(on: bool):
    """Replay iterations from captured hipGraphs (one per launch signature)."""
    _check(lib().pllm_set_graph_mode(int(bool(on))), "setGraphMode")


def getGraphCounters() -> dict:
    c = (C.c_long * 3)()
    _check(lib().pllm_get_graph_counters(c), "getGraphCounters")
    return dict(eager=c[0], captured=c[1], replayed=c[2])


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


# ---------------------------------------------------------------- batch former / serve loop

class ServeStats(C.Structure):
    _fields_ = [("cycles", C.c_int), ("retired", C.c_int), ("wall_s", C.c_double),
                ("tokens_per_s", C.c_double), ("cycle_ms", C.c_double), ("form_ms", C.c_double),
                ("wait_ms", C.c_double), ("update_ms", C.c_double), ("gpu_iter_ms", C.c_double),
                ("tokens_processed", C.c_longlong)]


SYMBOLS += [
    "pllm_sched_create", "pllm_sched_destroy", "pllm_sched_add_request", "pllm_sched_schedule",
    "pllm_sched_form", "pllm_sched_harvest", "pllm_sched_advance", "pllm_sched_state",
    "pllm_sched_retired_output", "pllm_sched_retired_info", "pllm_sched_future_page_usage", "pllm_serve",
]


def _sched_lib():
    l = lib()
    if not getattr(l, "_sched_declared", False):
        l.pllm_sched_create.restype = C.c_void_p
        l.pllm_sched_create.argtypes = [C.c_int] * 8
        l.pllm_sched_destroy.restype = None
        l.pllm_sched_destroy.argtypes = [C.c_void_p]
        l.pllm_sched_add_request.argtypes = [C.c_void_p, C.c_int, _i32p, C.c_int, C.c_int, C.c_double]
        l.pllm_sched_schedule.argtypes = [C.c_void_p]
        l.pllm_sched_form.argtypes = [C.c_void_p, C.POINTER(_CUpdateData)]
        l.pllm_sched_harvest.argtypes = [C.c_void_p, _i32p, C.c_int]
        l.pllm_sched_advance.argtypes = [C.c_void_p, C.c_double, C.c_int, C.POINTER(C.c_int)]
        l.pllm_sched_state.argtypes = [C.c_void_p, C.POINTER(C.c_int * 5)]
        l.pllm_sched_retired_output.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_int), _i32p, C.c_int]
        l.pllm_sched_retired_info.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int),
                                              C.POINTER(C.c_int), C.POINTER(C.c_double * 4)]
        l.pllm_sched_future_page_usage.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.c_int]
        l.pllm_serve.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.POINTER(ServeStats)]
        l._sched_declared = True
    return l


class BatchFormer:
    """The C++ batch former (scheduler + paged-KV bookkeeping) behind the C ABI."""

    def __init__(self, kv_pages, page_size, global_bsz, nano1, kqv1, kqv3, avg_prefill, avg_decode):
        self._l = _sched_lib()
        self._h = self._l.pllm_sched_create(kv_pages, page_size, global_bsz, nano1, kqv1, kqv3,
                                            avg_prefill, avg_decode)
        if not self._h:
            raise NanoflowPipelineError(self._l.pllm_last_error().decode())

    def close(self):
        if self._h:
            self._l.pllm_sched_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def add_request(self, req_idx, prompt, output_len, start_time=0.0):
        p = np.ascontiguousarray(prompt, dtype=np.int32)
        _check(self._l.pllm_sched_add_request(self._h, req_idx, p.ctypes.data_as(_i32p), len(p),
                                              output_len, start_time), "sched_add_request")

    def schedule(self):
        _check(self._l.pllm_sched_schedule(self._h), "sched_schedule")

    def form(self) -> dict:
        """Forms the next batch; returns copies of its arrays (numpy int32) and scalars."""
        u = _CUpdateData()
        _check(self._l.pllm_sched_form(self._h, C.byref(u)), "sched_form")
        req = u.decodePrefillBorder + u.prefillNum
        tok = u.decodePrefillBorder + u.prefillTokensNum

        def arr(addr, n):
            if n == 0 or not addr:
                return np.zeros(0, np.int32)
            return np.ctypeslib.as_array(C.cast(addr, _i32p), shape=(n,)).copy()

        kv_indptr = arr(u.kv_indptr, req + 1)
        return dict(decodePrefillBorder=u.decodePrefillBorder, prefillNum=u.prefillNum,
                    prefillTokensNum=u.prefillTokensNum, keepTokenListLength=u.keepTokenListLength,
                    input_tokens=arr(u.input_tokens, u.prefillTokensNum),
                    input_indptr=arr(u.input_indptr, req + 1),
                    rev_input_indptr=arr(u.rev_input_indptr, tok),
                    per_token_offset=arr(u.per_token_offset, tok), kv_indptr=kv_indptr,
                    kv_indices=arr(u.kv_indices, int(kv_indptr[-1]) if len(kv_indptr) else 0),
                    kv_last_page_len=arr(u.kv_last_page_len, req),
                    keep_token_list=arr(u.keep_token_list, u.keepTokenListLength),
                    gemv_batch_size=arr(u.gemv_batch_size, 4))

    def harvest(self, ids):
        a = np.ascontiguousarray(ids, dtype=np.int32)
        _check(self._l.pllm_sched_harvest(self._h, a.ctypes.data_as(_i32p), len(a)), "sched_harvest")

    def advance(self, now=0.0, placeholder_zero=False) -> int:
        n = C.c_int()
        _check(self._l.pllm_sched_advance(self._h, now, int(placeholder_zero), C.byref(n)), "sched_advance")
        return n.value

    def state(self) -> dict:
        c = (C.c_int * 5)()
        _check(self._l.pllm_sched_state(self._h, C.byref(c)), "sched_state")
        return dict(queued=c[0], decoding=c[1], prefilling=c[2], free_pages=c[3], retired=c[4])

    def retired_output(self, which, cap=65536):
        out = np.empty(cap, np.int32)
        idx = C.c_int()
        n = self._l.pllm_sched_retired_output(self._h, which, C.byref(idx), out.ctypes.data_as(_i32p), cap)
        if n < 0:
            _check(n, "sched_retired_output")
        return idx.value, out[:n].copy()

    def retired_info(self, which) -> dict:
        idx, il, ol, t = C.c_int(), C.c_int(), C.c_int(), (C.c_double * 4)()
        _check(self._l.pllm_sched_retired_info(self._h, which, C.byref(idx), C.byref(il), C.byref(ol), C.byref(t)),
               "sched_retired_info")
        return dict(req_idx=idx.value, input_len=il.value, output_len=ol.value, request_comein_time=t[0],
                    encode_latency=t[1], decode_start_at=t[2], decode_latency=t[3])

    def future_page_usage(self):
        n = self._l.pllm_sched_future_page_usage(self._h, None, 0)
        out = np.empty(n, np.int64)
        self._l.pllm_sched_future_page_usage(self._h, out.ctypes.data_as(C.POINTER(C.c_int64)), n)
        return out

    def serve(self, skip_cycles, run_cycles, warmup_cycles=0) -> ServeStats:
        st = ServeStats()
        _check(self._l.pllm_serve(self._h, skip_cycles, warmup_cycles, run_cycles, C.byref(st)), "serve")
        return st
