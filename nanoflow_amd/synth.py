"""Synthetic workloads for the nano-batch pipeline: shapes, random-init weights and
iteration batches with a paged KV cache.

Mirrors what the reference builds for its own synthetic runs
(pipeline/src/vortexData.cu:61-204 ``createUpdateData`` and
pipeline/src/vortexData.cu:386-406 ``createModelWeight``), with seeded contents
instead of uninitialised memory so results can be compared.

Generators are numpy ``default_rng`` (PCG64) streams: seed+0 weights, seed+1
activations / KV contents, seed+2 lengths, seed+3 page permutation.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np


@dataclass
class ModelShape:
    hidden: int = 4096
    Hq: int = 32
    Hkv: int = 8
    d: int = 128
    ffn: int = 14336
    vocab: int = 128256
    layers: int = 32
    page_size: int = 16
    eps: float = 1e-5
    rope_theta: float = 5e5
    rope_scale: float = 1.0
    smooth_a: float = 0.0
    smooth_b: float = 0.0
    # the Llama-3.1 "rope_scaling" block of a model config (factor, low_freq_factor, high_freq_factor,
    # original_max_position_embeddings); when given, rope_scale / smooth_a / smooth_b are derived from
    # it as the pipeline's configuration does (pipeline/include/config.h:101-110)
    rope_scaling: dict | None = None

    def __post_init__(self):
        rs = self.rope_scaling
        if rs:
            lo, hi = float(rs["low_freq_factor"]), float(rs["high_freq_factor"])
            self.rope_scale = float(rs["factor"])
            self.smooth_a = float(rs["original_max_position_embeddings"]) / (2 * np.pi * hi - 2 * np.pi * lo)
            self.smooth_b = -1.0 / (hi / lo - 1.0)

    @property
    def kqv_n(self) -> int:
        return (self.Hq + 2 * self.Hkv) * self.d

    def as_dict(self) -> dict:
        return dict(self.__dict__)


LLAMA3_8B = ModelShape()
LLAMA3_70B = ModelShape(hidden=8192, Hq=64, Hkv=8, d=128, ffn=28672, vocab=128256, layers=80)


def tiny_shape(layers: int = 2, vocab: int = 1024, Hq: int = 8, Hkv: int = 2, ffn: int = 512,
               hidden: int | None = None) -> ModelShape:
    """Small shape with the real head_dim/page_size, for end-to-end parity checks.  The
    pipeline derives head_dim as hidden / Hq (as the reference does), so hidden = Hq * 128."""
    return ModelShape(hidden=Hq * 128 if hidden is None else hidden, Hq=Hq, Hkv=Hkv, d=128, ffn=ffn,
                      vocab=vocab, layers=layers)


def normal_f16(rng: np.random.Generator, shape, std: float = 1.0, mean: float = 0.0) -> np.ndarray:
    return (rng.standard_normal(shape, dtype=np.float32) * std + mean).astype(np.float16)


def make_weights(shape: ModelShape, seed: int = 0, layers: int | None = None, kqv_bias: bool = False) -> dict:
    """fp16 N(0, 0.02) weights in the reference's orientation (K x N row-major,
    KQV columns ordered K | V | Q; pipeline/utils/weightSaver.py:89-149).  kqv_bias adds the
    k | v | q bias rows of the bias pipelines, N(0, 0.5), drawn after everything else."""
    rng = np.random.default_rng(seed)
    L = shape.layers if layers is None else layers
    w = {
        "embedding": normal_f16(rng, (shape.vocab, shape.hidden), 0.02),
        "lm_head": normal_f16(rng, (shape.hidden, shape.vocab), 0.02),
        "model_norm": normal_f16(rng, (shape.hidden,), 0.02, 1.0),
        "w_kqv": [], "w_o": [], "w_gate": [], "w_up": [], "w_down": [], "ln_attn": [], "ln_ffn": [],
    }
    for _ in range(L):
        w["w_kqv"].append(normal_f16(rng, (shape.hidden, shape.kqv_n), 0.02))
        w["w_o"].append(normal_f16(rng, (shape.Hq * shape.d, shape.hidden), 0.02))
        w["w_gate"].append(normal_f16(rng, (shape.hidden, shape.ffn), 0.02))
        w["w_up"].append(normal_f16(rng, (shape.hidden, shape.ffn), 0.02))
        w["w_down"].append(normal_f16(rng, (shape.ffn, shape.hidden), 0.02))
        w["ln_attn"].append(normal_f16(rng, (shape.hidden,), 0.02, 1.0))
        w["ln_ffn"].append(normal_f16(rng, (shape.hidden,), 0.02, 1.0))
    if kqv_bias:
        w["b_kqv"] = [normal_f16(rng, (shape.kqv_n,), 0.5) for _ in range(L)]
    return w


@dataclass
class Batch:
    """One iteration's update data (pipeline/include/vortexData.cuh:55-90), host side."""
    decodePrefillBorder: int
    prefillNum: int
    prefillTokensNum: int
    input_tokens: np.ndarray
    input_indptr: np.ndarray
    rev_input_indptr: np.ndarray
    per_token_offset: np.ndarray
    kv_indptr: np.ndarray
    kv_indices: np.ndarray
    kv_last_page_len: np.ndarray
    kv_len: np.ndarray            # per request, after this iteration's append
    num_pages: int                # pool size the page ids were drawn from
    keep_token_list: np.ndarray = field(default_factory=lambda: np.zeros(0, np.int32))

    @property
    def tokens(self) -> int:
        return self.decodePrefillBorder + self.prefillTokensNum

    @property
    def req_num(self) -> int:
        return self.decodePrefillBorder + self.prefillNum

    def as_dict(self) -> dict:
        return {k: getattr(self, k) for k in (
            "decodePrefillBorder", "prefillNum", "prefillTokensNum", "input_tokens", "input_indptr",
            "rev_input_indptr", "per_token_offset", "kv_indptr", "kv_indices", "kv_last_page_len")}


def make_batch(decode_kv_lens, prefill_chunks, vocab: int, page_size: int = 16, seed: int = 0,
               extra_pages: int = 0, permute: bool = True) -> Batch:
    """decode_kv_lens[i]: KV length of decode request i BEFORE this step (the new token
    lands at that position).  prefill_chunks: list of (prev_len, chunk_len).  Page ids are
    a random permutation of the pool (seed+3) unless ``permute`` is False."""
    rng_len = np.random.default_rng(seed + 2)
    rng_perm = np.random.default_rng(seed + 3)
    decode_kv_lens = [int(x) for x in decode_kv_lens]
    nd = len(decode_kv_lens)
    qo_lens = [1] * nd + [int(c) for _, c in prefill_chunks]
    prev = decode_kv_lens + [int(p) for p, _ in prefill_chunks]
    kv_len = np.array([p + q for p, q in zip(prev, qo_lens)], np.int32)
    pages_per_req = (kv_len + page_size - 1) // page_size
    total_pages = int(pages_per_req.sum())
    pool = total_pages + extra_pages
    page_ids = rng_perm.permutation(pool).astype(np.int32) if permute else np.arange(pool, dtype=np.int32)
    kv_indices = page_ids[:total_pages].copy()
    kv_indptr = np.zeros(len(kv_len) + 1, np.int32)
    kv_indptr[1:] = np.cumsum(pages_per_req)
    kv_last = ((kv_len - 1) % page_size + 1).astype(np.int32)
    input_indptr = np.zeros(len(qo_lens) + 1, np.int32)
    input_indptr[1:] = np.cumsum(qo_lens)
    T = int(input_indptr[-1])
    rev = np.repeat(np.arange(len(qo_lens), dtype=np.int32), qo_lens)
    off = np.concatenate([np.arange(q, dtype=np.int32) + p for p, q in zip(prev, qo_lens)]) \
        if T else np.zeros(0, np.int32)
    tokens = rng_len.integers(0, vocab, size=T, dtype=np.int32)
    return Batch(decodePrefillBorder=nd, prefillNum=len(prefill_chunks),
                 prefillTokensNum=T - nd, input_tokens=tokens, input_indptr=input_indptr,
                 rev_input_indptr=rev.astype(np.int32), per_token_offset=off.astype(np.int32),
                 kv_indptr=kv_indptr, kv_indices=kv_indices, kv_last_page_len=kv_last,
                 kv_len=kv_len, num_pages=pool,
                 keep_token_list=np.ones(nd, np.int32))


def config1_batch(seed: int = 0, n_decode: int = 64, lo: int = 512, hi: int = 1024,
                  vocab: int = 128256) -> Batch:
    """64 decode tokens, KV length uniform in [lo, hi], permuted page table."""
    rng = np.random.default_rng(seed + 2)
    lens = rng.integers(lo, hi + 1, size=n_decode)
    return make_batch(lens, [], vocab, seed=seed)


def config2_batch(seed: int = 0, n_decode: int = 1792, lo: int = 1024, hi: int = 1536,
                  prefill_chunk: int = 256, prefill_prev: int = 0, vocab: int = 128256) -> Batch:
    """One dense 2048-token iteration: 1792 decode tokens + one 256-token prefill chunk."""
    rng = np.random.default_rng(seed + 2)
    lens = rng.integers(lo, hi + 1, size=n_decode)
    return make_batch(lens, [(prefill_prev, prefill_chunk)], vocab, seed=seed)


def kv_pool_elems(num_pages: int, shape: ModelShape) -> int:
    return num_pages * 2 * shape.page_size * shape.Hkv * shape.d


def make_kv_pool(num_pages: int, shape: ModelShape, rng: np.random.Generator) -> np.ndarray:
    """One layer's pool [pages, 2, page_size, Hkv, d] fp16 N(0,1)
    (pipeline/include/vortexData.cuh:39)."""
    return normal_f16(rng, (num_pages, 2, shape.page_size, shape.Hkv, shape.d), 1.0)


def gemv_batch_split(decode_num: int, kqv1: int, nano1: int, kqv3: int):
    """Split of the decode requests over the four decode-attention launches
    (pipeline/utils/serve_8B.py:391-394)."""
    g0 = min(decode_num, kqv1)
    g1 = min(decode_num - g0, nano1 - kqv1)
    g2 = min(decode_num - g0 - g1, kqv3)
    g3 = decode_num - g0 - g1 - g2
    return [g0, g1, g2, g3]
