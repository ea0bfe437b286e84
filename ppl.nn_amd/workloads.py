"""Seeded synthetic ragged batches for the dynamic-batching attention path (numpy only, no device code).

A `Batch` describes one call of MultiHeadCacheAttention the way the reference's harness would lay it out
(tools/benchmark_llama/generation_state.cc:60-192): decode sequences first, then prefill sequences; every
sequence owns a contiguous slab region starting at cachestarts[b].
"""
from dataclasses import dataclass, field

import numpy as np


@dataclass
class Batch:
    num_heads: int
    num_kv_heads: int
    head_dim: int
    seqlens: np.ndarray  # new tokens per sequence (int64 [B])
    start_pos: np.ndarray  # tokens already cached per sequence (int64 [B])
    decoding_batches: int
    num_layer: int = 1
    layer_idx: int = 0
    is_causal: int = 1
    slack_tokens: int = 0  # unused slab tokens left after each sequence's region
    name: str = ""
    cachestarts: np.ndarray = field(default=None)

    def __post_init__(self):
        self.seqlens = np.asarray(self.seqlens, dtype=np.int64)
        self.start_pos = np.asarray(self.start_pos, dtype=np.int64)
        assert self.seqlens.shape == self.start_pos.shape
        kv = self.kvlens
        if self.cachestarts is None:
            region = kv + self.slack_tokens
            self.cachestarts = np.concatenate([[0], np.cumsum(region)[:-1]]).astype(np.int64) if len(kv) else \
                np.zeros(0, np.int64)
        self.cachestarts = np.asarray(self.cachestarts, dtype=np.int64)

    @property
    def batch(self):
        return len(self.seqlens)

    @property
    def kvlens(self):
        return self.start_pos + self.seqlens

    @property
    def seqstarts(self):
        return np.concatenate([[0], np.cumsum(self.seqlens)]).astype(np.int64)

    @property
    def kvstarts(self):
        return np.concatenate([[0], np.cumsum(self.kvlens)]).astype(np.int64)

    @property
    def histstarts(self):
        return np.concatenate([[0], np.cumsum(self.start_pos)]).astype(np.int64)

    @property
    def total_new_tokens(self):
        return int(self.seqlens.sum())

    @property
    def total_hist_tokens(self):
        return int(self.start_pos.sum())

    @property
    def max_tokens(self):
        if self.batch == 0:
            return 1
        return int((self.cachestarts + self.kvlens + self.slack_tokens).max())

    @property
    def max_seqlen(self):
        return int(self.seqlens.max()) if self.batch else 0

    @property
    def max_kvlen(self):
        return int(self.kvlens.max()) if self.batch else 0

    # ---- algorithmic work (formulas the roofline figures are computed from) ----
    def decode_bytes(self):
        """HBM bytes a decode call must move: int8 K,V + fp16 scales of every cached token, Q, O, the new
        token's fp16 K,V read and its quantised write, and the tables."""
        nd = self.decoding_batches
        kv_tokens = int(self.kvlens[:nd].sum())
        per_tok = 2 * self.num_kv_heads * (self.head_dim + 2 * self.head_dim // 8)
        s = int(self.seqlens[:nd].sum())
        qo = 2 * s * self.num_heads * self.head_dim * 2
        cur = s * 2 * self.num_kv_heads * self.head_dim * 2
        wr = s * 2 * self.num_kv_heads * (self.head_dim + 2 * self.head_dim // 8)
        tables = (3 * nd + 2) * 8
        return kv_tokens * per_tok + qo + cur + wr + tables

    def prefill_flops(self):
        """4*H*Dh*sum_t (start_pos + t + 1) per prefill sequence (QK^T and PV, 2 flop/MAC, causal half only)."""
        nd = self.decoding_batches
        tot = 0
        for L, sp in zip(self.seqlens[nd:], self.start_pos[nd:]):
            L, sp = int(L), int(sp)
            keys = L * sp + L * (L + 1) // 2 if self.is_causal else L * (sp + L)
            tot += 4 * self.num_heads * self.head_dim * keys
        return tot


def _randn_f16(rng, shape):
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float16)
    step = 1 << 24
    for i in range(0, n, step):
        m = min(step, n - i)
        out[i:i + m] = rng.standard_normal(m, dtype=np.float32).astype(np.float16)
    return out.reshape(shape)


def make_tensors(b: Batch, seed: int):
    """fp16 N(0,1) tensors: query/current_key/current_value for the new tokens and hist_key/hist_value for the
    already-cached tokens (packed in batch order, histstarts)."""
    rng = np.random.default_rng(seed)
    S, Hs = b.total_new_tokens, b.total_hist_tokens
    return dict(
        query=_randn_f16(rng, (S, b.num_heads, b.head_dim)),
        current_key=_randn_f16(rng, (S, b.num_kv_heads, b.head_dim)),
        current_value=_randn_f16(rng, (S, b.num_kv_heads, b.head_dim)),
        hist_key=_randn_f16(rng, (Hs, b.num_kv_heads, b.head_dim)),
        hist_value=_randn_f16(rng, (Hs, b.num_kv_heads, b.head_dim)),
    )


def cfg1_llama2_7b_decode(seed=0, batch=64, lo=128, hi=2048):
    """64 decode sequences, H = KVH = 32, Dh 128, kv length (new token included) uniform in [128, 2048]."""
    rng = np.random.default_rng(seed)
    kv = rng.integers(lo, hi + 1, size=batch)
    return Batch(32, 32, 128, np.ones(batch, np.int64), kv - 1, batch, name="cfg1_llama2_7b_decode")


def cfg2_llama3_8b_mixed(seed=1, n_decode=120, n_prefill=8, dlo=256, dhi=4096, plo=64, phi=1024):
    """120 decode sequences (kv length uniform in [256, 4096]) packed first, then 8 causal prefill sequences
    (length uniform in [64, 1024]); H 32, KVH 8, Dh 128."""
    rng = np.random.default_rng(seed)
    kv = rng.integers(dlo, dhi + 1, size=n_decode)
    pl = rng.integers(plo, phi + 1, size=n_prefill)
    seqlens = np.concatenate([np.ones(n_decode, np.int64), pl])
    start = np.concatenate([kv - 1, np.zeros(n_prefill, np.int64)])
    return Batch(32, 8, 128, seqlens, start, n_decode, name="cfg2_llama3_8b_mixed")


def cfg2_decode_part(seed=1, **kw):
    b = cfg2_llama3_8b_mixed(seed, **kw)
    nd = b.decoding_batches
    return Batch(32, 8, 128, b.seqlens[:nd], b.start_pos[:nd], nd, name="cfg2_llama3_8b_decode_part")


def cfg2_prefill_part(seed=1, **kw):
    b = cfg2_llama3_8b_mixed(seed, **kw)
    nd = b.decoding_batches
    return Batch(32, 8, 128, b.seqlens[nd:], b.start_pos[nd:], 0, name="cfg2_llama3_8b_prefill_part")


def cfg3_long_context(seed=3, batch=8, lo=32768, hi=131072):
    """One GPU's share of Llama-3-70B under 8-way head sharding: 8 query heads, 1 KV head, batch 8."""
    rng = np.random.default_rng(seed)
    kv = rng.integers(lo, hi + 1, size=batch)
    return Batch(8, 1, 128, np.ones(batch, np.int64), kv - 1, batch, name="cfg3_long_context_decode")


class ChurnSchedule:
    """Continuous-batching churn (Llama-2-13B shape: H = KVH = 40): `num_slots` slots, each with a fixed slab
    region of `region` tokens. Every step each active sequence retires with probability `p_retire`; a freed
    (or empty) slot admits a new prompt with length uniform in [lo, hi]; everything else decodes one token."""

    def __init__(self, seed=2, num_slots=256, region=1024, p_retire=0.02, lo=32, hi=512):
        self.rng = np.random.default_rng(seed)
        self.num_slots, self.region, self.p, self.lo, self.hi = num_slots, region, p_retire, lo, hi
        self.kvlen = np.zeros(num_slots, np.int64)  # tokens cached before the coming step
        self.cachestart = (np.arange(num_slots, dtype=np.int64) * region)
        self.num_heads, self.num_kv_heads, self.head_dim = 40, 40, 128

    def next_step(self):
        """Returns (slot_kvlen, slot_newlen) for the coming step and advances the host copy of the state."""
        n = self.num_slots
        retire = (self.kvlen > 0) & (self.rng.random(n) < self.p)
        full = self.kvlen + 1 > self.region
        self.kvlen[retire | full] = 0
        newlen = np.ones(n, np.int64)
        fresh = self.kvlen == 0
        prompts = self.rng.integers(self.lo, self.hi + 1, size=n)
        newlen[fresh] = prompts[fresh]
        kv_before = self.kvlen.copy()
        self.kvlen = self.kvlen + newlen
        return kv_before, newlen
