"""Shared test plumbing: runs one MultiHeadCacheAttention call through the CPU oracle and through the HIP
library's C ABI on the same seeded inputs. torch is used only to own device memory and the stream."""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

pkg = entry.load_package()
from ppl_nn_amd import cabi, workloads  # noqa: E402,F401

ABS_TOL = 2e-3  # BASELINE.json: attention outputs within 2e-3 absolute / 1e-2 relative in fp16
REL_TOL = 1e-2
CACHE_FILL = 0x5A
SCALE_FILL = 0x3C00


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


class PagedLayout:
    """cache_mode 1: every sequence owns ceil(kvlen / page_size) pages scattered over the slab in a seeded random
    order; table[b, p] = first slab token of page p of sequence b (unused entries -1)."""

    def __init__(self, b, page_size=128, seed=0):
        kv = b.kvlens
        pages = (kv + page_size - 1) // page_size
        self.page_size = page_size
        self.max_pages = int(max(1, pages.max())) if len(pages) else 1
        total = int(pages.sum())
        order = np.random.default_rng(seed).permutation(total + 3)  # a few pages stay unused
        self.slab_tokens = (total + 3) * page_size
        self.table = np.full((b.batch, self.max_pages), -1, np.int64)
        k = 0
        for i, n in enumerate(pages):
            self.table[i, :n] = order[k:k + n] * page_size
            k += int(n)

    def token(self, i, j):
        return int(self.table[i, j // self.page_size] + j % self.page_size)


def _set_cache_mode(a, paged):
    a.cache_mode, a.page_size = (1, paged.page_size) if paged else (0, 128)
    a.cachestart_stride_b = paged.max_pages if paged else 0


def _strides(b, paged, layout):
    tokens = paged.slab_tokens if paged else b.max_tokens
    if layout == 3:
        return cabi.cache_strides_layout3(b.num_layer, b.num_kv_heads, b.head_dim, tokens)
    return cabi.cache_strides_layout0(b.num_layer, b.num_kv_heads, b.head_dim)


def new_slab(b, paged=None, layout=0):
    tokens = paged.slab_tokens if paged else b.max_tokens
    shape = (tokens, b.num_layer, 2, b.num_kv_heads, b.head_dim) if layout == 0 else \
        (b.num_layer, 2, b.num_kv_heads, tokens, b.head_dim)  # cache_layout 3
    cache = np.full(shape, CACHE_FILL, dtype=np.int8)
    scale = np.full(shape[:-1] + (b.head_dim // 8,), SCALE_FILL, dtype=np.uint16).view(np.float16)
    return cache, scale


def fill_write_args(w, b, key, value, seqstarts, start_pos, cachestarts, cache, scale, ptr=_ptr, paged=None, layout=0):
    st = _strides(b, paged, layout)
    w.d_current_key, w.d_current_value = ptr(key), ptr(value)
    w.d_seqstarts, w.d_cachestarts, w.d_start_pos = ptr(seqstarts), ptr(cachestarts), ptr(start_pos)
    w.batch, w.total_new_tokens = b.batch, int(key.shape[0])
    w.layer_idx, w.num_layer, w.num_kv_heads, w.head_dim = b.layer_idx, b.num_layer, b.num_kv_heads, b.head_dim
    for k, v in st.items():
        setattr(w, k, v)
    w.d_cache, w.d_scale = ptr(cache), ptr(scale)
    _set_cache_mode(w, paged)
    # the struct only holds raw addresses: keep the arrays (often temporaries such as b.histstarts) alive with it
    w._refs = getattr(w, "_refs", []) + [key, value, seqstarts, start_pos, cachestarts, cache, scale]
    return w


def _set_mask(a, mask, ptr):
    """mask: None, or an fp16 array / device tensor [tokens, keys] (all heads) or [heads, tokens, keys]."""
    if mask is None:
        a.d_attn_mask, a.attn_mask_stride_h, a.attn_mask_stride_q = None, 0, 0
        return
    a.d_attn_mask = ptr(mask)
    a.attn_mask_stride_q = int(mask.shape[-1])
    a.attn_mask_stride_h = int(mask.shape[-2]) * int(mask.shape[-1]) if len(mask.shape) == 3 else 0


def fill_mhca_args(a, b, q, k, v, seqstarts, kvstarts, cachestarts, start_pos, cache, scale, out, ptr=_ptr,
                   cache_prefill=0, split_k=1, paged=None, layout=0, mask=None):
    st = _strides(b, paged, layout)
    a.d_query, a.d_current_key, a.d_current_value = ptr(q), ptr(k), ptr(v)
    _set_mask(a, mask, ptr)
    a.d_alibi_slopes = None
    a.d_seqstarts, a.d_kvstarts = ptr(seqstarts), ptr(kvstarts)
    a.d_cachestarts, a.d_start_pos = ptr(cachestarts), ptr(start_pos)
    a.is_causal = b.is_causal
    a.batch, a.decoding_batches = b.batch, b.decoding_batches
    a.max_seqlen, a.max_kvlen = b.max_seqlen, b.max_kvlen
    a.layer_idx, a.num_layer = b.layer_idx, b.num_layer
    a.num_heads, a.num_kv_heads, a.head_dim = b.num_heads, b.num_kv_heads, b.head_dim
    for kk, vv in st.items():
        setattr(a, kk, vv)
    _set_cache_mode(a, paged)
    a.enable_cache_prefill = cache_prefill
    a.enable_decoding_sharemem_mhca = a.enable_decoding_infinity_mhca = a.enable_decoding_infinity_gqca = 1
    a.specify_decoding_attn_split_k = split_k
    a.specify_decoding_attn_tpb = 0
    a.d_cache, a.d_scale, a.d_output = ptr(cache), ptr(scale), ptr(out)
    a.total_new_tokens = b.total_new_tokens
    a._refs = [q, k, v, seqstarts, kvstarts, cachestarts, start_pos, cache, scale, out, mask]
    return a


def run_oracle(b, t, cache_prefill=0, want_f64=True, paged=None, layout=0, mask=None):
    """History write + MHCA on the CPU oracle. Returns cache (int8), scale (fp16), output (fp16), output_f64."""
    import oracle
    L = oracle.lib()
    cache, scale = new_slab(b, paged, layout)
    zeros = np.zeros(b.batch, np.int64)
    cs = np.ascontiguousarray(paged.table) if paged else b.cachestarts
    if b.total_hist_tokens:
        w = fill_write_args(cabi.KvWriteArgs(), b, t["hist_key"], t["hist_value"], b.histstarts, zeros,
                            cs, cache, scale, paged=paged, layout=layout)
        assert L.oracle_kv_quantize_write(C.byref(w)) == 0
    out = np.zeros((b.total_new_tokens, b.num_heads, b.head_dim), np.float16)
    out64 = np.zeros(out.shape, np.float64) if want_f64 else None
    seqstarts, kvstarts, sp = b.seqstarts, b.kvstarts, b.start_pos.copy()
    a = fill_mhca_args(cabi.MhcaArgs(), b, t["query"], t["current_key"], t["current_value"], seqstarts, kvstarts,
                       cs, sp, cache, scale, out, cache_prefill=cache_prefill, paged=paged, layout=layout, mask=mask)
    rc = L.oracle_mhca_forward(C.byref(a), _ptr(out64))
    assert rc == 0, rc
    return dict(cache=cache, scale=scale, output=out, output_f64=out64)


def dev_ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def to_dev(a):
    import torch
    if a.dtype == np.float16:
        return torch.from_numpy(a.view(np.int16).copy()).cuda().view(torch.float16)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run_device(b, t, cache_prefill=0, split_k=1, plan_out=None, paged=None, layout=0, staging=None, lib=None,
               mask=None, slab=None):
    """Same call through the C ABI on cuda:0. staging=0 clears plan.prefill_staging (the caller's way to keep a
    cache-prefill call on the kernel that reads the int8 slab itself). lib: another build of the kernel library than
    the product one. slab: (cache, scale) device tensors the caller made (a slab too large to mirror on the host);
    they are then inspected by the caller and not copied back."""
    import torch
    lib = lib or pkg.load_library()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    if slab is None:
        cache_h, scale_h = new_slab(b, paged, layout)
        cache, scale = to_dev(cache_h), to_dev(scale_h)
    else:
        cache, scale = slab
    d = {k: to_dev(v) for k, v in t.items()}
    tabs = dict(seqstarts=b.seqstarts, kvstarts=b.kvstarts,
                cachestarts=np.ascontiguousarray(paged.table) if paged else b.cachestarts, start_pos=b.start_pos,
                histstarts=b.histstarts, zeros=np.zeros(max(b.batch, 1), np.int64))
    dt = {k: to_dev(v) for k, v in tabs.items()}
    if b.total_hist_tokens:
        w = fill_write_args(cabi.KvWriteArgs(), b, d["hist_key"], d["hist_value"], dt["histstarts"], dt["zeros"],
                            dt["cachestarts"], cache, scale, ptr=dev_ptr, paged=paged, layout=layout)
        pkg.check(lib.pplhip_kv_quantize_write(C.byref(w), stream), "kv_quantize_write(history)")
    out = torch.zeros((b.total_new_tokens, b.num_heads, b.head_dim), dtype=torch.float16, device="cuda")
    a = fill_mhca_args(cabi.MhcaArgs(), b, d["query"], d["current_key"], d["current_value"], dt["seqstarts"],
                       dt["kvstarts"], dt["cachestarts"], dt["start_pos"], cache, scale, out, ptr=dev_ptr,
                       cache_prefill=cache_prefill, split_k=split_k, paged=paged, layout=layout,
                       mask=None if mask is None else to_dev(mask))
    plan = cabi.MhcaPlan()
    pkg.check(lib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)), "mhca_prepare")
    ws = torch.empty(max(int(plan.workspace_bytes), 256), dtype=torch.uint8, device="cuda")
    if staging is not None:
        assert staging == 0, "a plan can only be taken OFF the staged route"
        plan.prefill_staging = 0
    pkg.check(lib.pplhip_mhca_forward(C.byref(a), C.byref(plan), dev_ptr(ws), stream), "mhca_forward")
    torch.cuda.synchronize()
    if plan_out is not None:
        plan_out.append(plan)
    output = out.cpu().view(torch.int16).numpy().view(np.float16)
    if slab is not None:
        return dict(output=output)
    return dict(cache=cache.cpu().numpy(), scale=scale.cpu().view(torch.int16).numpy().view(np.float16), output=output)


def mha_inputs(b, t):
    """Packed fp16 key/value of every sequence (history rows then new rows) for MultiHeadAttention."""
    hs, ss = b.histstarts, b.seqstarts
    keys, values = [], []
    for i in range(b.batch):
        keys += [t["hist_key"][hs[i]:hs[i + 1]], t["current_key"][ss[i]:ss[i + 1]]]
        values += [t["hist_value"][hs[i]:hs[i + 1]], t["current_value"][ss[i]:ss[i + 1]]]
    shape = (0, b.num_kv_heads, b.head_dim)
    cat = lambda xs: np.ascontiguousarray(np.concatenate(xs)) if xs else np.zeros(shape, np.float16)
    return cat(keys), cat(values)


def fill_mha_args(a, b, q, key, value, seqstarts, kvstarts, out, ptr=_ptr, mask=None):
    a.d_query, a.d_key, a.d_value = ptr(q), ptr(key), ptr(value)
    _set_mask(a, mask, ptr)
    a.d_seqstarts, a.d_kvstarts = ptr(seqstarts), ptr(kvstarts)
    a.is_causal, a.is_alibi = b.is_causal, 0
    a.batch, a.decoding_batches = b.batch, b.decoding_batches
    a.max_seqlen, a.max_kvlen = b.max_seqlen, b.max_kvlen
    a.num_heads, a.num_kv_heads, a.head_dim = b.num_heads, b.num_kv_heads, b.head_dim
    a.d_output = ptr(out)
    a._refs = [q, key, value, seqstarts, kvstarts, out, mask]
    return a


def run_oracle_mha(b, q, key, value, mask=None):
    import oracle
    out = np.zeros((b.total_new_tokens, b.num_heads, b.head_dim), np.float16)
    out64 = np.zeros(out.shape, np.float64)
    a = fill_mha_args(cabi.MhaArgs(), b, q, key, value, b.seqstarts, b.kvstarts, out, mask=mask)
    rc = oracle.lib().oracle_mha_forward(C.byref(a), _ptr(out64))
    assert rc == 0, rc
    return dict(output=out, output_f64=out64)


def run_device_mha(b, q, key, value, mask=None):
    import torch
    lib = pkg.load_library()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    dq, dk, dv = to_dev(q), to_dev(key), to_dev(value)
    ss, ks = to_dev(b.seqstarts), to_dev(b.kvstarts)
    out = torch.zeros((b.total_new_tokens, b.num_heads, b.head_dim), dtype=torch.float16, device="cuda")
    a = fill_mha_args(cabi.MhaArgs(), b, dq, dk, dv, ss, ks, out, ptr=dev_ptr, mask=None if mask is None else to_dev(mask))
    pkg.check(lib.pplhip_mha_forward(C.byref(a), stream), "mha_forward")
    torch.cuda.synchronize()
    return dict(output=out.cpu().view(torch.int16).numpy().view(np.float16))


def fill_rope_args(a, q, k, seqlens, start_pos, q_out, k_out, theta=10000.0, rotary_dim=0, bypass_key=0,
                   scaling_type=0, scaling_factor=1.0, max_pos=2048, ptr=_ptr, tables=None, pair_layout=0):
    seqlens = np.asarray(seqlens, np.int64)
    ss = np.concatenate([[0], np.cumsum(seqlens)]).astype(np.int64)
    sp = np.asarray(start_pos, np.int64)
    if tables is not None:  # device copies supplied by the caller
        ss_arg, sp_arg = tables
    else:
        ss_arg, sp_arg = ss, sp
    a.d_query, a.d_key, a.d_start_pos, a.d_seqstarts = ptr(q), ptr(k), ptr(sp_arg), ptr(ss_arg)
    a.theta, a.bypass_key, a.rotary_dim, a.pair_layout = theta, bypass_key, rotary_dim, pair_layout
    a.batch, a.total_tokens = len(seqlens), int(ss[-1])
    a.num_heads, a.num_key_heads, a.head_dim = int(q.shape[1]), int(k.shape[1]), int(q.shape[2])
    a.max_position_embeddings, a.max_seqlen = max_pos, int(seqlens.max()) if len(seqlens) else 0
    a.scaling_type, a.scaling_factor = scaling_type, scaling_factor
    a.d_rotated_query, a.d_rotated_key = ptr(q_out), ptr(k_out)
    a._refs = [q, k, ss_arg, sp_arg, q_out, k_out]
    return a


def assert_attn_close(got_f16, ref_f64, abs_tol=ABS_TOL, rel_tol=REL_TOL, what="attention output"):
    got = got_f16.astype(np.float64)
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    err = np.abs(got - ref_f64)
    lim = abs_tol + rel_tol * np.abs(ref_f64)
    bad = err > lim
    if bad.any():
        i = np.unravel_index(np.argmax(err - lim), err.shape)
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.size} elements outside {abs_tol} abs + {rel_tol} rel; "
                             f"worst at {i}: got {got[i]}, want {ref_f64[i]}")
    return float(err.max())


def textbook_attention(q, k, v, causal_offset=None, mask=None):
    """float64 softmax(q k^T / sqrt(d) + mask) v for one head. q [Lq, d], k/v [Lk, d].
    causal_offset: query row i sees keys j <= causal_offset + i (None = no causal mask); mask: additive [Lq, Lk]."""
    q, k, v = (x.astype(np.float64) for x in (q, k, v))
    s = q @ k.T / np.sqrt(q.shape[-1])
    if mask is not None:
        s = s + mask.astype(np.float64)
    if causal_offset is not None:
        i = np.arange(q.shape[0])[:, None]
        j = np.arange(k.shape[0])[None, :]
        s = np.where(j <= causal_offset + i, s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    return p @ v
