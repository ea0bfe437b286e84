"""Pins oracle_mhca_forward / oracle_kv_cache_forward / oracle_mha_forward against a float64 textbook
softmax(QK^T/sqrt(d)+mask)V and closed forms, so a dropped term, wrong index or transposed operand fails."""
import ctypes as C

import numpy as np
import pytest

import harness
from harness import cabi, workloads


def dequant_slab(cache, scale):
    return cache.astype(np.float64) * np.repeat(scale.astype(np.float64), 8, axis=-1)


def textbook_batch(b, t, res, cache_prefill=0):
    """Expected outputs from the oracle's own slab (dequantised independently in numpy) and fp16 tensors."""
    deq = dequant_slab(res["cache"], res["scale"])
    out = np.zeros((b.total_new_tokens, b.num_heads, b.head_dim))
    rep = b.num_heads // b.num_kv_heads
    ss = b.seqstarts
    for i in range(b.batch):
        s0, L, sp, kv = ss[i], b.seqlens[i], b.start_pos[i], b.kvlens[i]
        for h in range(b.num_heads):
            kvh = h // rep
            if i < b.decoding_batches or cache_prefill:
                rows = slice(b.cachestarts[i], b.cachestarts[i] + kv)
                k, v = deq[rows, b.layer_idx, 0, kvh], deq[rows, b.layer_idx, 1, kvh]
            else:
                k, v = t["current_key"][s0:s0 + L, kvh], t["current_value"][s0:s0 + L, kvh]
            out[s0:s0 + L, h] = harness.textbook_attention(
                t["query"][s0:s0 + L, h], k, v, causal_offset=sp if b.is_causal else None)
    return out


@pytest.mark.parametrize("H,KVH,Dh,L,li", [(4, 4, 128, 1, 0), (8, 2, 128, 2, 1), (6, 1, 64, 3, 2)])
def test_mixed_batch_vs_textbook(H, KVH, Dh, L, li):
    b = workloads.Batch(H, KVH, Dh, [1, 1, 1, 9, 33, 1], [40, 1, 17, 0, 0, 0], 3, num_layer=L, layer_idx=li,
                        slack_tokens=3)
    t = workloads.make_tensors(b, seed=H * 100 + KVH)
    res = harness.run_oracle(b, t)
    want = textbook_batch(b, t, res)
    assert np.abs(res["output_f64"] - want).max() < 1e-12
    assert np.array_equal(res["output"], want.astype(np.float32).astype(np.float16))
    # other layers and the slack tokens keep their fill pattern
    other = [l for l in range(L) if l != li]
    assert (res["cache"][:, other] == harness.CACHE_FILL).all()
    for i in range(b.batch):
        end = b.cachestarts[i] + b.kvlens[i]
        assert (res["cache"][end:end + b.slack_tokens] == harness.CACHE_FILL).all()


def test_cache_prefill_and_chunked_start_pos():
    b = workloads.Batch(4, 2, 128, [1, 20, 7], [12, 30, 0], 1, num_layer=1)
    t = workloads.make_tensors(b, seed=9)
    res = harness.run_oracle(b, t, cache_prefill=1)
    want = textbook_batch(b, t, res, cache_prefill=1)
    assert np.abs(res["output_f64"] - want).max() < 1e-12


def test_non_causal():
    b = workloads.Batch(2, 2, 64, [5, 8], [0, 0], 0, is_causal=0)
    t = workloads.make_tensors(b, seed=4)
    res = harness.run_oracle(b, t)
    assert np.abs(res["output_f64"] - textbook_batch(b, t, res)).max() < 1e-12


def test_closed_forms():
    # kvlen == 1: output is exactly the (dequantised) value row
    b = workloads.Batch(4, 2, 128, [1, 1], [0, 0], 0)
    t = workloads.make_tensors(b, seed=1)
    res = harness.run_oracle(b, t)
    for s in range(2):
        for h in range(4):
            assert np.array_equal(res["output"][s, h], t["current_value"][s, h // 2])
    # all keys equal -> uniform softmax -> mean of values (prefill, non causal)
    b = workloads.Batch(2, 1, 64, [6], [0], 0, is_causal=0)
    t = workloads.make_tensors(b, seed=2)
    t["current_key"][:] = t["current_key"][0]
    res = harness.run_oracle(b, t)
    mean = t["current_value"][:, 0].astype(np.float64).mean(axis=0)
    assert np.abs(res["output_f64"][:, 0] - mean).max() < 1e-12
    # one dominant key: q = 30*k_3 direction makes key 3 win by a huge margin
    b = workloads.Batch(1, 1, 128, [1], [7], 1)
    t = workloads.make_tensors(b, seed=3)
    t["hist_key"][3, 0] = np.float16(4.0)
    t["query"][0, 0] = np.float16(8.0)
    t["hist_key"][[0, 1, 2, 4, 5, 6], 0] = np.float16(-4.0)
    t["current_key"][0, 0] = np.float16(-4.0)
    res = harness.run_oracle(b, t)
    deq = dequant_slab(res["cache"], res["scale"])
    assert np.abs(res["output_f64"][0, 0] - deq[3, 0, 1, 0]).max() < 1e-9


def test_gqa_equals_mha_with_repeated_heads():
    bg = workloads.Batch(8, 2, 128, [1, 11], [25, 0], 1)
    tg = workloads.make_tensors(bg, seed=21)
    rg = harness.run_oracle(bg, tg)
    bm = workloads.Batch(8, 8, 128, [1, 11], [25, 0], 1)
    tm = dict(tg)
    for k in ("current_key", "current_value", "hist_key", "hist_value"):
        tm[k] = np.ascontiguousarray(np.repeat(tg[k], 4, axis=1))
    rm = harness.run_oracle(bm, tm)
    assert np.array_equal(rg["output"], rm["output"])


def test_decode_equals_last_row_of_cache_prefill_and_permutation():
    # decode over history == last row of a causal prefill that reads the same cache
    bd = workloads.Batch(4, 2, 128, [1], [29], 1)
    t = workloads.make_tensors(bd, seed=31)
    rd = harness.run_oracle(bd, t)
    bp = workloads.Batch(4, 2, 128, [30], [0], 0)
    tp = dict(
        query=np.concatenate([np.zeros((29, 4, 128), np.float16), t["query"]]),
        current_key=np.concatenate([t["hist_key"], t["current_key"]]),
        current_value=np.concatenate([t["hist_value"], t["current_value"]]),
        hist_key=np.zeros((0, 2, 128), np.float16), hist_value=np.zeros((0, 2, 128), np.float16))
    rp = harness.run_oracle(bp, tp, cache_prefill=1)
    assert np.array_equal(rp["cache"], rd["cache"])
    assert np.abs(rp["output_f64"][29] - rd["output_f64"][0]).max() < 1e-12
    # permuting the sequences permutes the outputs
    b1 = workloads.Batch(4, 4, 64, [1, 1, 1], [5, 9, 2], 3)
    t1 = workloads.make_tensors(b1, seed=32)
    r1 = harness.run_oracle(b1, t1)
    perm = [2, 0, 1]
    b2 = workloads.Batch(4, 4, 64, [1, 1, 1], b1.start_pos[perm], 3)
    hs = b1.histstarts
    t2 = {k: t1[k][perm] for k in ("query", "current_key", "current_value")}
    for k in ("hist_key", "hist_value"):
        t2[k] = np.concatenate([t1[k][hs[i]:hs[i + 1]] for i in perm])
    r2 = harness.run_oracle(b2, t2)
    assert np.array_equal(r2["output"], r1["output"][perm])


def test_causal_ignores_future_tokens():
    b = workloads.Batch(2, 1, 64, [10], [0], 0)
    t = workloads.make_tensors(b, seed=41)
    r0 = harness.run_oracle(b, t)
    t2 = {k: v.copy() for k, v in t.items()}
    t2["current_key"][6:] = np.nan
    t2["current_value"][6:] = np.nan
    r1 = harness.run_oracle(b, t2)
    assert np.array_equal(r0["output"][:6], r1["output"][:6])


def test_kv_cache_op(olib):
    b = workloads.Batch(4, 2, 128, [1, 6, 1], [9, 0, 3], 0, num_layer=2, layer_idx=1, slack_tokens=2)
    t = workloads.make_tensors(b, seed=51)
    cache, scale = harness.new_slab(b)
    zeros = np.zeros(b.batch, np.int64)
    w = harness.fill_write_args(cabi.KvWriteArgs(), b, t["hist_key"], t["hist_value"], b.histstarts, zeros,
                                b.cachestarts, cache, scale)
    assert olib.oracle_kv_quantize_write(C.byref(w)) == 0
    a = cabi.KvCacheArgs()
    seqstarts, kvstarts, sp = b.seqstarts, b.kvstarts, b.start_pos
    harness.fill_write_args(a.write, b, t["current_key"], t["current_value"], seqstarts, sp, b.cachestarts, cache,
                            scale)
    a.d_kvstarts = kvstarts.ctypes.data
    a._refs2 = [kvstarts]
    a.total_kv_tokens, a.max_kvlen = int(kvstarts[-1]), b.max_kvlen
    a.num_repeat, a.cache_mode, a.cache_layout = 1, 0, 0
    ko = np.zeros((int(kvstarts[-1]), 2, 128), np.float16)
    vo = np.zeros_like(ko)
    a.d_key_out, a.d_value_out = ko.ctypes.data, vo.ctypes.data
    assert olib.oracle_kv_cache_forward(C.byref(a)) == 0
    # rows come out in batch order: [history of seq b, new tokens of seq b]; error <= (1/2+1/32)*scale + fp16 rounding
    hs = b.histstarts
    for i in range(b.batch):
        want_k = np.concatenate([t["hist_key"][hs[i]:hs[i + 1]], t["current_key"][seqstarts[i]:seqstarts[i + 1]]])
        want_v = np.concatenate([t["hist_value"][hs[i]:hs[i + 1]], t["current_value"][seqstarts[i]:seqstarts[i + 1]]])
        rows = slice(b.cachestarts[i], b.cachestarts[i] + b.kvlens[i])
        sk = np.repeat(scale[rows, 1, 0].astype(np.float64), 8, axis=-1)
        sv = np.repeat(scale[rows, 1, 1].astype(np.float64), 8, axis=-1)
        gk, gv = ko[kvstarts[i]:kvstarts[i + 1]].astype(np.float64), vo[kvstarts[i]:kvstarts[i + 1]].astype(np.float64)
        assert (np.abs(gk - want_k) <= 0.54 * sk + 2e-3 * np.abs(want_k)).all()
        assert (np.abs(gv - want_v) <= 0.54 * sv + 2e-3 * np.abs(want_v)).all()
    deq = dequant_slab(cache, scale)
    i = 1
    assert np.array_equal(ko[kvstarts[i]:kvstarts[i + 1]],
                          deq[b.cachestarts[i]:b.cachestarts[i] + b.kvlens[i], 1, 0].astype(np.float32).astype(np.float16))
    a.num_repeat = 2
    assert olib.oracle_kv_cache_forward(C.byref(a)) == cabi.RC_UNSUPPORTED


@pytest.mark.parametrize("causal", [1, 0])
def test_mha_vs_textbook_and_mhca_identity(causal):
    # explicit K/V with kvlen > seqlen (decode rows, chunked rows) and kvlen == seqlen (fresh prompts)
    b = workloads.Batch(8, 2, 128, [1, 1, 7, 33, 5], [12, 0, 0, 20, 64], 2, is_causal=causal, name="mha_mixed")
    t = workloads.make_tensors(b, seed=21)
    key, value = harness.mha_inputs(b, t)
    got = harness.run_oracle_mha(b, t["query"], key, value)
    ss, ks = b.seqstarts, b.kvstarts
    for i in range(b.batch):
        L, kv = int(ss[i + 1] - ss[i]), int(ks[i + 1] - ks[i])
        for h in range(b.num_heads):
            ref = harness.textbook_attention(t["query"][ss[i]:ss[i + 1], h], key[ks[i]:ks[i + 1], h // 4],
                                             value[ks[i]:ks[i + 1], h // 4], causal_offset=(kv - L) if causal else None)
            assert np.abs(got["output_f64"][ss[i]:ss[i + 1], h] - ref).max() < 1e-9
    # MultiHeadCacheAttention == MultiHeadAttention over the KeyValueCache outputs: feed MHA the de-quantised cache
    # rows the cache path attends to (cache-prefill on, so every sequence reads the slab)
    mhca = harness.run_oracle(b, t, cache_prefill=1)
    import oracle
    n = int(ks[-1])
    deq = lambda kv_idx: np.concatenate([
        (mhca["cache"][b.cachestarts[i]:b.cachestarts[i] + (ks[i + 1] - ks[i]), 0, kv_idx].astype(np.float32).reshape(-1, 2, 16, 8)
         * mhca["scale"][b.cachestarts[i]:b.cachestarts[i] + (ks[i + 1] - ks[i]), 0, kv_idx].astype(np.float32)[..., None]
         ).reshape(-1, 2, 128) for i in range(b.batch)]).astype(np.float16)
    kd, vd = deq(0), deq(1)
    assert kd.shape == (n, 2, 128)
    via_mha = harness.run_oracle_mha(b, t["query"], kd, vd)
    # int8 * fp16 scale is exact in fp32 and, with |q| <= 127, needs at most 18 significant bits: rounding it to
    # fp16 here is the KeyValueCache op's output rounding, which the cache path does not apply -> small difference
    assert np.abs(via_mha["output_f64"] - mhca["output_f64"]).max() < 2e-3


def test_paged_cache_equals_contiguous_cache():
    """cache_mode 1: the same tokens reached through a scattered page table give the same bytes and the same outputs."""
    b = workloads.Batch(8, 2, 128, [1, 1, 1, 70, 300], [130, 5, 1000, 0, 64], 3, num_layer=2, layer_idx=1,
                        name="paged_mixed")
    t = workloads.make_tensors(b, seed=51)
    for page_size in (64, 128):
        paged = harness.PagedLayout(b, page_size=page_size, seed=page_size)
        flat = harness.run_oracle(b, t, cache_prefill=1)
        pg = harness.run_oracle(b, t, cache_prefill=1, paged=paged)
        assert np.array_equal(flat["output_f64"], pg["output_f64"])
        kv = b.kvlens
        for i in range(b.batch):
            for j in (0, int(kv[i]) // 2, int(kv[i]) - 1):
                a, c = int(b.cachestarts[i]) + j, paged.token(i, j)
                assert np.array_equal(flat["cache"][a], pg["cache"][c])
                assert np.array_equal(flat["scale"][a].view(np.uint16), pg["scale"][c].view(np.uint16))
        # untouched pages keep the fill pattern
        used = set()
        for i in range(b.batch):
            used |= {int(x) // page_size for x in paged.table[i] if x >= 0}
        free = sorted(set(range(paged.slab_tokens // page_size)) - used)
        assert free and (pg["cache"][free[0] * page_size:(free[0] + 1) * page_size] == harness.CACHE_FILL).all()


def test_cache_layout_3_equals_layout_0():
    """cache_layout 3 = (L, 2, KVH, MaxT, Dh): same bytes, transposed; strides of multi_head_cache_attention_kernel.cc:149-155."""
    b = workloads.Batch(8, 2, 128, [1, 1, 40], [77, 3, 0], 2, num_layer=3, layer_idx=2, name="layout3")
    t = workloads.make_tensors(b, seed=54)
    l0 = harness.run_oracle(b, t, cache_prefill=1)
    l3 = harness.run_oracle(b, t, cache_prefill=1, layout=3)
    assert np.array_equal(l0["output_f64"], l3["output_f64"])
    assert np.array_equal(l0["cache"].transpose(1, 2, 3, 0, 4), l3["cache"])
    assert np.array_equal(l0["scale"].view(np.uint16).transpose(1, 2, 3, 0, 4), l3["scale"].view(np.uint16))


def _random_mask(rng, shape, kstart_pad=0, frac_inf=0.15):
    """fp16 additive mask with some keys masked out completely (-inf), never a whole row."""
    m = (rng.standard_normal(shape) * 2).astype(np.float16)
    drop = rng.random(shape) < frac_inf
    drop[..., 0] = False  # key 0 of the packed axis is not what rows see; rows are fixed up by the callers
    m[drop] = -np.inf
    return m


def _mask_for(b, rng, per_head):
    """A mask over packed query tokens x packed keys, last extent padded to a multiple of 8 (as exporters do); every
    row keeps its sequence's first key so that no row is masked out entirely."""
    S, K = b.total_new_tokens, int(b.kvstarts[-1])
    kpad = (K + 7) // 8 * 8
    shape = (b.num_heads, S, kpad) if per_head else (S, kpad)
    m = _random_mask(rng, shape)
    for i in range(b.batch):
        m[..., b.seqstarts[i]:b.seqstarts[i + 1], b.kvstarts[i]] = np.float16(0.25)
    return m


@pytest.mark.parametrize("per_head", [False, True])
@pytest.mark.parametrize("causal", [1, 0])
def test_attn_mask_vs_textbook(per_head, causal):
    """The additive mask: entry [h?, seqstarts[b] + t, kvstarts[b] + j] is added to the scaled score of query t and key
    j of sequence b, on top of the causal rule. Checked per head against the float64 textbook routine."""
    b = workloads.Batch(6, 2, 64, [1, 1, 9, 33], [40, 3, 0, 0], 2, is_causal=causal)
    t = workloads.make_tensors(b, seed=77)
    mask = _mask_for(b, np.random.default_rng(5), per_head)
    res = harness.run_oracle(b, t, mask=mask)
    deq = dequant_slab(res["cache"], res["scale"])
    rep = b.num_heads // b.num_kv_heads
    for i in range(b.batch):
        s0, L, sp, kv, k0 = b.seqstarts[i], b.seqlens[i], b.start_pos[i], b.kvlens[i], b.kvstarts[i]
        for h in range(b.num_heads):
            if i < b.decoding_batches:
                rows = slice(b.cachestarts[i], b.cachestarts[i] + kv)
                k, v = deq[rows, 0, 0, h // rep], deq[rows, 0, 1, h // rep]
            else:
                k, v = t["current_key"][s0:s0 + L, h // rep], t["current_value"][s0:s0 + L, h // rep]
            mm = (mask[h] if per_head else mask)[s0:s0 + L, k0:k0 + kv]
            want = harness.textbook_attention(t["query"][s0:s0 + L, h], k, v, causal_offset=sp if causal else None,
                                              mask=mm)
            assert np.abs(res["output_f64"][s0:s0 + L, h] - want).max() < 1e-12, (i, h)
    # the mask matters: without it the result differs
    plain = harness.run_oracle(b, t)
    assert np.abs(plain["output_f64"] - res["output_f64"]).max() > 1e-3


def test_attn_mask_special_cases():
    b = workloads.Batch(4, 2, 32, [1, 5], [6, 0], 1)
    t = workloads.make_tensors(b, seed=78)
    S, K = b.total_new_tokens, int(b.kvstarts[-1])
    # an all-zero mask changes nothing
    zero = np.zeros((S, K), np.float16)
    plain = harness.run_oracle(b, t)
    assert np.array_equal(harness.run_oracle(b, t, mask=zero)["output_f64"], plain["output_f64"])
    # a constant added to a whole row cancels in the softmax
    const = np.full((S, K), 3.0, np.float16)
    assert np.abs(harness.run_oracle(b, t, mask=const)["output_f64"] - plain["output_f64"]).max() < 1e-12
    # -inf on every key but one: the output is that key's value row
    only = np.full((S, K), -np.inf, np.float16)
    only[0, b.kvstarts[0] + 2] = 0
    for tq in range(5):
        only[1 + tq, b.kvstarts[1] + 0] = 0
    res = harness.run_oracle(b, t, mask=only)
    deq = dequant_slab(res["cache"], res["scale"])
    assert np.abs(res["output_f64"][0, 3] - deq[b.cachestarts[0] + 2, 0, 1, 1]).max() < 1e-12
    assert np.abs(res["output_f64"][3, 0] - t["current_value"][b.seqstarts[1], 0].astype(np.float64)).max() < 1e-12
    # every key of a row masked out: zeros, not NaN
    none = only.copy()
    none[0, :] = -np.inf
    res = harness.run_oracle(b, t, mask=none)
    assert (res["output_f64"][0] == 0).all() and np.isfinite(res["output_f64"]).all()


def test_mha_attn_mask_vs_textbook():
    b = workloads.Batch(4, 1, 96, [1, 7, 20], [30, 0, 12], 1)
    t = workloads.make_tensors(b, seed=79)
    key, value = harness.mha_inputs(b, t)
    mask = _mask_for(b, np.random.default_rng(6), per_head=True)
    res = harness.run_oracle_mha(b, t["query"], key, value, mask=mask)
    for i in range(b.batch):
        s0, L, kv, k0 = b.seqstarts[i], b.seqlens[i], b.kvlens[i], b.kvstarts[i]
        for h in range(b.num_heads):
            want = harness.textbook_attention(t["query"][s0:s0 + L, h], key[k0:k0 + kv, 0], value[k0:k0 + kv, 0],
                                              causal_offset=kv - L, mask=mask[h, s0:s0 + L, k0:k0 + kv])
            assert np.abs(res["output_f64"][s0:s0 + L, h] - want).max() < 1e-12
