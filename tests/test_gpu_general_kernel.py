"""The general attention kernel through the C ABI: head_dim other than 128, more than 16 query heads per kv head and
the additive attn_mask, for MultiHeadCacheAttention (decode sequences, prompts, cache-prefill, paged slab, layer
strides) and MultiHeadAttention. Same bar as the tuned kernels: slab bytes and scales bit-exact against the oracle,
outputs within 2e-3 abs + 1e-2 rel of its float64 result."""
import ctypes as C

import numpy as np
import pytest

import harness
from harness import cabi, workloads
from test_oracle_attention import _mask_for

pytestmark = pytest.mark.gpu


def check(b, t, what, pieces=None, **kw):
    print(f"case {what}: H={b.num_heads} KVH={b.num_kv_heads} Dh={b.head_dim} B={b.batch} nd={b.decoding_batches} "
          f"S={b.total_new_tokens} hist={b.total_hist_tokens} {sorted(k for k in kw)}", flush=True)
    plans = []
    ref = harness.run_oracle(b, t, **kw)
    got = harness.run_device(b, t, plan_out=plans, **kw)
    assert plans[0].general_kernel == 1
    # head_dim 64 / 32 with kv heads that pair up in the slab: the decode sequences run the head_dim-128 decode kernel
    # over groups of kv heads (its ranges and workspace), the general kernel takes the prompts
    grouped = plans[0].decode_num_ranges > 0
    assert grouped or (plans[0].workspace_bytes == 0) == (plans[0].general_decode_splits <= 1)
    if pieces is not None and not grouped:
        assert plans[0].general_decode_splits == pieces
    assert np.array_equal(ref["cache"], got["cache"]), "int8 cache bytes differ"
    assert np.array_equal(ref["scale"].view(np.uint16), got["scale"].view(np.uint16)), "fp16 scales differ"
    harness.assert_attn_close(got["output"], ref["output_f64"], what=what)
    return ref, got


@pytest.mark.parametrize("Dh", [32, 64, 96, 160, 192, 224, 256])
@pytest.mark.parametrize("H,KVH", [(8, 2), (5, 5), (6, 1)])
def test_head_dims_mixed_batch(Dh, H, KVH):
    # decode sequences of 1 .. several tiles of history, prompts that straddle the 64-row and 64-token tile edges
    b = workloads.Batch(H, KVH, Dh, [1, 1, 1, 1, 7, 65, 130], [300, 1, 63, 64, 0, 0, 0], 4, num_layer=2, layer_idx=1,
                        name="general_mixed")
    check(b, workloads.make_tensors(b, seed=Dh + H), f"head_dim {Dh}")


@pytest.mark.parametrize("Dh,H,KVH", [(80, 8, 2), (112, 5, 5), (48, 6, 1), (16, 4, 2), (144, 8, 2), (240, 6, 1), (176, 34, 2)])
def test_head_dims_that_are_not_multiples_of_32(Dh, H, KVH):
    """head_dim 80, 112, ...: the kernels run the next multiple of 32 with the channels past head_dim held as zeros;
    rows in memory (queries, fp16 keys, slab heads, outputs) keep their real length, so the neighbouring head's
    channels must neither be read into a score nor be overwritten. Decode sequences long enough for pieces, prompts
    over the tile edges, with and without cache-prefill."""
    b = workloads.Batch(H, KVH, Dh, [1, 1, 1, 1, 7, 65, 130], [700, 1, 63, 64, 0, 0, 33], 4, num_layer=2, layer_idx=1,
                        name="general_padded")
    t = workloads.make_tensors(b, seed=Dh + H)
    check(b, t, f"head_dim {Dh}")
    check(b, t, f"head_dim {Dh}, cache-prefill", cache_prefill=1)
    check(b, t, f"head_dim {Dh}, cache_layout 3", layout=3)


@pytest.mark.parametrize("Dh,H,KVH", [(64, 8, 2), (64, 32, 8), (64, 16, 16), (64, 6, 6), (32, 16, 4), (32, 8, 8)])
def test_head_dim_64_and_32_decode_sequences_run_the_decode_kernel_over_groups_of_kv_heads(Dh, H, KVH):
    """Two (four) kv heads that are neighbours in the slab are streamed as one head of 128 channels by the head_dim-128
    decode kernel, every query head's channels in its own part of the 128-channel query operand: ragged decode
    sequences (short, one stage, many stages, split over ranges), with prompts in the same call, contiguous and paged
    (same bits); heads that are not neighbours (cache_layout 3) keep the general decode kernel."""
    b = workloads.Batch(H, KVH, Dh, [1] * 7 + [70, 5], [2000, 5, 0, 319, 1300, 31, 32, 0, 0], 7, num_layer=2,
                        layer_idx=1, name="grouped_heads")
    t = workloads.make_tensors(b, seed=H + Dh)
    plans = []
    ref = harness.run_oracle(b, t)
    got = harness.run_device(b, t, plan_out=plans)
    assert plans[0].general_kernel == 1 and plans[0].decode_num_ranges > 0 and plans[0].workspace_bytes > 0
    assert np.array_equal(ref["cache"], got["cache"]) and np.array_equal(ref["scale"].view(np.uint16), got["scale"].view(np.uint16))
    harness.assert_attn_close(got["output"], ref["output_f64"], what=f"grouped kv heads, head_dim {Dh}")
    paged = harness.PagedLayout(b, page_size=64, seed=3)
    gotp = harness.run_device(b, t, paged=paged)
    assert np.array_equal(gotp["output"].view(np.uint16), got["output"].view(np.uint16))
    plans3 = []
    got3 = harness.run_device(b, t, plan_out=plans3, layout=3)
    assert plans3[0].general_kernel == 1 and plans3[0].decode_num_ranges == 0
    harness.assert_attn_close(got3["output"], ref["output_f64"], what="cache_layout 3 keeps the general decode kernel")
    # decode only, and the split knob at its two other settings
    bd = workloads.Batch(H, KVH, Dh, [1] * 5, [4000, 700, 64, 1, 129], 5, name="grouped_heads_decode_only")
    td = workloads.make_tensors(bd, seed=7)
    refd = harness.run_oracle(bd, td)
    for split_k in (0, 1, 2):
        gd = harness.run_device(bd, td, split_k=split_k)
        assert np.array_equal(refd["cache"], gd["cache"])
        harness.assert_attn_close(gd["output"], refd["output_f64"], what=f"decode only, split knob {split_k}")


@pytest.mark.parametrize("H,KVH", [(34, 2), (20, 1), (48, 2)])
def test_more_than_16_query_heads_per_kv_head(H, KVH):
    b = workloads.Batch(H, KVH, 128, [1, 1, 40, 3], [500, 17, 0, 0], 2, name="general_rep")
    check(b, workloads.make_tensors(b, seed=H), f"{H // KVH} query heads per kv head")


@pytest.mark.parametrize("Dh", [64, 128])
@pytest.mark.parametrize("per_head", [False, True])
@pytest.mark.parametrize("causal", [1, 0])
def test_attn_mask(Dh, per_head, causal):
    b = workloads.Batch(8, 2, Dh, [1, 1, 1, 9, 70, 129], [200, 3, 64, 0, 0, 0], 3, is_causal=causal, name="general_mask")
    t = workloads.make_tensors(b, seed=7 + Dh)
    mask = _mask_for(b, np.random.default_rng(Dh + per_head), per_head)
    ref, got = check(b, t, f"attn_mask per_head={per_head} causal={causal}", mask=mask)
    plain = harness.run_oracle(b, t)
    assert np.abs(plain["output_f64"] - ref["output_f64"]).max() > 1e-3  # the mask matters


@pytest.mark.parametrize("H,KVH,Dh", [(8, 2, 64), (6, 6, 96), (34, 2, 128), (4, 1, 256), (8, 2, 80)])
def test_long_decode_sequences_are_cut_into_pieces(H, KVH, Dh):
    """Decode sequences long enough for the plan to share their keys out among several workgroups: pieces that end
    inside a tile, pieces past a short sequence's end (empty), one sequence of exactly one piece; with a paged slab
    the same bits."""
    b = workloads.Batch(H, KVH, Dh, [1] * 6 + [70, 5], [2000, 5, 700, 319, 1300, 255, 0, 0], 6, num_layer=2,
                        layer_idx=1, name="general_pieces")
    t = workloads.make_tensors(b, seed=H + Dh)
    _, flat = check(b, t, f"pieces {H}/{KVH}/{Dh}", pieces=32)  # 2001 keys, a tile each
    paged = harness.PagedLayout(b, page_size=64, seed=11)
    _, got = check(b, t, f"pieces, paged slab {H}/{KVH}/{Dh}", pieces=32, paged=paged)
    assert np.array_equal(got["output"].view(np.uint16), flat["output"].view(np.uint16))


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes(seed):
    """Seeded random head shapes and ragged batches through the general path: decode sequences of 1 .. 1500 cached
    tokens (pieces or none, sequence ends inside and on block and piece edges), prompts, any number of kv heads (so
    that a decode workgroup's four waves belong to different sequences and pieces), contiguous / paged / layout 3."""
    rng = np.random.default_rng(1000 + seed)
    Dh = int(rng.choice([32, 64, 96, 160, 192, 224, 256, 16, 48, 80, 112, 144, 240]))
    KVH = int(rng.integers(1, 9))
    rep = int(rng.choice([1, 2, 3, 4, 7, 8, 16, 17, 33]))
    nd = int(rng.integers(1, 9))
    npf = int(rng.integers(0, 3))
    edges = [1, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 256, 319, 320, 321]
    hist = [int(rng.choice(edges)) - 1 if rng.random() < 0.5 else int(rng.integers(0, 1500)) for _ in range(nd)]
    seqlens = [1] * nd + [int(rng.integers(1, 150)) for _ in range(npf)]
    start = hist + [0] * npf
    causal = int(rng.random() < 0.8)
    b = workloads.Batch(KVH * rep, KVH, Dh, seqlens, start, nd, num_layer=2, layer_idx=int(rng.integers(0, 2)),
                        is_causal=causal, slack_tokens=int(rng.integers(0, 3)), name="general_random")
    t = workloads.make_tensors(b, seed=seed)
    kw = {}
    how = int(rng.integers(0, 4))
    if how == 1:
        kw["paged"] = harness.PagedLayout(b, page_size=int(rng.choice([64, 128])), seed=seed)
    elif how == 2:
        kw["layout"] = 3
    if rng.random() < 0.3:
        kw["mask"] = _mask_for(b, rng, per_head=bool(rng.random() < 0.5))
    check(b, t, f"random shapes, seed {seed}", **kw)


def test_pieces_with_attn_mask_and_a_fully_masked_piece():
    b = workloads.Batch(8, 2, 64, [1, 1, 1, 9], [1500, 600, 40, 0], 3, name="general_pieces_mask")
    t = workloads.make_tensors(b, seed=77)
    mask = _mask_for(b, np.random.default_rng(5), per_head=True).copy()
    mask[:, 0, 64:192] = -np.inf  # every key of the first sequence's second and third piece (24 pieces of 64 keys)
    mask[:, 1, :] = -np.inf  # the second decode sequence sees nothing at all
    ref, got = check(b, t, "pieces + mask", pieces=24, mask=mask)
    assert (got["output"][1] == 0).all()
    plain = harness.run_oracle(b, t)
    assert np.abs(plain["output_f64"] - ref["output_f64"]).max() > 1e-3


def test_attn_mask_with_a_fully_masked_row():
    b = workloads.Batch(4, 2, 64, [1, 5], [70, 0], 1, name="general_mask_row")
    t = workloads.make_tensors(b, seed=3)
    mask = _mask_for(b, np.random.default_rng(9), per_head=False)
    mask[0, :] = -np.inf  # the decode sequence sees nothing
    mask[3, :] = -np.inf  # so does one prompt token
    ref, got = check(b, t, "fully masked rows", mask=mask)
    assert (got["output"][0] == 0).all() and (got["output"][3] == 0).all()


def test_cache_prefill_paged_and_layout_3():
    b = workloads.Batch(8, 2, 64, [1, 1, 70, 300], [130, 1000, 64, 0], 2, num_layer=2, layer_idx=1, name="general_cp")
    t = workloads.make_tensors(b, seed=52)
    ref, flat = check(b, t, "cache-prefill", cache_prefill=1)
    paged = harness.PagedLayout(b, page_size=64, seed=5)
    _, got = check(b, t, "cache-prefill, paged slab", cache_prefill=1, paged=paged)
    assert np.array_equal(got["output"].view(np.uint16), flat["output"].view(np.uint16))
    _, got3 = check(b, t, "cache-prefill, cache_layout 3", cache_prefill=1, layout=3)
    # (the decode tokens' kernel takes two kv heads per wave where they are neighbours in the slab, one in layout 3:
    # another order of summation, so those rows are only held to the oracle's tolerance)
    nd = b.decoding_batches
    assert np.array_equal(got3["output"][nd:].view(np.uint16), flat["output"][nd:].view(np.uint16))


@pytest.mark.parametrize("Dh,mask_on", [(64, False), (96, True), (256, False), (128, True), (80, False), (112, True)])
def test_multi_head_attention_general(Dh, mask_on):
    b = workloads.Batch(8, 2, Dh, [1, 1, 7, 130, 64], [300, 0, 0, 70, 64], 2, name="general_mha")
    t = workloads.make_tensors(b, seed=31)
    key, value = harness.mha_inputs(b, t)
    mask = _mask_for(b, np.random.default_rng(2), per_head=True) if mask_on else None
    print(f"case {b.name} Dh={Dh} mask={mask_on}", flush=True)
    ref = harness.run_oracle_mha(b, t["query"], key, value, mask=mask)
    got = harness.run_device_mha(b, t["query"], key, value, mask=mask)
    harness.assert_attn_close(got["output"], ref["output_f64"], what="MultiHeadAttention (general kernel)")


def test_general_kernel_agrees_with_the_tuned_kernels():
    """At head_dim 128 an all-zero mask sends the same call through the general kernel: both paths must agree with
    the oracle, and with each other within twice the tolerance."""
    b = workloads.Batch(32, 8, 128, [1] * 6 + [100, 257], [900, 64, 1, 2047, 333, 65, 0, 0], 6, name="general_vs_tuned")
    t = workloads.make_tensors(b, seed=4)
    zero = np.zeros((b.total_new_tokens, (int(b.kvstarts[-1]) + 7) // 8 * 8), np.float16)
    ref, gen = check(b, t, "zero mask", mask=zero)
    tuned = harness.run_device(b, t)
    harness.assert_attn_close(tuned["output"], ref["output_f64"])
    assert np.array_equal(tuned["cache"], gen["cache"])
    d = np.abs(tuned["output"].astype(np.float64) - gen["output"].astype(np.float64))
    assert d.max() <= 2 * (2e-3 + 1e-2 * np.abs(ref["output_f64"]).max())


@pytest.mark.parametrize("Dh", [96, 80, 16])
def test_key_value_cache_op_other_head_dim(hiplib, olib, Dh):
    """KeyValueCache (quantise-write + gather) at head_dim 96 and at head dims whose last unit of four quantisation
    groups is half empty: slab and gathered rows bit-exact."""
    import torch
    b = workloads.Batch(3, 3, Dh, [1, 6, 40], [9, 0, 3], 0, num_layer=2, layer_idx=1, slack_tokens=2)
    t = workloads.make_tensors(b, seed=9)
    zeros = np.zeros(b.batch, np.int64)
    total_kv = int(b.kvstarts[-1])

    def run(lib_write, lib_fwd, ptr, conv, stream_args):
        cache, scale = harness.new_slab(b)
        cache, scale = conv(cache), conv(scale)
        tt = {k: conv(v) for k, v in t.items()}
        tabs = {k: conv(v) for k, v in dict(hs=b.histstarts, z=zeros, cs=b.cachestarts, ss=b.seqstarts,
                                            ks=b.kvstarts, sp=b.start_pos).items()}
        w = harness.fill_write_args(cabi.KvWriteArgs(), b, tt["hist_key"], tt["hist_value"], tabs["hs"], tabs["z"],
                                    tabs["cs"], cache, scale, ptr=ptr)
        assert lib_write(C.byref(w), *stream_args) == 0
        a = cabi.KvCacheArgs()
        harness.fill_write_args(a.write, b, tt["current_key"], tt["current_value"], tabs["ss"], tabs["sp"], tabs["cs"],
                                cache, scale, ptr=ptr)
        a.d_kvstarts = ptr(tabs["ks"])
        a.total_kv_tokens, a.max_kvlen = total_kv, b.max_kvlen
        a.num_repeat, a.cache_mode, a.cache_layout = 1, 0, 0
        ko = conv(np.zeros((total_kv, 3, Dh), np.float16))
        vo = conv(np.zeros((total_kv, 3, Dh), np.float16))
        a.d_key_out, a.d_value_out = ptr(ko), ptr(vo)
        assert lib_fwd(C.byref(a), *stream_args) == 0
        return cache, scale, ko, vo

    co, so, ko, vo = run(lambda w: olib.oracle_kv_quantize_write(w), lambda a: olib.oracle_kv_cache_forward(a),
                         harness._ptr, lambda x: np.ascontiguousarray(x).copy(), ())
    cd, sd, kd, vd = run(hiplib.pplhip_kv_quantize_write, hiplib.pplhip_kv_cache_forward, harness.dev_ptr,
                         harness.to_dev, (None,))
    torch.cuda.synchronize()
    f16 = lambda x: x.cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(cd.cpu().numpy(), co) and np.array_equal(f16(sd), so.view(np.uint16))
    assert np.array_equal(f16(kd), ko.view(np.uint16)) and np.array_equal(f16(vd), vo.view(np.uint16))


@pytest.mark.parametrize("Dh", [64, 128])
def test_prompt_with_history_but_no_cache_prefill_sees_its_new_tokens_only(Dh):
    """A prompt with start_pos > 0 in a call WITHOUT cache-prefill (a chunk whose history the caller chose not to
    attend to): current_key / current_value hold only its seqlen rows, so its keys are those rows on every path. The
    general path (here through an all-zero mask at head_dim 128, and natively at 64) must agree with the oracle and,
    at head_dim 128, with the tuned path; the last sequence's rows end exactly at the end of current_key."""
    b = workloads.Batch(8, 2, Dh, [1, 1, 70, 33, 130], [40, 900, 300, 0, 77], 2, num_layer=2, layer_idx=1,
                        name="general_prompt_history")
    t = workloads.make_tensors(b, seed=91 + Dh)
    zero_mask = np.zeros((b.total_new_tokens, (int(b.kvstarts[-1]) + 7) // 8 * 8), np.float16)
    ref, got = check(b, t, f"prompt history, no cache-prefill, Dh {Dh}", mask=zero_mask)
    if Dh == 128:
        tuned = harness.run_device(b, t)
        harness.assert_attn_close(tuned["output"], ref["output_f64"], what="tuned path")
        assert np.array_equal(tuned["cache"], got["cache"])
    else:
        check(b, t, f"prompt history, no cache-prefill, no mask, Dh {Dh}")
