"""Parity at the baseline's full configuration sizes (the oracle runs on the host cores with OpenMP)."""
import ctypes as C

import numpy as np
import pytest

import harness
from harness import cabi, workloads
from test_gpu_parity import check

pytestmark = pytest.mark.gpu


def test_cfg1_llama2_7b_decode_full():
    b = workloads.cfg1_llama2_7b_decode()
    check(b, workloads.make_tensors(b, seed=0))


def test_cfg2_llama3_8b_mixed_full():
    b = workloads.cfg2_llama3_8b_mixed()
    check(b, workloads.make_tensors(b, seed=1))


@pytest.mark.parametrize("split_k", [1, 2])
def test_cfg3_long_context_full(split_k):
    """8 sequences of 32 768 .. 131 072 cached tokens on one kv head, against the oracle at full length: every sequence
    spans dozens of split-k ranges (about 63 at the default knob, twice that at the finest), which is where the merge of
    the partial results does the most work."""
    b = workloads.cfg3_long_context()
    check(b, workloads.make_tensors(b, seed=3), split_k=split_k)


def test_cfg3_uniform_softmax_property_at_full_length():
    # a size-independent property at the maximum length: with every cached key equal, softmax is uniform and the
    # output is the mean of the dequantised values, whatever the split count
    b = workloads.Batch(8, 1, 128, [1, 1], [131071, 40000], 2, name="cfg3_full_property")
    rng = np.random.default_rng(5)
    t = dict(query=rng.standard_normal((2, 8, 128)).astype(np.float16),
             current_key=np.ones((2, 1, 128), np.float16), current_value=np.zeros((2, 1, 128), np.float16),
             hist_key=np.ones((b.total_hist_tokens, 1, 128), np.float16),
             hist_value=rng.integers(-8, 9, (b.total_hist_tokens, 1, 128)).astype(np.float16))
    t["hist_value"][:, :, ::8] = np.float16(127.0)  # scale exactly 1 per group: dequantised values == inputs
    got = harness.run_device(b, t)
    hs = b.histstarts
    for i in range(2):
        vals = np.concatenate([t["hist_value"][hs[i]:hs[i + 1], 0], t["current_value"][i]]).astype(np.float64)
        want = vals.mean(axis=0)
        for h in range(8):
            assert np.abs(got["output"][i, h].astype(np.float64) - want).max() <= 2e-3 + 1e-2 * np.abs(want).max()


def test_chunked_prefill_both_routes_at_full_size():
    """Chunks of 512 tokens on top of 0 .. 4096 cached tokens (H32 / KVH8), with decode sequences in front: the staged
    route (fp16 staging rows + the fp16 kernel, what the plan chooses) against the oracle, and against the route that
    reads the int8 slab in the attention kernel (the caller cleared plan.prefill_staging): same slab bytes, outputs
    within the attention tolerance of each other."""
    b = workloads.Batch(32, 8, 128, [1, 1, 512, 512, 512, 512], [3000, 500, 2048, 4096, 1000, 0], 2,
                        name="chunked_prefill_full")
    t = workloads.make_tensors(b, seed=7)
    plans = []
    _, ref, staged = check(b, t, cache_prefill=1, plans=plans)
    assert plans[-1].prefill_staging == 1
    direct = harness.run_device(b, t, cache_prefill=1, staging=0)
    assert np.array_equal(direct["cache"], staged["cache"])
    assert np.array_equal(direct["scale"].view(np.uint16), staged["scale"].view(np.uint16))
    harness.assert_attn_close(direct["output"], ref["output_f64"])
    diff = np.abs(direct["output"].astype(np.float64) - staged["output"].astype(np.float64))
    assert diff.max() <= 2 * (2e-3 + 1e-2 * np.abs(ref["output_f64"]).max())


def test_cfg4_churn_attention_over_device_built_tables(hiplib, olib):
    """Continuous-batching churn at its full shape (256 slots, H = KVH = 40, Dh 128, one 1024-token region per slot):
    the first steps of the seeded schedule -- step 0 admits 256 prompts, every later step retires a few sequences, admits
    new prompts into their slots and decodes the rest. Every step the tables are rebuilt ON THE DEVICE by
    pplhip_pack_tables from the slot state, MultiHeadCacheAttention runs on those device tables with the sizes read
    from the device-built header, and pplhip_advance_slots grows the slots. The oracle replays the same steps on the
    host with host-built tables (tools/benchmark_llama/generation_state.cc:127-192): the slab rows written in a step
    must match bit-exactly, the outputs within the attention tolerance, and the whole slab bit-exactly at the end."""
    import torch
    import test_oracle_pack as top
    sch = workloads.ChurnSchedule(seed=2)
    n, H, KVH, Dh = sch.num_slots, sch.num_heads, sch.num_kv_heads, sch.head_dim
    tokens = n * sch.region
    st = cabi.cache_strides_layout0(1, KVH, Dh)
    cache_h = np.full((tokens, 1, 2, KVH, Dh), harness.CACHE_FILL, np.int8)
    scale_h = np.full((tokens, 1, 2, KVH, Dh // 8), harness.SCALE_FILL, np.uint16).view(np.float16)
    cache_d, scale_d = harness.to_dev(cache_h), harness.to_dev(scale_h)
    slot_kv = torch.zeros(n, dtype=torch.int64, device="cuda")
    slot_cs = harness.to_dev(sch.cachestart)
    tabs = {k: torch.zeros(m, dtype=torch.int64, device="cuda") for k, m in
            dict(seqstarts=n + 1, kvstarts=n + 1, cachestarts=n, start_pos=n, batch_slots=n, header=6).items()}
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    saw_retirement = saw_admission_among_decodes = False
    for step in range(6):
        kv, nl = sch.next_step()
        retired = step > 0 and bool(((kv == 0) & (prev_after > 0)).any())
        saw_retirement |= retired
        saw_admission_among_decodes |= step > 0 and bool((kv == 0).any()) and bool((kv > 0).any())
        # ---- host side: tables by the oracle, inputs in packed order
        want = top.run_pack(olib.oracle_pack_tables, kv, nl, sch.cachestart)
        B, nd, max_seqlen, max_kvlen, S, _ = (int(x) for x in want["header"])
        order = want["batch_slots"][:B]
        b = workloads.Batch(H, KVH, Dh, nl[order], kv[order], nd, cachestarts=sch.cachestart[order], name="cfg4_step")
        assert np.array_equal(b.seqstarts, want["seqstarts"][:B + 1]) and np.array_equal(b.kvstarts, want["kvstarts"][:B + 1])
        print(f"case cfg4 churn step {step}: batch {B} decode {nd} new tokens {S} max_seqlen {max_seqlen} "
              f"max_kvlen {max_kvlen} retired {retired}", flush=True)
        rng = np.random.default_rng(100 + step)
        q = workloads._randn_f16(rng, (S, H, Dh))
        k = workloads._randn_f16(rng, (S, KVH, Dh))
        v = workloads._randn_f16(rng, (S, KVH, Dh))
        out_h = np.zeros((S, H, Dh), np.float16)
        out64 = np.zeros((S, H, Dh), np.float64)
        a = harness.fill_mhca_args(cabi.MhcaArgs(), b, q, k, v, b.seqstarts, b.kvstarts, b.cachestarts, b.start_pos.copy(),
                                   cache_h, scale_h, out_h)
        a.max_seqlen, a.max_kvlen = max_seqlen, max_kvlen
        assert olib.oracle_mhca_forward(C.byref(a), harness._ptr(out64)) == 0
        # ---- device side: scheduler's decisions (resets, new-token counts) in, tables rebuilt on the device
        slot_kv.copy_(harness.to_dev(kv))
        slot_nl = harness.to_dev(nl)
        pa = cabi.PackArgs()
        pa.d_slot_kvlen, pa.d_slot_newlen, pa.d_slot_cachestart = slot_kv.data_ptr(), slot_nl.data_ptr(), slot_cs.data_ptr()
        pa.num_slots = n
        pa.d_seqstarts, pa.d_kvstarts = tabs["seqstarts"].data_ptr(), tabs["kvstarts"].data_ptr()
        pa.d_cachestarts, pa.d_start_pos = tabs["cachestarts"].data_ptr(), tabs["start_pos"].data_ptr()
        pa.d_batch_slots, pa.d_header = tabs["batch_slots"].data_ptr(), tabs["header"].data_ptr()
        harness.pkg.check(hiplib.pplhip_pack_tables(C.byref(pa), stream), "pack_tables")
        hdr = tabs["header"].cpu().numpy()  # what a serving loop would read back (or keep in mapped host memory)
        assert hdr.tolist() == want["header"].tolist()
        dq, dk, dv = harness.to_dev(q), harness.to_dev(k), harness.to_dev(v)
        dout = torch.zeros((S, H, Dh), dtype=torch.float16, device="cuda")
        da = cabi.MhcaArgs()
        da.d_query, da.d_current_key, da.d_current_value = (harness.dev_ptr(x) for x in (dq, dk, dv))
        da.d_seqstarts, da.d_kvstarts = harness.dev_ptr(tabs["seqstarts"]), harness.dev_ptr(tabs["kvstarts"])
        da.d_cachestarts, da.d_start_pos = harness.dev_ptr(tabs["cachestarts"]), harness.dev_ptr(tabs["start_pos"])
        da.is_causal = 1
        da.batch, da.decoding_batches, da.max_seqlen, da.max_kvlen, da.total_new_tokens = (int(x) for x in hdr[:5])
        da.layer_idx, da.num_layer, da.num_heads, da.num_kv_heads, da.head_dim = 0, 1, H, KVH, Dh
        da.cache_mode, da.page_size = 0, 128
        for kk, vv in st.items():
            setattr(da, kk, vv)
        da.specify_decoding_attn_split_k = 1
        da.d_cache, da.d_scale, da.d_output = harness.dev_ptr(cache_d), harness.dev_ptr(scale_d), harness.dev_ptr(dout)
        plan = cabi.MhcaPlan()
        harness.pkg.check(hiplib.pplhip_mhca_prepare(C.byref(da), C.byref(plan)), "prepare")
        if nd:  # 10 groups of 4 kv heads: ranges x groups fill at most the 512 workgroup slots of one round
            assert plan.decode_heads_per_block == 4 and plan.decode_num_ranges * 10 <= 512
        ws = torch.empty(max(int(plan.workspace_bytes), 256), dtype=torch.uint8, device="cuda")
        harness.pkg.check(hiplib.pplhip_mhca_forward(C.byref(da), C.byref(plan), harness.dev_ptr(ws), stream), "forward")
        harness.pkg.check(hiplib.pplhip_advance_slots(slot_kv.data_ptr(), slot_nl.data_ptr(), n, stream), "advance")
        torch.cuda.synchronize()
        # ---- compare: tables, the slab rows this step wrote, outputs, slot state
        for name in ("seqstarts", "kvstarts", "cachestarts", "start_pos", "batch_slots"):
            assert np.array_equal(tabs[name].cpu().numpy(), want[name]), (step, name)
        rows = np.concatenate([np.arange(c + p, c + p + l) for c, p, l in zip(b.cachestarts, b.start_pos, b.seqlens)])
        drows = harness.to_dev(rows)
        assert np.array_equal(cache_d[drows].cpu().numpy(), cache_h[rows]), f"step {step}: int8 rows differ"
        assert np.array_equal(scale_d[drows].cpu().view(torch.int16).numpy(), scale_h[rows].view(np.int16)), \
            f"step {step}: fp16 scales differ"
        got = dout.cpu().view(torch.int16).numpy().view(np.float16)
        harness.assert_attn_close(got, out64, what=f"cfg4 step {step} output")
        assert np.array_equal(slot_kv.cpu().numpy(), kv + nl)
        prev_after = kv + nl
    assert saw_retirement and saw_admission_among_decodes
    assert np.array_equal(cache_d.cpu().numpy(), cache_h), "slab bytes differ after the replay"
    assert np.array_equal(scale_d.cpu().view(torch.int16).numpy(), scale_h.view(np.int16))
