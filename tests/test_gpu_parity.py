"""GPU parity tests: every call goes through the C ABI of the HIP library and is compared with the CPU oracle on
the same seeded inputs. int8 cache bytes and fp16 scales must match bit-exactly; attention outputs must be within
2e-3 absolute + 1e-2 relative of the oracle's float64 result."""
import ctypes as C

import numpy as np
import pytest

import harness
from harness import cabi, workloads

pytestmark = pytest.mark.gpu


def check(b, t, cache_prefill=0, split_k=1, plans=None):
    print(f"case {b.name} H={b.num_heads} KVH={b.num_kv_heads} B={b.batch} nd={b.decoding_batches} "
          f"S={b.total_new_tokens} hist={b.total_hist_tokens} split_k={split_k} cache_prefill={cache_prefill}",
          flush=True)
    ref = harness.run_oracle(b, t, cache_prefill=cache_prefill)
    got = harness.run_device(b, t, cache_prefill=cache_prefill, split_k=split_k, plan_out=plans)
    assert np.array_equal(ref["cache"], got["cache"]), "int8 cache bytes differ"
    assert np.array_equal(ref["scale"].view(np.uint16), got["scale"].view(np.uint16)), "fp16 scales differ"
    return harness.assert_attn_close(got["output"], ref["output_f64"]), ref, got


def test_quantize_write_all_finite_absmax_bit_exact(hiplib, olib):
    """Every non-negative finite fp16 as a group's absmax, with tie-prone companions, through the write kernel."""
    import torch
    finite = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16)
    a32 = finite.astype(np.float32)
    rng = np.random.default_rng(3)
    cols = [finite, -finite] + [(a32 * np.float32((k + 0.5) / 127.0)).astype(np.float16) for k in (0, 1, 63, 125, 126)]
    cols.append((a32 * rng.uniform(-1, 1, a32.size).astype(np.float32)).astype(np.float16))
    groups = np.stack(cols, axis=1)  # [31744, 8]
    n_tok = groups.shape[0] // 16  # 16 groups per 128-channel head row
    key = np.ascontiguousarray(groups[:n_tok * 16].reshape(n_tok, 1, 128))
    val = np.ascontiguousarray(-key[::-1])
    b = workloads.Batch(1, 1, 128, [n_tok], [0], 0)
    cache_o, scale_o = harness.new_slab(b)
    zeros = np.zeros(1, np.int64)
    w = harness.fill_write_args(cabi.KvWriteArgs(), b, key, val, b.seqstarts, zeros, b.cachestarts, cache_o, scale_o)
    assert olib.oracle_kv_quantize_write(C.byref(w)) == 0
    cache_d, scale_d = harness.to_dev(harness.new_slab(b)[0]), harness.to_dev(harness.new_slab(b)[1])
    kd, vd = harness.to_dev(key), harness.to_dev(val)
    ss, cs, sp = harness.to_dev(b.seqstarts), harness.to_dev(b.cachestarts), harness.to_dev(zeros)
    w = harness.fill_write_args(cabi.KvWriteArgs(), b, kd, vd, ss, sp, cs, cache_d, scale_d, ptr=harness.dev_ptr)
    harness.pkg.check(hiplib.pplhip_kv_quantize_write(C.byref(w), None), "kv_quantize_write")
    torch.cuda.synchronize()
    assert np.array_equal(cache_d.cpu().numpy(), cache_o)
    assert np.array_equal(scale_d.cpu().view(torch.int16).numpy().view(np.uint16), scale_o.view(np.uint16))


def test_quantizer_quotients_enumerated(probelib):
    """x * (1 / s) against x / s over every (absmax, x) pair of fp16 values, through the kernel library's own quantiser
    (compiled into the probe library from the same source with the same flags): no int8 differs."""
    import torch
    bad = torch.zeros(1, dtype=torch.int64, device="cuda")
    assert probelib.pplhip_probe_quantizer(harness.dev_ptr(bad), None) == 0, probelib.pplhip_probe_last_error()
    torch.cuda.synchronize()
    assert int(bad.item()) == 0


def test_quantize_write_every_value_against_a_spread_of_scales(hiplib, olib):
    """The device forms x / s as x * (1 / s), one division per group instead of eight; that the int8 results are those
    of the division for EVERY fp16 x and EVERY scale was established by enumerating all pairs on the device. Here: 200
    absmax values spread over the finite range (and the extremes), each with every fp16 value of no larger magnitude
    as its companions, through the write kernel against the oracle's divisions."""
    import torch
    pos = np.arange(0, 0x7c00, dtype=np.uint16)
    picks = np.unique(np.concatenate([pos[:: len(pos) // 190], [1, 2, 0x03ff, 0x0400, 0x7bff, 0x7bfe, 0x3c00]]))
    picks = picks[picks > 0].astype(np.uint16)
    groups = []
    for a in picks:
        mag = np.arange(0, int(a) + 1, dtype=np.uint16)  # bit patterns 0 .. a are the magnitudes <= absmax
        xs = np.concatenate([mag, mag | np.uint16(0x8000)])
        pad = (-len(xs)) % 7
        xs = np.concatenate([xs, np.zeros(pad, np.uint16)]).reshape(-1, 7)
        groups.append(np.concatenate([np.full((len(xs), 1), a, np.uint16), xs], axis=1))
    groups = np.concatenate(groups).view(np.float16)  # [n, 8], first element = the group's absmax
    n_tok = groups.shape[0] // 16
    key = np.ascontiguousarray(groups[:n_tok * 16].reshape(n_tok, 1, 128))
    val = np.ascontiguousarray(-key[::-1])
    print(f"case every value x {len(picks)} scales: {n_tok} tokens", flush=True)
    b = workloads.Batch(1, 1, 128, [n_tok], [0], 0)
    cache_o, scale_o = harness.new_slab(b)
    zeros = np.zeros(1, np.int64)
    w = harness.fill_write_args(cabi.KvWriteArgs(), b, key, val, b.seqstarts, zeros, b.cachestarts, cache_o, scale_o)
    assert olib.oracle_kv_quantize_write(C.byref(w)) == 0
    cache_d, scale_d = harness.to_dev(harness.new_slab(b)[0]), harness.to_dev(harness.new_slab(b)[1])
    kd, vd = harness.to_dev(key), harness.to_dev(val)
    ss, cs, sp = harness.to_dev(b.seqstarts), harness.to_dev(b.cachestarts), harness.to_dev(zeros)
    w = harness.fill_write_args(cabi.KvWriteArgs(), b, kd, vd, ss, sp, cs, cache_d, scale_d, ptr=harness.dev_ptr)
    harness.pkg.check(hiplib.pplhip_kv_quantize_write(C.byref(w), None), "kv_quantize_write")
    torch.cuda.synchronize()
    assert np.array_equal(cache_d.cpu().numpy(), cache_o)
    assert np.array_equal(scale_d.cpu().view(torch.int16).numpy().view(np.uint16), scale_o.view(np.uint16))


@pytest.mark.parametrize("H,KVH", [(4, 4), (8, 2), (8, 1), (32, 8), (16, 1), (40, 40)])
def test_small_mixed_batches(H, KVH):
    b = workloads.Batch(H, KVH, 128, [1, 1, 1, 1, 9, 130, 64, 1], [40, 0 + 1, 300, 63, 0, 0, 0, 0], 4,
                        num_layer=2, layer_idx=1, slack_tokens=3, name="small_mixed")
    t = workloads.make_tensors(b, seed=H * 100 + KVH)
    check(b, t)


def test_decode_only_and_prefill_only_and_layer_strides():
    b = workloads.Batch(8, 2, 128, [1] * 7, [1, 15, 16, 17, 63, 64, 65], 7, num_layer=3, layer_idx=0, name="decode_only")
    check(b, workloads.make_tensors(b, seed=1))
    b = workloads.Batch(8, 2, 128, [1, 2, 31, 32, 33, 127, 128, 129, 257], [0] * 9, 0, num_layer=3, layer_idx=2,
                        name="prefill_only")
    check(b, workloads.make_tensors(b, seed=2))


def test_prefill_non_causal():
    b = workloads.Batch(4, 2, 128, [70, 5, 200], [0, 0, 0], 0, is_causal=0, name="non_causal")
    check(b, workloads.make_tensors(b, seed=3))


def test_cache_prefill_with_start_pos():
    b = workloads.Batch(8, 4, 128, [1, 20, 130, 7], [12, 30, 100, 0], 1, name="cache_prefill")
    check(b, workloads.make_tensors(b, seed=4), cache_prefill=1)


def test_split_k_modes_agree():
    """Split count must not change the result beyond fp32 reassociation."""
    b = workloads.Batch(8, 2, 128, [1, 1, 1], [49999, 7000, 64], 3, name="split_k")
    t = workloads.make_tensors(b, seed=5)
    outs, plans = [], []
    for mode in (0, 1, 2):
        _, ref, got = check(b, t, split_k=mode, plans=plans)
        outs.append(got["output"].astype(np.float64))
    assert plans[0].decode_num_ranges < plans[1].decode_num_ranges <= plans[2].decode_num_ranges
    assert np.abs(outs[0] - outs[1]).max() < 1e-3 and np.abs(outs[0] - outs[2]).max() < 1e-3


def test_closed_forms_on_device():
    # kv length 1: output is exactly the dequantised value row (softmax over one key)
    b = workloads.Batch(8, 2, 128, [1, 1], [0, 0], 0, name="kvlen1_prefill")
    t = workloads.make_tensors(b, seed=6)
    got = harness.run_device(b, t)
    for s in range(2):
        for h in range(8):
            assert np.array_equal(got["output"][s, h], t["current_value"][s, h // 4])
    # poisoned future tokens must not leak into causal rows (finite poison: masked probabilities are exact zeros,
    # and 0 * finite = 0 in the PV product; NaN/Inf inputs are outside the op's contract)
    b = workloads.Batch(2, 1, 128, [100], [0], 0, name="causal_poison")
    t = workloads.make_tensors(b, seed=7)
    clean = harness.run_device(b, t)["output"]
    t["current_key"][60:] = np.float16(6e4)
    t["current_value"][60:] = np.float16(-6e4)
    dirty = harness.run_device(b, t)["output"]
    assert np.array_equal(clean[:60], dirty[:60])


def test_decode_equals_last_row_of_cache_prefill_on_device():
    bd = workloads.Batch(8, 2, 128, [1], [199], 1, name="decode_vs_prefill")
    t = workloads.make_tensors(bd, seed=8)
    d = harness.run_device(bd, t)
    bp = workloads.Batch(8, 2, 128, [200], [0], 0)
    tp = dict(query=np.concatenate([np.zeros((199, 8, 128), np.float16), t["query"]]),
              current_key=np.concatenate([t["hist_key"], t["current_key"]]),
              current_value=np.concatenate([t["hist_value"], t["current_value"]]),
              hist_key=np.zeros((0, 2, 128), np.float16), hist_value=np.zeros((0, 2, 128), np.float16))
    pr = harness.run_device(bp, tp, cache_prefill=1)
    assert np.array_equal(pr["cache"], d["cache"])
    assert np.abs(pr["output"][199].astype(np.float64) - d["output"][0].astype(np.float64)).max() < 2e-3


def test_kv_cache_op(hiplib, olib):
    import torch
    b = workloads.Batch(4, 4, 128, [1, 6, 1, 40], [9, 0, 3, 0], 0, num_layer=2, layer_idx=1, slack_tokens=2)
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
        ko = conv(np.zeros((total_kv, 4, 128), np.float16))
        vo = conv(np.zeros((total_kv, 4, 128), np.float16))
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


def test_pack_tables_random_and_churn(hiplib, olib):
    import torch
    import test_oracle_pack as top

    def dev_pack(a_ptr):
        return hiplib.pplhip_pack_tables(a_ptr, None)

    def run_dev(kvlen, newlen, cs):
        n = len(kvlen)
        d = dict(kv=harness.to_dev(kvlen), nl=harness.to_dev(newlen), cs=harness.to_dev(cs))
        out = {k: torch.full((m,), -7, dtype=torch.int64, device="cuda") for k, m in
               dict(seqstarts=n + 1, kvstarts=n + 1, cachestarts=n, start_pos=n, batch_slots=n, header=6).items()}
        a = cabi.PackArgs()
        a.d_slot_kvlen, a.d_slot_newlen, a.d_slot_cachestart = d["kv"].data_ptr(), d["nl"].data_ptr(), d["cs"].data_ptr()
        a.num_slots = n
        a.d_seqstarts, a.d_kvstarts = out["seqstarts"].data_ptr(), out["kvstarts"].data_ptr()
        a.d_cachestarts, a.d_start_pos = out["cachestarts"].data_ptr(), out["start_pos"].data_ptr()
        a.d_batch_slots, a.d_header = out["batch_slots"].data_ptr(), out["header"].data_ptr()
        harness.pkg.check(hiplib.pplhip_pack_tables(C.byref(a), None), "pack_tables")
        torch.cuda.synchronize()
        return {k: v.cpu().numpy() for k, v in out.items()}

    rng = np.random.default_rng(12)
    for n in (1, 2, 63, 64, 65, 256, 1000, 1024):
        for _ in range(3):
            kvlen = (rng.integers(0, 50, n) * (rng.random(n) < 0.7)).astype(np.int64)
            newlen = np.where(rng.random(n) < 0.2, 0, np.where(kvlen > 0, 1, rng.integers(1, 40, n))).astype(np.int64)
            newlen = np.where(rng.random(n) < 0.05, rng.integers(2, 9, n), newlen).astype(np.int64)
            cs = (np.arange(n) * 1024).astype(np.int64)
            got = run_dev(kvlen, newlen, cs)
            want = top.run_pack(olib.oracle_pack_tables, kvlen, newlen, cs)
            for k in want:
                assert np.array_equal(got[k], want[k]), (n, k)
    # churn schedule (the continuous-batching configuration), 100 steps, device state advanced on the device
    sch = workloads.ChurnSchedule(seed=2)
    for step in range(100):
        kv, nl = sch.next_step()
        got = run_dev(kv, nl, sch.cachestart)
        want = top.run_pack(olib.oracle_pack_tables, kv, nl, sch.cachestart)
        for k in want:
            assert np.array_equal(got[k], want[k]), (step, k)
        dkv, dnl = harness.to_dev(kv), harness.to_dev(nl)
        harness.pkg.check(hiplib.pplhip_advance_slots(dkv.data_ptr(), dnl.data_ptr(), len(kv), None), "advance")
        torch.cuda.synchronize()
        assert np.array_equal(dkv.cpu().numpy(), kv + nl)


def test_pack_tables_can_advance_the_slots_in_the_same_launch(hiplib, olib):
    """pplhip_pack_args.advance_slots: the tables are those of the plain call, and slot_kvlen has moved on by
    slot_newlen for every active slot when the launch is done (what pplhip_advance_slots does as a second launch).
    Against the oracle's pack with the same flag, over the churn schedule with the state kept on the device."""
    import torch
    import test_oracle_pack as top
    sch = workloads.ChurnSchedule(seed=2)
    n = sch.num_slots
    out = {k: torch.full((m,), -7, dtype=torch.int64, device="cuda") for k, m in
           dict(seqstarts=n + 1, kvstarts=n + 1, cachestarts=n, start_pos=n, batch_slots=n, header=6).items()}
    dcs = harness.to_dev(sch.cachestart)
    for step in range(30):
        kv, nl = sch.next_step()
        dkv, dnl = harness.to_dev(kv), harness.to_dev(nl)  # (retirements reset slots: the scheduler's upload)
        a = cabi.PackArgs()
        a.d_slot_kvlen, a.d_slot_newlen, a.d_slot_cachestart = dkv.data_ptr(), dnl.data_ptr(), dcs.data_ptr()
        a.num_slots, a.advance_slots = n, 1
        a.d_seqstarts, a.d_kvstarts = out["seqstarts"].data_ptr(), out["kvstarts"].data_ptr()
        a.d_cachestarts, a.d_start_pos = out["cachestarts"].data_ptr(), out["start_pos"].data_ptr()
        a.d_batch_slots, a.d_header = out["batch_slots"].data_ptr(), out["header"].data_ptr()
        harness.pkg.check(hiplib.pplhip_pack_tables(C.byref(a), None), "pack_tables")
        torch.cuda.synchronize()
        want = top.run_pack(olib.oracle_pack_tables, kv, nl, sch.cachestart)
        for k in want:
            assert np.array_equal(out[k].cpu().numpy(), want[k]), (step, k)
        assert np.array_equal(dkv.cpu().numpy(), kv + nl), step
    # the oracle with the flag: same tables, state advanced
    kv, nl = sch.next_step()
    kv2 = kv.copy()
    want = top.run_pack(olib.oracle_pack_tables, kv, nl, sch.cachestart)
    got = top.run_pack(olib.oracle_pack_tables, kv2, nl, sch.cachestart, advance=1)
    for k in want:
        assert np.array_equal(got[k], want[k])
    assert np.array_equal(kv2, kv + nl)


@pytest.mark.parametrize("causal", [1, 0])
def test_multi_head_attention_vs_oracle(causal):
    # decode rows (1 query, long history), chunked rows (kvlen > seqlen), fresh prompts; tiles that straddle 64/128
    b = workloads.Batch(8, 2, 128, [1, 1, 7, 130, 64, 257], [300, 0, 0, 70, 64, 0], 2, is_causal=causal,
                        name="mha_mixed")
    t = workloads.make_tensors(b, seed=31)
    key, value = harness.mha_inputs(b, t)
    print(f"case {b.name} causal={causal} S={b.total_new_tokens} KV={int(b.kvstarts[-1])}", flush=True)
    ref = harness.run_oracle_mha(b, t["query"], key, value)
    got = harness.run_device_mha(b, t["query"], key, value)
    harness.assert_attn_close(got["output"], ref["output_f64"], what="MultiHeadAttention output")


def test_mhca_equals_mha_over_kv_cache_outputs(hiplib):
    """The operator identity MultiHeadCacheAttention == MultiHeadAttention o KeyValueCache, all on the device."""
    import torch
    b = workloads.Batch(8, 2, 128, [1, 1, 40, 200], [99, 7, 0, 0], 2, name="mhca_identity")
    t = workloads.make_tensors(b, seed=32)
    print(f"case {b.name}", flush=True)
    mhca = harness.run_device(b, t, cache_prefill=1)
    # KeyValueCache on a fresh slab with the same history, then MultiHeadAttention over its fp16 outputs
    cache, scale = (harness.to_dev(x) for x in harness.new_slab(b))
    d = {k: harness.to_dev(v) for k, v in t.items()}
    tabs = {k: harness.to_dev(v) for k, v in dict(hs=b.histstarts, z=np.zeros(b.batch, np.int64), cs=b.cachestarts,
                                                  ss=b.seqstarts, ks=b.kvstarts, sp=b.start_pos).items()}
    w = harness.fill_write_args(cabi.KvWriteArgs(), b, d["hist_key"], d["hist_value"], tabs["hs"], tabs["z"],
                                tabs["cs"], cache, scale, ptr=harness.dev_ptr)
    harness.pkg.check(hiplib.pplhip_kv_quantize_write(C.byref(w), None), "history write")
    a = cabi.KvCacheArgs()
    harness.fill_write_args(a.write, b, d["current_key"], d["current_value"], tabs["ss"], tabs["sp"], tabs["cs"],
                            cache, scale, ptr=harness.dev_ptr)
    total_kv = int(b.kvstarts[-1])
    a.d_kvstarts = harness.dev_ptr(tabs["ks"])
    a.total_kv_tokens, a.max_kvlen = total_kv, b.max_kvlen
    a.num_repeat, a.cache_mode, a.cache_layout = 1, 0, 0
    ko = torch.zeros((total_kv, 2, 128), dtype=torch.float16, device="cuda")
    vo = torch.zeros_like(ko)
    a.d_key_out, a.d_value_out = harness.dev_ptr(ko), harness.dev_ptr(vo)
    harness.pkg.check(hiplib.pplhip_kv_cache_forward(C.byref(a), None), "kv_cache_forward")
    out = torch.zeros((b.total_new_tokens, 8, 128), dtype=torch.float16, device="cuda")
    m = harness.fill_mha_args(cabi.MhaArgs(), b, d["query"], ko, vo, tabs["ss"], tabs["ks"], out, ptr=harness.dev_ptr)
    harness.pkg.check(hiplib.pplhip_mha_forward(C.byref(m), None), "mha_forward")
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), mhca["cache"])
    via = out.cpu().view(torch.int16).numpy().view(np.float16).astype(np.float64)
    assert np.abs(via - mhca["output"].astype(np.float64)).max() < 2e-3


@pytest.mark.parametrize("page_size", [64, 128, 256])
def test_paged_cache_mode(page_size):
    """cache_mode 1 on the device: bit-identical slab rows and outputs to the contiguous mode, parity with the oracle.
    Long decode sequences make 32-token stages straddle page boundaries at every offset."""
    for cache_prefill in (0, 1):
        # without cache-prefill the prompts start at position 0; with it one of them is a chunk at position 64
        b = workloads.Batch(8, 2, 128, [1, 1, 1, 1, 70, 300], [130, 5, 1000, 2047, 0, 64 * cache_prefill], 4,
                            num_layer=2, layer_idx=1, name="paged_mixed")
        t = workloads.make_tensors(b, seed=52)
        paged = harness.PagedLayout(b, page_size=page_size, seed=page_size)
        print(f"case {b.name} page_size={page_size} max_pages={paged.max_pages} cache_prefill={cache_prefill}",
              flush=True)
        ref = harness.run_oracle(b, t, cache_prefill=cache_prefill, paged=paged)
        got = harness.run_device(b, t, cache_prefill=cache_prefill, paged=paged)
        flat = harness.run_device(b, t, cache_prefill=cache_prefill)
        assert np.array_equal(ref["cache"], got["cache"]), "int8 cache bytes differ"
        assert np.array_equal(ref["scale"].view(np.uint16), got["scale"].view(np.uint16)), "fp16 scales differ"
        harness.assert_attn_close(got["output"], ref["output_f64"])
        assert np.array_equal(got["output"].view(np.uint16), flat["output"].view(np.uint16))


def test_paged_cache_full_size_decode():
    b = workloads.cfg2_decode_part()
    t = workloads.make_tensors(b, seed=53)
    paged = harness.PagedLayout(b, page_size=128, seed=9)
    print(f"case {b.name} paged full size: {int(b.kvstarts[-1])} cached tokens, {paged.max_pages} pages max", flush=True)
    got = harness.run_device(b, t, paged=paged)
    flat = harness.run_device(b, t)
    assert np.array_equal(got["output"].view(np.uint16), flat["output"].view(np.uint16))


def test_cache_layout_3_on_device():
    """cache_layout 3 (L, 2, KVH, MaxT, Dh): token rows of one head are 128 bytes apart instead of a whole slab row."""
    for cache_prefill in (0, 1):
        b = workloads.Batch(8, 2, 128, [1, 1, 1, 70, 200], [130, 5, 1000, 0, 64 * cache_prefill], 3, num_layer=3,
                            layer_idx=2, name="layout3")
        t = workloads.make_tensors(b, seed=55)
        print(f"case {b.name} cache_prefill={cache_prefill}", flush=True)
        ref = harness.run_oracle(b, t, cache_prefill=cache_prefill, layout=3)
        got = harness.run_device(b, t, cache_prefill=cache_prefill, layout=3)
        flat = harness.run_device(b, t, cache_prefill=cache_prefill)
        assert np.array_equal(ref["cache"], got["cache"]) and np.array_equal(ref["scale"].view(np.uint16),
                                                                               got["scale"].view(np.uint16))
        harness.assert_attn_close(got["output"], ref["output_f64"])
        assert np.array_equal(got["output"].view(np.uint16), flat["output"].view(np.uint16))
        paged = harness.PagedLayout(b, page_size=64, seed=3)
        both = harness.run_device(b, t, cache_prefill=cache_prefill, layout=3, paged=paged)
        assert np.array_equal(both["output"].view(np.uint16), flat["output"].view(np.uint16))


@pytest.mark.parametrize("KVH", [8, 1])
def test_decode_writes_its_new_tokens_into_a_slab_of_garbage(monkeypatch, KVH):
    """Rows of the slab nobody has written hold NaN scales and -128 bytes: the decode kernel fetches the row of the
    new token before it has quantised it, and the rows it pads a partial last stage with are multiplied by zero
    probabilities, so none of that may reach the output. History lengths cover a last stage that is full (31 old
    tokens + the new one), one that holds only the new token (32, 64, 0 old tokens) and ragged ones; KVH = 1 splits a
    sequence's tokens between the waves of a workgroup."""
    monkeypatch.setattr(harness, "SCALE_FILL", 0x7E00)
    monkeypatch.setattr(harness, "CACHE_FILL", -128)
    hist = [31, 32, 64, 0, 1, 33, 63, 95, 100, 257, 1024, 7]
    b = workloads.Batch(8, KVH, 128, [1] * len(hist), hist, len(hist), name="decode into garbage")
    check(b, workloads.make_tensors(b, seed=11))
    # and next to prompts in the same call
    b = workloads.Batch(8, KVH, 128, [1] * 5 + [70, 129], [31, 32, 0, 5, 200, 0, 0], 5, name="mixed into garbage")
    check(b, workloads.make_tensors(b, seed=12))


def test_decode_new_tokens_in_a_paged_slab_of_garbage(monkeypatch):
    """The same with a page table: new tokens that open a page (kv position 64, 128), close one (63) or sit alone in
    the stage that straddles two pages."""
    monkeypatch.setattr(harness, "SCALE_FILL", 0x7E00)
    monkeypatch.setattr(harness, "CACHE_FILL", -128)
    hist = [63, 64, 127, 128, 0, 95, 96, 500, 1000]
    b = workloads.Batch(8, 2, 128, [1] * len(hist), hist, len(hist), name="paged decode into garbage")
    t = workloads.make_tensors(b, seed=13)
    paged = harness.PagedLayout(b, page_size=64, seed=5)
    ref = harness.run_oracle(b, t, paged=paged)
    got = harness.run_device(b, t, paged=paged)
    assert np.array_equal(ref["cache"], got["cache"]), "int8 cache bytes differ"
    assert np.array_equal(ref["scale"].view(np.uint16), got["scale"].view(np.uint16)), "fp16 scales differ"
    harness.assert_attn_close(got["output"], ref["output_f64"])


@pytest.mark.parametrize("KVH", [8, 2])
def test_more_decode_sequences_than_ranges(KVH):
    """20 to 40 short sequences over 8 ranges: several sequence boundaries inside every range, the partial results of
    the sequences that straddle a range boundary are merged by the (head, boundary) grid, and some ranges hold whole
    sequences only."""
    plans = []
    b = workloads.Batch(8, KVH, 128, [1] * 20, [100] * 20, 20, name="20 short sequences")
    check(b, workloads.make_tensors(b, seed=21), plans=plans)
    assert plans[-1].decode_num_ranges <= 20
    rng = np.random.default_rng(22)
    hist = rng.integers(0, 90, 40).tolist()
    b = workloads.Batch(8, KVH, 128, [1] * 40, hist, 40, name="40 ragged short sequences")
    check(b, workloads.make_tensors(b, seed=23), plans=plans)
    assert plans[-1].decode_num_ranges <= 40


def test_one_long_prompt_among_many_short_ones():
    """Prompt lengths so uneven that the prefill launch switches to its compact tile grid (one workgroup per possible
    tile, tile found by a search in the kernel): 100 short prompts around one of 1024 tokens (two passes of 64
    sequences in the search), then 300 short ones around one of 700 (more sequences than the search keeps in registers),
    with decode sequences in front."""
    rng = np.random.default_rng(31)
    lens = rng.integers(1, 41, 100).tolist()
    lens.insert(37, 1024)
    b = workloads.Batch(32, 8, 128, [1, 1, 1] + lens, [17, 200, 64] + [0] * 101, 3, name="1 long + 100 short prompts")
    check(b, workloads.make_tensors(b, seed=32))
    lens = rng.integers(1, 7, 300).tolist()
    lens.insert(280, 700)
    lens[5] = 129
    b = workloads.Batch(32, 8, 128, lens, [0] * 301, 0, name="1 long + 300 short prompts")
    check(b, workloads.make_tensors(b, seed=33))


def test_cache_prefill_over_staged_rows():
    """Chunks large enough that the plan stages the prompts' cached K/V as fp16 rows (one dequantisation pass) and
    runs attention over those: contiguous slab, paged slab, cache_layout 3, with decode sequences in front; the three
    must agree bit for bit with each other and match the oracle."""
    b = workloads.Batch(8, 2, 128, [1, 1, 300, 700, 260, 5], [77, 1500, 100, 0, 513, 31], 2, num_layer=2, layer_idx=1,
                        name="staged_cache_prefill")
    t = workloads.make_tensors(b, seed=61)
    plans = []
    _, ref, flat = check(b, t, cache_prefill=1, plans=plans)
    assert plans[-1].prefill_staging == 1
    paged = harness.PagedLayout(b, page_size=128, seed=5)
    got = harness.run_device(b, t, cache_prefill=1, paged=paged)
    assert np.array_equal(got["output"].view(np.uint16), flat["output"].view(np.uint16))
    lay3 = harness.run_device(b, t, cache_prefill=1, layout=3)
    assert np.array_equal(lay3["output"].view(np.uint16), flat["output"].view(np.uint16))
    # small chunks keep the kernel that dequantises the slab itself
    b = workloads.Batch(8, 2, 128, [1, 20, 130, 7], [12, 30, 100, 0], 1, name="small_chunks")
    plans = []
    check(b, workloads.make_tensors(b, seed=62), cache_prefill=1, plans=plans)
    assert plans[-1].prefill_staging == 0
    # uneven chunks: staged rows and the compact tile grid together
    rng = np.random.default_rng(63)
    lens = [1024] + rng.integers(200, 300, 40).tolist()
    hist = [256] + rng.integers(0, 50, 40).tolist()
    b = workloads.Batch(32, 8, 128, lens, hist, 0, name="staged_uneven_chunks")
    plans = []
    check(b, workloads.make_tensors(b, seed=64), cache_prefill=1, plans=plans)
    assert plans[-1].prefill_staging == 1


@pytest.mark.parametrize("cache_prefill", [0, 1])
def test_forward_replays_from_a_hip_graph(cache_prefill):
    """pplhip_mhca_forward only enqueues kernels: captured into a HIP graph on a side stream, every replay (with the
    program's own eager work and synchronisations between replays, new queries each time) gives bit for bit what the
    eager call gives. With cache_prefill the chunks are large enough for the staged route (one more kernel)."""
    import torch
    import bench
    lib = harness.pkg.load_library()
    if cache_prefill:
        b = workloads.Batch(8, 2, 128, [1, 1, 300, 700], [77, 1500, 100, 0], 2, name="graph_staged")
    else:
        b = workloads.Batch(8, 2, 128, [1, 1, 1, 150, 40], [300, 17, 1000, 0, 0], 3, name="graph_mixed")
    db = bench.DeviceBatch(harness.pkg, lib, b, seed=3, n_slabs=1, cache_prefill=cache_prefill)
    assert int(db.plan.prefill_staging) == cache_prefill
    default_stream = db.stream
    db.step(0)  # also takes the one-time per-device set-up out of the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        db.stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        db.step(0)
    db.stream = default_stream
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    for rep in range(3):
        db.q.copy_(torch.randn(db.q.shape, generator=gen, dtype=torch.float16, device="cuda"))
        db.out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = db.out.clone()
        db.out.zero_()
        db.step(0)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), db.out.view(torch.int16)), f"replay {rep} differs from the eager call"
        assert bool(got.float().abs().sum() > 0)


def test_degenerate_batches():
    """An empty call; decode sequences whose cache is empty (their new token is their only key); one-token prompts; a
    single sequence of each kind."""
    import torch
    lib = harness.pkg.load_library()
    a, plan = cabi.MhcaArgs(), cabi.MhcaPlan()
    b0 = workloads.Batch(8, 2, 128, [], [], 0, name="empty")
    harness.fill_mhca_args(a, b0, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, ptr=lambda t: C.c_void_p(0x1000))
    assert lib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS
    assert lib.pplhip_mhca_forward(C.byref(a), C.byref(plan), None, None) == cabi.RC_SUCCESS
    torch.cuda.synchronize()
    for kvh in (2, 8):
        b = workloads.Batch(8, kvh, 128, [1, 1, 1], [0, 5, 0], 3, name="decode_with_empty_cache")
        check(b, workloads.make_tensors(b, seed=71))
        b = workloads.Batch(8, kvh, 128, [1, 1, 1, 1], [0, 33, 0, 0], 2, name="one_token_prompts")
        check(b, workloads.make_tensors(b, seed=72))
        b = workloads.Batch(8, kvh, 128, [1], [0], 1, name="single_decode_empty_cache")
        check(b, workloads.make_tensors(b, seed=73))
        b = workloads.Batch(8, kvh, 128, [1], [0], 0, name="single_one_token_prompt")
        check(b, workloads.make_tensors(b, seed=74))


@pytest.mark.parametrize("KVH", [8, 1])
def test_hundreds_of_decode_sequences(KVH):
    """300 decode sequences (five passes of the 64-wide table search), some with an empty cache, a few long ones that
    span many ranges among them, and prompts behind them."""
    rng = np.random.default_rng(81)
    hist = rng.integers(0, 60, 300)
    hist[[7, 150, 299]] = [3000, 1777, 2500]
    b = workloads.Batch(8, KVH, 128, [1] * 300 + [40, 3], hist.tolist() + [0, 0], 300, name="300 decode sequences")
    check(b, workloads.make_tensors(b, seed=82))


@pytest.mark.parametrize("seed", range(12))
def test_random_batches_through_the_tuned_kernels(seed):
    """Seeded random batches at head_dim 128: any number of kv heads (workgroups of 1, 2 or 4 heads, range counts that
    are no multiple of 8), 0 .. 39 decode sequences whose lengths sit on and around the stage, tile and page edges,
    prompts with and without cache-prefill (and history), contiguous / paged / cache_layout 3 slabs, every split knob.
    Slab bytes and scales bit-exact, outputs within tolerance."""
    rng = np.random.default_rng(5000 + seed)
    KVH = int(rng.choice([1, 2, 3, 4, 5, 8, 10, 12]))
    rep = int(rng.choice([1, 2, 4, 8, 16]))
    nd = int(rng.integers(0, 40))
    npf = int(rng.integers(0, 4)) if nd else int(rng.integers(1, 4))
    edges = [1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 1023, 1024, 1025]
    hist = [int(rng.choice(edges)) - 1 if rng.random() < 0.4 else int(rng.integers(0, 3000)) for _ in range(nd)]
    cp = int(rng.random() < 0.3)
    seqlens = [1] * nd + [int(rng.integers(1, 400)) for _ in range(npf)]
    start = hist + [int(rng.integers(0, 300)) if cp else 0 for _ in range(npf)]
    b = workloads.Batch(KVH * rep, KVH, 128, seqlens, start, nd, num_layer=int(rng.integers(1, 3)), layer_idx=0,
                        is_causal=1, slack_tokens=int(rng.integers(0, 3)), name="random_tuned")
    t = workloads.make_tensors(b, seed=seed)
    kw = {}
    how = int(rng.integers(0, 4))
    if how == 1:
        kw["paged"] = harness.PagedLayout(b, page_size=int(rng.choice([64, 128, 256])), seed=seed)
    elif how == 2:
        kw["layout"] = 3
    if cp:
        kw["cache_prefill"] = 1
    split_k = int(rng.integers(0, 3))
    print(f"case random tuned, seed {seed}: H={b.num_heads} KVH={KVH} nd={nd} prompts={npf} split_k={split_k} {sorted(kw)}",
          flush=True)
    ref = harness.run_oracle(b, t, **kw)
    plans = []
    got = harness.run_device(b, t, split_k=split_k, plan_out=plans, **kw)
    assert plans[0].general_kernel == 0
    assert np.array_equal(ref["cache"], got["cache"]), "int8 cache bytes differ"
    assert np.array_equal(ref["scale"].view(np.uint16), got["scale"].view(np.uint16)), "fp16 scales differ"
    harness.assert_attn_close(got["output"], ref["output_f64"], what=f"random tuned batch, seed {seed}")
