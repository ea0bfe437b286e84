#!/usr/bin/env python3
"""Benchmark of the dynamic-batching attention path on one MI355X.

Default workload = the Llama-3-8B mixed ragged batch of the baseline (120 decode sequences with kv length uniform
in [256, 4096] + 8 causal prefill sequences with length uniform in [64, 1024]; H 32, KVH 8, Dh 128; int8 group-8
KV cache). One "step" of the headline loop is one MultiHeadCacheAttention call through the C ABI on the decode
part of that batch (quantize-on-write of the new tokens + split-k decode + merge); the prefill part and the fused
mixed call are timed in the same run and reported as extra fields. Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg1|cfg3] [--no-cpu-baseline]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16, published (no sparsity)
N_SLABS = 4  # distinct KV slabs rotated between steps so reads are served by HBM, not the 256 MB Infinity Cache


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2", choices=["cfg1", "cfg2", "cfg3"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--split-k", type=int, default=1)
    ap.add_argument("--no-other-configs", action="store_true", help="skip the cfg1 / cfg3 decode runs")
    ap.add_argument("--no-churn", action="store_true", help="skip the cfg4 continuous-batching churn run")
    ap.add_argument("--churn-only", action="store_true",
                    help="run only the cfg4 churn loop and print its entry (the command of the churn kernel trace)")
    ap.add_argument("--no-engine", action="store_true", help="skip the run through the llm_hip host engine")
    ap.add_argument("--no-layer-slab", action="store_true", help="skip the decode runs inside a 32-layer slab")
    ap.add_argument("--sections", default="all",
                    help="comma-separated subset of the secondary measurements to run: probes, prefill (cfg2 prefill "
                         "part, fused mixed call, rope + cache write), engine, churn, layer_slab, other (cfg1, cfg3, "
                         "8k prompts, chunked prefill, general kernels), prefill_lengths (32 768 prompt tokens as prompts of 128 ... "
                         "8 192 tokens), cpu; the headline decode loop always runs")
    ap.add_argument("--quick", action="store_true",
                    help="a dozen calls per secondary figure instead of >= 100 calls and >= 200 ms: for counter runs "
                         "(rocprofv3 --pmc serialises dispatches), not for reported timings")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device-to-device copy (the reference point for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run of this same command)")
    return ap.parse_args()


class DeviceBatch:
    """Device-resident tensors + argument block of one MHCA call; history is quantised by the library itself."""

    def __init__(self, pkg, lib, b, seed, n_slabs, split_k=1, cache_prefill=0, layout=0, layers=None):
        """layers: instead of n_slabs separate one-layer slabs, ONE slab of b.num_layer layers whose listed layers all
        hold the history; the steps rotate over them (distinct memory per step, like the slab rotation, inside a slab
        of the size a whole model allocates). layout: cache_layout 0 (MaxT, L, 2, KVH, Dh) or 3 (L, 2, KVH, MaxT, Dh)."""
        import torch
        from ppl_nn_amd import cabi
        self.pkg, self.lib, self.b, self.cabi = pkg, lib, b, cabi
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        S, Hs = b.total_new_tokens, b.total_hist_tokens
        f16 = dict(dtype=torch.float16, device="cuda")
        self.q = torch.randn((S, b.num_heads, b.head_dim), generator=g, **f16)
        self.k = torch.randn((S, b.num_kv_heads, b.head_dim), generator=g, **f16)
        self.v = torch.randn((S, b.num_kv_heads, b.head_dim), generator=g, **f16)
        self.out = torch.zeros((S, b.num_heads, b.head_dim), **f16)
        i64 = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).cuda()
        self.seqstarts, self.kvstarts = i64(b.seqstarts), i64(b.kvstarts)
        self.cachestarts, self.start_pos = i64(b.cachestarts), i64(b.start_pos)
        histstarts, zeros = i64(b.histstarts), i64(np.zeros(max(b.batch, 1)))
        if layout == 3:
            shape = (b.num_layer, 2, b.num_kv_heads, b.max_tokens, b.head_dim)
            st = cabi.cache_strides_layout3(b.num_layer, b.num_kv_heads, b.head_dim, b.max_tokens)
        else:
            shape = (b.max_tokens, b.num_layer, 2, b.num_kv_heads, b.head_dim)
            st = cabi.cache_strides_layout0(b.num_layer, b.num_kv_heads, b.head_dim)
        self.slabs = []
        self.stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        ptr = lambda t: C.c_void_p(t.data_ptr())
        # (slab, layer) of every step of the rotation
        places = [(0, l) for l in layers] if layers else [(s, b.layer_idx) for s in range(n_slabs)]
        for s in range(1 if layers else n_slabs):
            cache = torch.zeros(shape, dtype=torch.int8, device="cuda")
            scale = torch.zeros(shape[:-1] + (b.head_dim // 8,), **f16)
            self.slabs.append((cache, scale))
        for slab, layer in places:
            cache, scale = self.slabs[slab]
            if Hs:
                hk = torch.randn((Hs, b.num_kv_heads, b.head_dim), generator=g, **f16)
                hv = torch.randn((Hs, b.num_kv_heads, b.head_dim), generator=g, **f16)
                w = cabi.KvWriteArgs()
                w.d_current_key, w.d_current_value = ptr(hk), ptr(hv)
                w.d_seqstarts, w.d_cachestarts, w.d_start_pos = ptr(histstarts), ptr(self.cachestarts), ptr(zeros)
                w.batch, w.total_new_tokens = b.batch, Hs
                w.layer_idx, w.num_layer, w.num_kv_heads, w.head_dim = layer, b.num_layer, b.num_kv_heads, b.head_dim
                for kk, vv in st.items():
                    setattr(w, kk, vv)
                w.d_cache, w.d_scale = ptr(cache), ptr(scale)
                pkg.check(lib.pplhip_kv_quantize_write(C.byref(w), self.stream), "history write")
                torch.cuda.synchronize()
                del hk, hv
        self.args = []
        for slab, layer in places:
            cache, scale = self.slabs[slab]
            a = cabi.MhcaArgs()
            a.d_query, a.d_current_key, a.d_current_value = ptr(self.q), ptr(self.k), ptr(self.v)
            a.d_seqstarts, a.d_kvstarts = ptr(self.seqstarts), ptr(self.kvstarts)
            a.d_cachestarts, a.d_start_pos = ptr(self.cachestarts), ptr(self.start_pos)
            a.is_causal, a.batch, a.decoding_batches = 1, b.batch, b.decoding_batches
            a.max_seqlen, a.max_kvlen = b.max_seqlen, b.max_kvlen
            a.layer_idx, a.num_layer = layer, b.num_layer
            a.num_heads, a.num_kv_heads, a.head_dim = b.num_heads, b.num_kv_heads, b.head_dim
            a.cache_mode, a.page_size = 0, 128
            for kk, vv in st.items():
                setattr(a, kk, vv)
            a.enable_decoding_sharemem_mhca = a.enable_decoding_infinity_mhca = a.enable_decoding_infinity_gqca = 1
            a.specify_decoding_attn_split_k = split_k
            a.enable_cache_prefill = cache_prefill
            a.d_cache, a.d_scale, a.d_output = ptr(cache), ptr(scale), ptr(self.out)
            a.total_new_tokens = S
            self.args.append(a)
        self.plan = cabi.MhcaPlan()
        pkg.check(lib.pplhip_mhca_prepare(C.byref(self.args[0]), C.byref(self.plan)), "prepare")
        self.ws = torch.empty(max(int(self.plan.workspace_bytes), 256), dtype=torch.uint8, device="cuda")
        self.ws_ptr = ptr(self.ws)

    def step(self, i):
        a = self.args[i % len(self.args)]
        rc = self.lib.pplhip_mhca_forward(C.byref(a), C.byref(self.plan), self.ws_ptr, self.stream)
        if rc:
            self.pkg.check(rc, "mhca_forward")


def timed(db, steps, warmup):
    """W untimed steps, then exactly K steps bracketed by synchronize; returns (wall ms/step, event ms/step)."""
    import torch
    for i in range(warmup):
        db.step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        db.step(i)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, e0.elapsed_time(e1) / steps


QUICK = False  # --quick: a dozen calls per figure (counter collection), set by main()


def timed_robust(step, min_warmup=20, min_iters=100, min_ms=200.0, batches=10):
    """For the secondary figures: at least `min_warmup` untimed calls, then at least `min_iters` calls and `min_ms` of
    device time whatever --steps says, timed with events on the launch stream in `batches` equal batches.
    Returns (mean ms per call, median over the batches of ms per call, calls timed)."""
    import torch
    if QUICK:
        min_warmup, min_iters, min_ms, batches = 2, 10, 0.0, 2
    for i in range(min_warmup):
        step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    probe = max(min_iters // batches, 1)
    e0.record()
    for i in range(probe):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    per_call = max(e0.elapsed_time(e1) / probe, 1e-4)
    per_batch = max(-(-min_iters // batches), int(min_ms / per_call / batches) + 1)
    times = []
    k = 0
    for _ in range(batches):
        e0.record()
        for _ in range(per_batch):
            step(k)
            k += 1
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) / per_batch)
    return float(np.mean(times)), float(np.median(times)), per_batch * batches


def cpu_baseline(db, threads, min_seconds=10.0, max_prepare=24):
    """The decode part run through the x86 engine on the host cores: per sequence the fp32 ONNX attention subgraph
    (Transpose, MatMul, Mul, Add of a mask, Softmax, MatMul) over the sequence's dequantised K/V, loaded by the engine
    library's ONNX reader -- PPLNN-x86-semantics baseline with this build's own kernels (the reference's x86 arithmetic
    lives in its un-vendored ppl.kernel.cpu). A bounded sample: the first `max_prepare` decode sequences, repeated
    until about `min_seconds` of CPU work has been timed, once with `threads` OpenMP threads and once with 1."""
    from ppl_nn_amd import x86_baseline
    b = db.b
    cache, scale = db.slabs[0]
    n = min(b.decoding_batches, max_prepare)
    cases = []
    for i in range(n):
        kv = int(b.kvlens[i])
        rows = slice(int(b.cachestarts[i]), int(b.cachestarts[i]) + kv)
        deq = cache[rows, b.layer_idx].float() * scale[rows, b.layer_idx].float().repeat_interleave(8, dim=-1)
        k = deq[:, 0].permute(1, 0, 2).contiguous().cpu().numpy()  # [KVH, kv, Dh]
        v = deq[:, 1].permute(1, 0, 2).contiguous().cpu().numpy()
        s0 = int(b.seqstarts[i])
        q = db.q[s0:s0 + 1].float().permute(1, 0, 2).contiguous().cpu().numpy()  # [H, 1, Dh]
        cases.append((q, k, v, x86_baseline.causal_mask(1, kv)))

    def measure(nthreads, seconds):
        ab = x86_baseline.AttentionBaseline(b.head_dim, num_threads=nthreads)
        done, spent, passes = 0, 0.0, 0
        while spent < seconds:
            t0 = time.perf_counter()
            for q, k, v, m in cases:
                ab.run(q, k, v, m)
            dt = time.perf_counter() - t0
            if passes > 0:  # the first pass warms caches and the OpenMP pool
                spent += dt
                done += len(cases)
            passes += 1
        used = ab.num_threads
        ab.close()
        return done / spent, used, passes - 1, spent

    rate, used, passes, spent = measure(threads, min_seconds)
    rate1, _, passes1, spent1 = measure(1, min_seconds / 2)
    return dict(value=rate, unit="tokens/s", cores=used, kind="port", value_1_thread=rate1,
                host_cpus=os.cpu_count(), engine="x86 (own fp32 kernels behind the engine boundary)",
                sample=f"first {n} of {b.decoding_batches} decode sequences of the workload x {passes} passes "
                       f"({spent:.1f} s) with {used} threads, x {passes1} passes ({spent1:.1f} s) with 1 thread; per "
                       f"sequence the ONNX subgraph Transpose-MatMul-Mul-Add-Softmax-MatMul in fp32 on dequantised K/V "
                       f"resident in host memory")


def probe_check(probes, rc, what):
    if rc:
        raise RuntimeError("%s failed: %d: %s" % (what, rc, probes.pplhip_probe_last_error().decode()))


def mfma_sustained(probes):
    """TFLOP/s of a bare v_mfma_f32_32x32x16_f16 loop on the whole chip, with all-zero and with random fp16 operands:
    the clock the chip holds depends on how many operand bits toggle."""
    import torch
    out = {}
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    dst = torch.empty(1024 * 256, dtype=torch.float32, device="cuda")
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    for name, ops in (("zeros", torch.zeros(2048 * 8, dtype=torch.float16, device="cuda")),
                      ("random_normal", torch.randn(2048 * 8, generator=g, dtype=torch.float16, device="cuda"))):
        flops = C.c_double()
        call = lambda i: probe_check(probes, probes.pplhip_probe_mfma_f16(
            C.c_void_p(ops.data_ptr()), C.c_void_p(dst.data_ptr()), 1024, 2000, C.byref(flops), stream), "mfma probe")
        mean_ms, med_ms, _ = timed_robust(call, min_warmup=3, min_iters=10, min_ms=100.0, batches=5)
        out[name] = flops.value / (med_ms * 1e-3) / 1e12
    return out


def hbm_sustained(probes):
    """GB/s of a plain streaming read of 2 GiB (eight times the memory-side cache) by 512 / 2048 / 8192 workgroups:
    the practical ceiling of this box beside the published HBM peak."""
    import torch
    n = 2 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").fill_(1)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for wgs in (512, 2048, 8192):
        dst = torch.empty(wgs * 256, dtype=torch.int32, device="cuda")
        got = C.c_uint64()
        call = lambda i: probe_check(probes, probes.pplhip_probe_hbm_read(
            C.c_void_p(src.data_ptr()), n, C.c_void_p(dst.data_ptr()), wgs, C.byref(got), stream), "hbm probe")
        _, med_ms, _ = timed_robust(call, min_warmup=3, min_iters=20, min_ms=100.0, batches=5)
        out["%d_workgroups" % wgs] = got.value / (med_ms * 1e-3) / 1e9
    del src
    torch.cuda.empty_cache()
    return out


PROFILE_TRAFFIC = os.path.join(ROOT, "profiles", "decode_int8kv_cfg2_hbm_traffic.txt")


def recorded_traffic(workload):
    """HBM bytes per decode launch measured offline with rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE, scaled by the
    copy-kernel factor); the summary file carries the commands. None when no figure is recorded for the workload."""
    if workload != "cfg2" or not os.path.exists(PROFILE_TRAFFIC):
        return None
    with open(PROFILE_TRAFFIC) as f:
        for line in f:
            if line.startswith("traffic_bytes_per_launch="):
                return float(line.split("=", 1)[1])
    return None


def copy_calibration():
    import torch
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(3)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()


def churn_cfg4(pkg, lib, steps=100, warm_steps=5):
    """Continuous-batching churn (Llama-2-13B shape, H = KVH = 40): 256 slots, every step the tables are rebuilt on
    the GPU by pplhip_pack_tables from the slot state (the same launch grows the slots for the next step), and one
    mixed MultiHeadCacheAttention call runs on them. The host only supplies the sizes its scheduler knows anyway (batch,
    decoding_batches, maxima), precomputed for the seeded schedule; no table is uploaded and nothing is read back."""
    import torch
    from ppl_nn_amd import cabi, workloads
    sch = workloads.ChurnSchedule(seed=2)
    n, H, KVH, Dh = sch.num_slots, sch.num_heads, sch.num_kv_heads, sch.head_dim
    dev = "cuda"
    ptr = lambda t: C.c_void_p(t.data_ptr())
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    max_tokens = n * sch.region
    cache = torch.zeros((max_tokens, 1, 2, KVH, Dh), dtype=torch.int8, device=dev)
    scale = torch.zeros((max_tokens, 1, 2, KVH, Dh // 8), dtype=torch.float16, device=dev)
    plans, host = [], []
    for _ in range(steps + warm_steps):
        kv, nl = sch.next_step()
        is_dec = (nl == 1) & (kv > 0)
        host.append(dict(kv=kv, nl=nl, nd=int(is_dec.sum()), batch=int((nl > 0).sum()), S=int(nl.sum()),
                         max_seqlen=int(nl.max()), max_kvlen=int((kv + nl).max()),
                         dec_kv=int((kv + nl)[is_dec].sum()),
                         prefill_flops=int(sum(4 * H * Dh * (int(l) * (int(l) + 1) // 2) for l in nl[~is_dec & (nl > 0)]))))
    max_S = max(h["S"] for h in host)
    g = torch.Generator(device=dev)
    g.manual_seed(4)
    q = torch.randn((max_S, H, Dh), generator=g, dtype=torch.float16, device=dev)
    k = torch.randn((max_S, KVH, Dh), generator=g, dtype=torch.float16, device=dev)
    v = torch.randn((max_S, KVH, Dh), generator=g, dtype=torch.float16, device=dev)
    out = torch.zeros((max_S, H, Dh), dtype=torch.float16, device=dev)
    i64 = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(dev)
    slot_kv = i64(np.zeros(n))
    slot_cs = i64(sch.cachestart)
    # per-step new-token counts are the scheduler's decision: staged on the device before the timed loop
    slot_nl = [i64(h["nl"]) for h in host]
    slot_kv_reset = [i64(h["kv"]) for h in host]  # retirements reset a slot to 0 (the scheduler's decision too)
    seqstarts = torch.zeros(n + 1, dtype=torch.int64, device=dev)
    kvstarts = torch.zeros(n + 1, dtype=torch.int64, device=dev)
    cachestarts = torch.zeros(n, dtype=torch.int64, device=dev)
    start_pos = torch.zeros(n, dtype=torch.int64, device=dev)
    batch_slots = torch.zeros(n, dtype=torch.int64, device=dev)
    header = torch.zeros(6, dtype=torch.int64, device=dev)
    st = cabi.cache_strides_layout0(1, KVH, Dh)
    calls = []
    ws_bytes = 256
    for i, h in enumerate(host):
        pa = cabi.PackArgs()
        pa.d_slot_kvlen, pa.d_slot_newlen, pa.d_slot_cachestart = ptr(slot_kv), ptr(slot_nl[i]), ptr(slot_cs)
        pa.num_slots, pa.advance_slots = n, 1  # the slot state moves on inside the pack launch
        pa.d_seqstarts, pa.d_kvstarts, pa.d_cachestarts = ptr(seqstarts), ptr(kvstarts), ptr(cachestarts)
        pa.d_start_pos, pa.d_batch_slots, pa.d_header = ptr(start_pos), ptr(batch_slots), ptr(header)
        a = cabi.MhcaArgs()
        a.d_query, a.d_current_key, a.d_current_value = ptr(q), ptr(k), ptr(v)
        a.d_seqstarts, a.d_kvstarts, a.d_cachestarts, a.d_start_pos = ptr(seqstarts), ptr(kvstarts), ptr(cachestarts), ptr(start_pos)
        a.is_causal, a.batch, a.decoding_batches = 1, h["batch"], h["nd"]
        a.max_seqlen, a.max_kvlen = h["max_seqlen"], h["max_kvlen"]
        a.layer_idx, a.num_layer, a.num_heads, a.num_kv_heads, a.head_dim = 0, 1, H, KVH, Dh
        a.cache_mode, a.page_size = 0, 128
        for kk, vv in st.items():
            setattr(a, kk, vv)
        a.specify_decoding_attn_split_k = 1
        a.d_cache, a.d_scale, a.d_output = ptr(cache), ptr(scale), ptr(out)
        a.total_new_tokens = h["S"]
        plan = cabi.MhcaPlan()
        pkg.check(lib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)), "prepare(churn)")
        ws_bytes = max(ws_bytes, int(plan.workspace_bytes))
        calls.append((pa, a, plan))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

    def step(i):
        pa, a, plan = calls[i]
        slot_kv.copy_(slot_kv_reset[i])  # device-to-device: applies the scheduler's retirements
        rc = lib.pplhip_pack_tables(C.byref(pa), stream)
        rc = rc or lib.pplhip_mhca_forward(C.byref(a), C.byref(plan), ptr(ws), stream)
        if rc:
            pkg.check(rc, "churn step")

    for i in range(warm_steps):
        step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(warm_steps, warm_steps + steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    # the table rebuild alone (same slot state every call; one workgroup, latency-bound)
    pack_only = calls[-1][0]
    pack_only.advance_slots = 0  # (timed on a fixed slot state, after the loop's own check below has used it)
    timed = host[warm_steps:]
    dec_tokens = sum(h["nd"] for h in timed)
    dec_bytes = sum(h["dec_kv"] for h in timed) * 2.5 * KVH * Dh
    flops = sum(h["prefill_flops"] for h in timed)
    # check the on-device state against the host mirror once, after the timed region
    assert np.array_equal(slot_kv.cpu().numpy(), host[-1]["kv"] + host[-1]["nl"]), "slot state diverged"
    pack_mean, pack_med, _ = timed_robust(lambda i: lib.pplhip_pack_tables(C.byref(pack_only), stream), min_ms=50.0)
    # roofline of a step: the decode sequences' cache bytes at the HBM peak and the prompts' causal flops at the fp16
    # matrix peak; the step cannot be shorter than the larger of the two and, where the two do not overlap, than their
    # sum. Both fractions are given against the measured step (pack + attention + advance).
    new_tokens = sum(h["S"] for h in timed)
    write_bytes = new_tokens * 2 * KVH * Dh * (2 + 1.25)  # fp16 K/V rows read, int8 + scales written
    qo_bytes = 2 * new_tokens * H * Dh * 2
    step_bytes = (dec_bytes + write_bytes + qo_bytes) / steps
    t_hbm_us = step_bytes / (HBM_PEAK_GBS * 1e9) * 1e6
    t_mfma_us = flops / steps / (MFMA_FP16_PEAK_TFLOPS * 1e12) * 1e6
    return {"workload": "cfg4 churn: 256 slots x %d steps, H=KVH=40, Dh 128, retire p=0.02, prompts U[32,512], tables "
                        "rebuilt on the GPU every step" % steps,
            "ms_per_step": ms, "pack_tables_us": {"mean": pack_mean * 1e3, "median": pack_med * 1e3},
            "decode_tokens_per_s": dec_tokens / (ms * steps * 1e-3),
            "decode_kv_GB_per_step": dec_bytes / steps / 1e9, "prefill_GFLOP_per_step": flops / steps / 1e9,
            "decode_GBps_if_step_were_decode_only": dec_bytes / (ms * steps * 1e-3) / 1e9,
            "roofline": {"bound": "hbm", "algorithmic_bytes_per_step": step_bytes,
                         "achieved": step_bytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": t_hbm_us / (ms * 1e3), "hbm_us_at_peak": t_hbm_us, "mfma_us_at_peak": t_mfma_us,
                         "frac_if_bytes_and_flops_do_not_overlap": (t_hbm_us + t_mfma_us) / (ms * 1e3),
                         "note": "bytes: int8 K/V + scales of the decode sequences, Q/O, fp16 K/V of the new tokens read "
                                 "and their int8 rows written; flops: causal prompt attention; step = pack_tables (which also advances the "
                                 "slot state) + one mixed MultiHeadCacheAttention call"}}


def engine_run(pkg, lib, db):
    """The same MultiHeadCacheAttention call through the llm_hip host engine: a one-node OPMX graph loaded by the ONNX
    wire reader, run by Runtime::RunAsync on the caller's stream (the reference's wrapper reads three host scalars,
    computes the strides, plans, takes a workspace from the device's buffer manager and frees it again:
    multi_head_cache_attention_kernel.cc:116-132,218-228), beside the bare C-ABI call on the SAME slab. Also the node's
    time as the runtime's own profiling reports it (tools/pplnn_llm.cc:892-990 prints these per kernel)."""
    import torch
    from ppl_nn_amd import onnx_writer as ow
    eng = pkg.load_engine_library()
    b = db.b
    stream = torch.cuda.current_stream().cuda_stream
    engine = eng.pplnn_hip_engine_create_on_stream(0, 1, C.c_void_p(stream))
    builder = eng.pplnn_hip_builder_create()
    model = ow.mhca_model(b.num_heads, b.num_kv_heads, b.head_dim, b.num_layer, b.layer_idx)

    def ok(rc, what):
        if rc:
            raise RuntimeError("%s failed: %d: %s" % (what, rc, eng.pplnn_hip_last_error().decode()))
    ok(eng.pplnn_hip_builder_load_model(builder, model, len(model)), "load_model")
    ok(eng.pplnn_hip_builder_set_engine(builder, engine), "set_engine")
    ok(eng.pplnn_hip_builder_preprocess(builder), "preprocess")
    rt = eng.pplnn_hip_builder_create_runtime(builder)
    if not rt:
        raise RuntimeError("create_runtime failed: " + eng.pplnn_hip_last_error().decode())
    cache, scale = db.slabs[0]
    keep = []

    def dims_of(shape):
        return (C.c_int64 * len(shape))(*shape), len(shape)

    def borrow(i, t):  # caller-owned device memory, like the KV slab
        tensor = eng.pplnn_hip_runtime_input(rt, i)
        d, n = dims_of(tuple(t.shape))
        eng.pplnn_hip_tensor_reshape(tensor, d, n)
        eng.pplnn_hip_tensor_set_buffer_ptr(tensor, t.data_ptr())

    def host_scalar(i, v):
        tensor = eng.pplnn_hip_runtime_input(rt, i)
        eng.pplnn_hip_tensor_use_host_device(tensor)
        eng.pplnn_hip_tensor_reshape(tensor, None, 0)
        a = np.array([v], np.int64)
        keep.append(a)
        ok(eng.pplnn_hip_tensor_copy_from_host(tensor, a.ctypes.data), "scalar")
    for i, t in enumerate((db.q, db.k, db.v, db.seqstarts, db.kvstarts, db.cachestarts, db.start_pos)):
        borrow(i, t)
    for i, v in enumerate((b.decoding_batches, b.max_seqlen, b.max_kvlen)):
        host_scalar(7 + i, v)
    borrow(10, cache)
    borrow(11, scale)

    def via_engine(i):
        rc = eng.pplnn_hip_runtime_run_async(rt)
        if rc:
            ok(rc, "RunAsync")

    a0, plan = db.args[0], db.plan

    def via_cabi(i):
        rc = lib.pplhip_mhca_forward(C.byref(a0), C.byref(plan), db.ws_ptr, db.stream)
        if rc:
            pkg.check(rc, "mhca_forward")
    res = {}
    for rnd in range(2):  # interleaved, the second round is reported
        e_mean, e_med, e_n = timed_robust(via_engine)
        c_mean, c_med, c_n = timed_robust(via_cabi)
    # wall clock of a queue of calls as well: the host side of the engine call must keep ahead of the GPU
    def wall(fn, n=300):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            fn(i)
        host = (time.perf_counter() - t0) / n
        torch.cuda.synchronize()
        return host * 1e6, (time.perf_counter() - t0) / n * 1e6
    e_host, e_wall = wall(via_engine)
    c_host, c_wall = wall(via_cabi)
    # the runtime's own per-kernel profile (each profiled run waits for its kernel's end event)
    ok(eng.pplnn_hip_runtime_set_profiling(rt, 1), "profiling on")
    runs = 50
    for _ in range(runs):
        ok(eng.pplnn_hip_runtime_run(rt), "Run")
    micros, counts = (C.c_uint64 * 4)(), (C.c_uint32 * 4)()
    nk = eng.pplnn_hip_runtime_profiling(rt, micros, counts, 4)
    ok(eng.pplnn_hip_runtime_set_profiling(rt, 0), "profiling off")
    torch.cuda.synchronize()
    eng.pplnn_hip_runtime_destroy(rt)
    eng.pplnn_hip_builder_destroy(builder)
    eng.pplnn_hip_engine_destroy(engine)
    return {"workload": "decode part of the workload, one slab (no rotation), MultiHeadCacheAttention as a one-node graph",
            "engine_run_async_us": e_med * 1e3, "cabi_call_us": c_med * 1e3, "engine_minus_cabi_us": (e_med - c_med) * 1e3,
            "calls_timed": e_n, "host_us_per_engine_call": e_host, "host_us_per_cabi_call": c_host,
            "wall_us_per_engine_call": e_wall, "wall_us_per_cabi_call": c_wall,
            "profiling": {"kernels": int(nk), "exec_count": int(counts[0]),
                          "avg_us_per_run": micros[0] / max(int(counts[0]), 1),
                          "note": "GetProfilingStatistics of the node: HIP events around the op on an idle stream, "
                                  "so the host time between the first event and the first launch is inside"}}


def rope_cache_write(pkg, lib, b):
    """RotaryPositionEmbedding followed by the quantize-on-write of the same new tokens (two launches) against the
    one launch that does both, on the packed new tokens of batch `b` (decode tokens and prompts); HBM-bound streaming:
    the algorithmic bytes are Q, K read + written, V read, and the int8 + scale bytes written."""
    import torch
    from ppl_nn_amd import cabi
    S, H, KVH, Dh = b.total_new_tokens, b.num_heads, b.num_kv_heads, b.head_dim
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    f16 = dict(dtype=torch.float16, device="cuda")
    q = torch.randn((S, H, Dh), generator=g, **f16)
    k = torch.randn((S, KVH, Dh), generator=g, **f16)
    v = torch.randn((S, KVH, Dh), generator=g, **f16)
    qo, ko = torch.empty_like(q), torch.empty_like(k)
    i64 = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).cuda()
    ss, sp, cs = i64(b.seqstarts), i64(b.start_pos), i64(b.cachestarts)
    cache = torch.zeros((b.max_tokens, 1, 2, KVH, Dh), dtype=torch.int8, device="cuda")
    scale = torch.zeros((b.max_tokens, 1, 2, KVH, Dh // 8), **f16)
    ptr = lambda t: C.c_void_p(t.data_ptr())
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    r = cabi.RopeArgs()
    r.d_query, r.d_key, r.d_start_pos, r.d_seqstarts = ptr(q), ptr(k), ptr(sp), ptr(ss)
    r.theta, r.bypass_key, r.rotary_dim, r.pair_layout = 500000.0, 0, 0, 0
    r.batch, r.total_tokens, r.num_heads, r.num_key_heads, r.head_dim = b.batch, S, H, KVH, Dh
    r.max_position_embeddings, r.max_seqlen, r.scaling_type, r.scaling_factor = 8192, b.max_seqlen, 0, 1.0
    r.d_rotated_query, r.d_rotated_key = ptr(qo), ptr(ko)
    w = cabi.KvWriteArgs()
    w.d_current_key, w.d_current_value = ptr(ko), ptr(v)
    w.d_seqstarts, w.d_cachestarts, w.d_start_pos = ptr(ss), ptr(cs), ptr(sp)
    w.batch, w.total_new_tokens, w.layer_idx, w.num_layer, w.num_kv_heads, w.head_dim = b.batch, S, 0, 1, KVH, Dh
    for kk, vv in cabi.cache_strides_layout0(1, KVH, Dh).items():
        setattr(w, kk, vv)
    w.d_cache, w.d_scale = ptr(cache), ptr(scale)

    def two(i):
        rc = lib.pplhip_rope_forward(C.byref(r), stream) or lib.pplhip_kv_quantize_write(C.byref(w), stream)
        if rc:
            pkg.check(rc, "rope + write")

    def one(i):
        rc = lib.pplhip_rope_kv_write_forward(C.byref(r), C.byref(w), stream)
        if rc:
            pkg.check(rc, "rope_kv_write")

    _, two_ms, _ = timed_robust(two, min_ms=50.0)
    _, one_ms, n = timed_robust(one, min_ms=50.0)
    byts = S * (2 * (H + KVH) * Dh * 2 + KVH * Dh * 2 + 2 * KVH * (Dh + Dh // 4))
    return {"workload": "new tokens of the mixed batch: %d tokens, H%d/KVH%d/Dh%d" % (S, H, KVH, Dh),
            "two_launches_us": two_ms * 1e3, "one_launch_us": one_ms * 1e3, "calls_timed": n,
            "algorithmic_bytes": byts, "one_launch_GBs": byts / (one_ms * 1e-3) / 1e9}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the attention path has no collective: it would shard by kv head, "
              "every GPU holding its heads' slice of the cache). Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch
    pkg = entry.load_package()
    lib = pkg.load_library()
    probes = pkg.load_probe_library()  # roofline probes: measurement aids, not part of the drop-in ABI
    from ppl_nn_amd import workloads
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback.", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)

    if args.workload == "cfg2":
        full = workloads.cfg2_llama3_8b_mixed()
        dec_b, pre_b = workloads.cfg2_decode_part(), workloads.cfg2_prefill_part()
        wname = "cfg2 Llama-3-8B mixed ragged batch (H32/KVH8/Dh128, int8 group-8 KV): decode part 120 seqs kv~U[256,4096]"
    elif args.workload == "cfg1":
        full, pre_b = None, None
        dec_b = workloads.cfg1_llama2_7b_decode()
        wname = "cfg1 Llama-2-7B pure decode (H32/KVH32/Dh128): 64 seqs kv~U[128,2048]"
    else:
        full, pre_b = None, None
        dec_b = workloads.cfg3_long_context()
        wname = "cfg3 long-context decode (H8/KVH1/Dh128): 8 seqs kv~U[32768,131072]"

    global QUICK
    QUICK = args.quick
    sections = set(x.strip() for x in args.sections.split(","))

    def want(name):
        return "all" in sections or name in sections
    if args.churn_only:
        print(json.dumps({"churn_cfg4": churn_cfg4(pkg, lib, steps=20 if QUICK else 100)}))
        return
    # the two roofline probes run first: what this box sustains, measured before anything else has heated the chip
    stream_gbs = hbm_sustained(probes) if want("probes") else None
    sustained = mfma_sustained(probes) if pre_b is not None and want("probes") else None

    dec = DeviceBatch(pkg, lib, dec_b, seed=1, n_slabs=N_SLABS, split_k=args.split_k)
    wall_ms, ev_ms = timed(dec, args.steps, args.warmup)
    _, dec_med_ms, dec_n = timed_robust(dec.step)
    nd = dec_b.decoding_batches
    dec_bytes = dec_b.decode_bytes()
    gbs = dec_bytes / (ev_ms * 1e-3) / 1e9
    result = {
        "metric": "decode attn tokens/s + % of HBM roofline; prefill attn TFLOPS, Llama-3-8B shape",
        "value": nd / (wall_ms * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 KV + fp16 (fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": wname, "decode_seqs": nd, "kv_tokens": int(dec_b.kvlens.sum()),
                   "decode_ranges": int(dec.plan.decode_num_ranges), "kv_heads_per_workgroup": int(dec.plan.decode_heads_per_block),
                   "slabs_rotated": N_SLABS},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs / HBM_PEAK_GBS, "traffic": recorded_traffic(args.workload),
                     "kernel": "decode_int8kv_kernel (reads the int8 slab once, quantises the new tokens into it) + decode_merge in the same call",
                     "algorithmic_bytes_per_launch": dec_bytes, "event_ms_per_launch": ev_ms,
                     "median_ms_per_launch_long_run": dec_med_ms, "long_run_calls": dec_n,
                     "traffic_source": "recorded rocprofv3 --pmc summary under profiles/ (not re-measured in this run)"},
    }
    if stream_gbs:
        result["hbm_read_sustained_GBs"] = dict(
            stream_gbs, note="plain streaming read of 2 GiB measured in this run; the published peak is %.0f" % HBM_PEAK_GBS)
        result["roofline"]["frac_of_sustained_hbm_read"] = gbs / max(stream_gbs.values())

    def frac(tflops):
        return tflops / MFMA_FP16_PEAK_TFLOPS

    if sustained:
        result["mfma_f16_sustained_tflops"] = dict(
            sustained, note="bare v_mfma_f32_32x32x16_f16 loop on all CUs, measured in this run; the published peak is "
                            "%.0f" % MFMA_FP16_PEAK_TFLOPS)

    def prefill_entry(db, bb, extra=None):
        mean_ms, med_ms, n = timed_robust(db.step)
        fl = bb.prefill_flops()
        tf = fl / (med_ms * 1e-3) / 1e12
        e = {"tflops": tf, "ms": med_ms, "ms_mean": mean_ms, "calls_timed": n, "flops": fl,
             "frac_of_fp16_mfma_peak": frac(tf), "peak_tflops": MFMA_FP16_PEAK_TFLOPS}
        if sustained:
            e["frac_of_sustained_mfma_random_operands"] = tf / sustained["random_normal"]
        e.update(extra or {})
        return e

    if pre_b is not None and want("prefill"):
        pre = DeviceBatch(pkg, lib, pre_b, seed=2, n_slabs=1)
        result["prefill"] = prefill_entry(pre, pre_b, {"prefill_seqs": pre_b.batch, "prefill_tokens": pre_b.total_new_tokens})
        del pre
        mixed = DeviceBatch(pkg, lib, full, seed=3, n_slabs=N_SLABS)
        mix_mean, mix_med, _ = timed_robust(mixed.step)
        result["fused_mixed_call_ms"] = mix_med
        result["fused_mixed_call_ms_mean"] = mix_mean
        del mixed
        result["rope_cache_write"] = rope_cache_write(pkg, lib, full)
    if not args.no_engine and want("engine"):
        result["engine_run"] = engine_run(pkg, lib, dec)
    if args.workload == "cfg2" and not args.no_churn and want("churn"):
        del dec.slabs[1:], dec.args[1:]
        torch.cuda.empty_cache()
        result["churn_cfg4"] = churn_cfg4(pkg, lib)
    if args.workload == "cfg2" and not args.no_layer_slab and want("layer_slab"):
        # the same decode call inside the slab a whole model allocates (tools/benchmark_llama/text_generator.cc:200-211:
        # one cache tensor for all layers): 32 layers, the steps rotate over layers 28..31 so that every step reads
        # memory the previous ones did not (the role the rotated slabs play above)
        ls = {}
        for layout, name in ((0, "cache_layout_0 (MaxT, 32, 2, KVH, Dh): 64 KiB between a head group's tokens"),
                             (3, "cache_layout_3 (32, 2, KVH, MaxT, Dh): a head's tokens 128 bytes apart")):
            lb = workloads.Batch(32, 8, 128, dec_b.seqlens, dec_b.start_pos, dec_b.decoding_batches, num_layer=32,
                                 layer_idx=31, name="cfg2 decode part in a 32-layer slab")
            ldb = DeviceBatch(pkg, lib, lb, seed=1, n_slabs=1, split_k=args.split_k, layout=layout, layers=[28, 29, 30, 31])
            l_mean, l_med, l_n = timed_robust(ldb.step)
            l_gbs = lb.decode_bytes() / (l_med * 1e-3) / 1e9
            ls["cache_layout_%d" % layout] = {"layout": name, "ms_per_step": l_med, "ms_per_step_mean": l_mean,
                                              "calls_timed": l_n, "achieved_GBs": l_gbs,
                                              "frac_of_hbm_peak": l_gbs / HBM_PEAK_GBS, "layers_rotated": [28, 29, 30, 31],
                                              "slab_GB": (ldb.slabs[0][0].numel() + 2 * ldb.slabs[0][1].numel()) / 1e9}
            del ldb
            torch.cuda.empty_cache()
        result["decode_in_32_layer_slab"] = ls
    if args.workload == "cfg2" and not args.no_other_configs and want("other"):
        # the other decode configurations at their full sizes
        others = {}
        # (cfg1 twice: in cache_layout 0 the scale rows of 32 kv heads are 128 bytes per token and workgroup at a 2 KB
        # stride, which the memory system serves at two thirds of the K/V rows' rate; in cache_layout 3 a head's
        # tokens are neighbours)
        for name, ob, olayout in (("cfg1 Llama-2-7B pure decode (H32/KVH32/Dh128): 64 seqs kv~U[128,2048]",
                                   workloads.cfg1_llama2_7b_decode(), 0),
                                  ("cfg1 in cache_layout 3 (L, 2, KVH, MaxT, Dh)", workloads.cfg1_llama2_7b_decode(), 3),
                                  ("cfg3 long-context decode (H8/KVH1/Dh128): 8 seqs kv~U[32768,131072]",
                                   workloads.cfg3_long_context(), 0)):
            odb = DeviceBatch(pkg, lib, ob, seed=4, n_slabs=N_SLABS, layout=olayout)
            o_mean, o_med, o_n = timed_robust(odb.step)
            o_gbs = ob.decode_bytes() / (o_med * 1e-3) / 1e9
            others[name] = {"tokens_per_s": ob.decoding_batches / (o_med * 1e-3), "ms_per_step": o_med,
                            "ms_per_step_mean": o_mean, "calls_timed": o_n,
                            "achieved_GBs": o_gbs, "frac_of_hbm_peak": o_gbs / HBM_PEAK_GBS,
                            "kv_tokens": int(ob.kvlens.sum()), "decode_ranges": int(odb.plan.decode_num_ranges)}
            del odb
            torch.cuda.empty_cache()
        result["other_decode_configs"] = others
        # the prefill kernel away from launch and tail effects: four 8k-token prompts of the same head shape
        import numpy as _np
        lb = workloads.Batch(32, 8, 128, _np.full(4, 8192, _np.int64), _np.zeros(4, _np.int64), 0, name="4x8192 prefill")
        ldb = DeviceBatch(pkg, lib, lb, seed=5, n_slabs=1)
        result["prefill_long_prompts"] = prefill_entry(
            ldb, lb, {"workload": "4 prompts x 8192 tokens, H32/KVH8/Dh128, causal, incl. quantize-on-write"})
        del ldb
        torch.cuda.empty_cache()
        # chunked prefill: every prompt brings a 512-token chunk on top of 4096 tokens already in the int8 slab
        cb = workloads.Batch(32, 8, 128, _np.full(8, 512, _np.int64), _np.full(8, 4096, _np.int64), 0, name="chunked prefill")
        cdb = DeviceBatch(pkg, lib, cb, seed=6, n_slabs=1, cache_prefill=1)
        result["chunked_prefill"] = prefill_entry(
            cdb, cb, {"workload": "8 prompts x (4096 cached + 512 new tokens), H32/KVH8/Dh128, cache-prefill "
                                  "(quantize-on-write, fp16 staging of the cached K/V, attention)",
                      "staged": int(cdb.plan.prefill_staging)})
        del cdb
        torch.cuda.empty_cache()
        # other head dims (the plan's general_kernel route): the cfg2 shapes at head_dim 64, whose decode sequences
        # run the decode kernel over pairs of kv heads (decode_ranges > 0), and at head_dim 96, where they run the
        # general decode kernel
        gen = {}
        for gdh in (64, 96):
            gd = workloads.Batch(32, 8, gdh, dec_b.seqlens, dec_b.start_pos, dec_b.decoding_batches,
                                 name="cfg2 decode part, Dh %d" % gdh)
            gdb = DeviceBatch(pkg, lib, gd, seed=7, n_slabs=N_SLABS)
            g_mean, g_med, g_n = timed_robust(gdb.step)
            gen["decode_cfg2_shape_head_dim_%d" % gdh] = {
                "ms_per_step": g_med, "ms_per_step_mean": g_mean, "calls_timed": g_n,
                "achieved_GBs": gd.decode_bytes() / (g_med * 1e-3) / 1e9,
                "frac_of_hbm_peak": gd.decode_bytes() / (g_med * 1e-3) / 1e9 / HBM_PEAK_GBS,
                "general_kernel": int(gdb.plan.general_kernel), "decode_ranges": int(gdb.plan.decode_num_ranges),
                "general_decode_splits": int(gdb.plan.general_decode_splits)}
            del gdb
            torch.cuda.empty_cache()
        gp = workloads.Batch(32, 8, 64, _np.full(4, 2048, _np.int64), _np.zeros(4, _np.int64), 0, name="4x2048 prefill, Dh 64")
        gpb = DeviceBatch(pkg, lib, gp, seed=8, n_slabs=1)
        gen["prefill_4x2048_head_dim_64"] = prefill_entry(gpb, gp, {"general_kernel": int(gpb.plan.general_kernel)})
        del gpb
        torch.cuda.empty_cache()
        result["general_kernel"] = gen
    if args.workload == "cfg2" and want("prefill_lengths"):
        # 32 768 prompt tokens as prompts of one length: the same 8 192 tile workgroups every time, from 1.5 to 65
        # 64-key steps each -- separates what a workgroup costs from what a step costs
        import numpy as _np
        sweep = {}
        for plen in (128, 256, 512, 1024, 2048, 4096, 8192):
            n = 32768 // plen
            sb = workloads.Batch(32, 8, 128, _np.full(n, plen, _np.int64), _np.zeros(n, _np.int64), 0, name="%dx%d prefill" % (n, plen))
            sdb = DeviceBatch(pkg, lib, sb, seed=9, n_slabs=1)
            tiles = n * (plen // 128) * 32
            steps = n * 32 * sum(2 * (i + 1) for i in range(plen // 128))
            sweep["%d_prompts_x_%d_tokens" % (n, plen)] = prefill_entry(
                sdb, sb, {"tile_workgroups": tiles, "workgroup_steps": steps})
            del sdb
            torch.cuda.empty_cache()
        result["prefill_by_prompt_length"] = sweep
    if args.copy_calibration:
        copy_calibration()
    if not args.no_cpu_baseline and want("cpu"):
        threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
        result["cpu_baseline"] = cpu_baseline(dec, threads)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
