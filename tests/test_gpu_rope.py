"""GPU parity of RotaryPositionEmbedding / PositionIndex through the C ABI against the float64 CPU oracle.
PositionIndex is integer work: bit-exact. Rotated values are fp16 results of float32 arithmetic on float64-reduced
angles: within one fp16 unit in the last place of the oracle's float64 result (tolerance stated in close())."""
import ctypes as C

import numpy as np
import pytest

import harness
from harness import cabi

pytestmark = pytest.mark.gpu


def close(got, want, what):
    ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float64)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bad = err > 1.0 * ulp + 1e-6
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} beyond 1 fp16 ulp, worst {err.max()}"


def run_both(hiplib, olib, q, k, seqlens, start_pos, inplace=False, **kw):
    import torch
    qo, ko = np.zeros_like(q), np.zeros_like(k)
    a = harness.fill_rope_args(cabi.RopeArgs(), q, k, seqlens, start_pos, qo, ko, **kw)
    assert olib.oracle_rope_forward(C.byref(a)) == 0
    dq, dk = harness.to_dev(q), harness.to_dev(k)
    dqo, dko = (dq, dk) if inplace else (torch.zeros_like(dq), torch.zeros_like(dk))
    ss = np.concatenate([[0], np.cumsum(seqlens)]).astype(np.int64)
    tabs = (harness.to_dev(ss), harness.to_dev(np.asarray(start_pos, np.int64)))
    d = harness.fill_rope_args(cabi.RopeArgs(), dq, dk, seqlens, start_pos, dqo, dko, ptr=harness.dev_ptr, tables=tabs,
                               **kw)
    harness.pkg.check(hiplib.pplhip_rope_forward(C.byref(d), None), "rope_forward")
    torch.cuda.synchronize()
    f16 = lambda x: x.cpu().view(torch.int16).numpy().view(np.float16)
    return (qo, ko), (f16(dqo), f16(dko))


@pytest.mark.parametrize("H,KVH,Dh,rd", [(32, 8, 128, 0), (8, 8, 128, 64), (6, 2, 64, 0), (5, 1, 80, 32), (4, 4, 256, 0)])
def test_rope_vs_oracle(hiplib, olib, H, KVH, Dh, rd):
    rng = np.random.default_rng(11)
    seqlens = np.array([1, 1, 37, 1, 130, 5])
    start = np.array([131071, 0, 0, 4095, 900, 65536])
    T = int(seqlens.sum())
    print(f"case rope H={H} KVH={KVH} Dh={Dh} rotary_dim={rd} T={T}", flush=True)
    q = rng.standard_normal((T, H, Dh)).astype(np.float16)
    k = rng.standard_normal((T, KVH, Dh)).astype(np.float16)
    (qo, ko), (gq, gk) = run_both(hiplib, olib, q, k, seqlens, start, theta=500000.0, rotary_dim=rd)
    close(gq, qo, "rotated_query")
    close(gk, ko, "rotated_key")
    r = rd or Dh
    assert np.array_equal(gq[..., r:], q[..., r:]) and np.array_equal(gk[..., r:], k[..., r:])


@pytest.mark.parametrize("H,KVH,Dh,rd", [(32, 8, 128, 0), (8, 8, 128, 64), (6, 2, 64, 0), (5, 1, 80, 32), (4, 4, 256, 0),
                                         (2, 2, 512, 0), (24, 4, 96, 0), (22, 6, 80, 0), (20, 8, 160, 0), (3, 1, 1024, 0)])
def test_rope_half_split_layout_vs_oracle(hiplib, olib, H, KVH, Dh, rd):
    """Pairs (i, i + rotary_dim / 2) instead of consecutive channels, out of place and in place. At head_dim 80, 96
    and 160 a head row's lanes straddle two wavefronts (10, 12, 20 lanes a row) once a pass holds more than a few
    rows, and at 1024 a row is two wavefronts wide: the in-place result must still equal the out-of-place one."""
    rng = np.random.default_rng(21)
    seqlens = np.array([1, 1, 37, 1, 130, 5])
    start = np.array([131071, 0, 0, 4095, 900, 65536])
    T = int(seqlens.sum())
    print(f"case rope half-split H={H} KVH={KVH} Dh={Dh} rotary_dim={rd} T={T}", flush=True)
    q = rng.standard_normal((T, H, Dh)).astype(np.float16)
    k = rng.standard_normal((T, KVH, Dh)).astype(np.float16)
    kw = dict(theta=500000.0, rotary_dim=rd, pair_layout=cabi.ROPE_PAIRS_HALF_SPLIT)
    outs = []
    for inplace in (False, True):
        (qo, ko), (gq, gk) = run_both(hiplib, olib, q, k, seqlens, start, inplace=inplace, **kw)
        close(gq, qo, f"rotated_query in-place={inplace}")
        close(gk, ko, f"rotated_key in-place={inplace}")
        r = rd or Dh
        assert np.array_equal(gq[..., r:], q[..., r:]) and np.array_equal(gk[..., r:], k[..., r:])
        outs.append((gq, gk))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1]), \
        "in-place rotation differs from out-of-place"
    (io, _), _ = run_both(hiplib, olib, q, k, seqlens, start, theta=500000.0, rotary_dim=rd)
    assert not np.array_equal(io, qo)  # not the interleaved layout's result


def test_rope_layout_is_validated(hiplib):
    q = np.zeros((1, 1, 4096), np.float16)
    a = harness.fill_rope_args(cabi.RopeArgs(), q, q, [1], [0], q, q, pair_layout=cabi.ROPE_PAIRS_HALF_SPLIT,
                               ptr=lambda t: C.c_void_p(0x1000))
    assert hiplib.pplhip_rope_forward(C.byref(a), None) == cabi.RC_UNSUPPORTED  # head_dim > 2048
    a.head_dim, a.rotary_dim = 128, 24
    assert hiplib.pplhip_rope_forward(C.byref(a), None) == cabi.RC_INVALID_VALUE  # rotary_dim % 16
    a.rotary_dim, a.pair_layout = 0, 7
    assert hiplib.pplhip_rope_forward(C.byref(a), None) == cabi.RC_INVALID_VALUE


def test_rope_options_and_in_place(hiplib, olib):
    rng = np.random.default_rng(12)
    seqlens, start = np.array([3, 1, 64]), np.array([10, 5000, 0])
    T = int(seqlens.sum())
    q = rng.standard_normal((T, 8, 128)).astype(np.float16)
    k = rng.standard_normal((T, 2, 128)).astype(np.float16)
    for kw in (dict(bypass_key=1), dict(scaling_type=cabi.ROPE_SCALING_LINEAR, scaling_factor=8.0),
               dict(scaling_type=cabi.ROPE_SCALING_DYNAMIC, scaling_factor=2.0, max_pos=2048),
               dict(scaling_type=cabi.ROPE_SCALING_DYNAMIC, scaling_factor=4.0, max_pos=32)):
        print(f"case rope options {kw}", flush=True)
        (qo, ko), (gq, gk) = run_both(hiplib, olib, q, k, seqlens, start, **kw)
        close(gq, qo, f"rotated_query {kw}")
        close(gk, ko, f"rotated_key {kw}")
        if kw.get("bypass_key"):
            assert np.array_equal(gk, k)
    # outputs aliasing the inputs (the reference transfers the input buffers when it is their last consumer)
    (qo, ko), (gq, gk) = run_both(hiplib, olib, q, k, seqlens, start, inplace=True)
    close(gq, qo, "in-place rotated_query")
    close(gk, ko, "in-place rotated_key")


def test_position_index_bit_exact(hiplib, olib):
    import torch
    rng = np.random.default_rng(13)
    for batch in (1, 3, 257, 1000):
        seqlens = np.where(rng.random(batch) < 0.7, 1, rng.integers(1, 300, batch)).astype(np.int64)
        start = rng.integers(0, 200000, batch).astype(np.int64)
        ss = np.concatenate([[0], np.cumsum(seqlens)]).astype(np.int64)
        total = int(ss[-1])
        print(f"case position_index batch={batch} total={total}", flush=True)
        want = np.full(total, -1, np.int64)
        assert olib.oracle_position_index(harness._ptr(start), harness._ptr(ss), batch, harness._ptr(want)) == 0
        dss, dsp = harness.to_dev(ss), harness.to_dev(start)
        out = torch.full((total,), -1, dtype=torch.int64, device="cuda")
        harness.pkg.check(hiplib.pplhip_position_index(dsp.data_ptr(), dss.data_ptr(), batch, total,
                                                       int(seqlens.max()), out.data_ptr(), None), "position_index")
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("H,KVH,Dh,rd,layout,paged,cache_layout", [
    (32, 8, 128, 0, cabi.ROPE_PAIRS_INTERLEAVED, False, 0),
    (32, 8, 128, 64, cabi.ROPE_PAIRS_HALF_SPLIT, True, 0),
    (6, 2, 64, 0, cabi.ROPE_PAIRS_HALF_SPLIT, False, 3),
    (4, 4, 256, 0, cabi.ROPE_PAIRS_INTERLEAVED, True, 0),
])
def test_rope_with_cache_write_equals_the_two_steps(hiplib, olib, H, KVH, Dh, rd, layout, paged, cache_layout):
    """pplhip_rope_kv_write_forward against pplhip_rope_forward followed by pplhip_kv_quantize_write over the rotated
    keys: rotated outputs, int8 bytes and fp16 scales bit for bit (byte work: no tolerance), and the slab bytes also
    against the CPU oracle's quantisation of the rotated keys the GPU produced."""
    import torch
    from ppl_nn_amd import workloads
    rng = np.random.default_rng(31)
    seqlens = np.array([1, 1, 37, 1, 130, 5])
    start = np.array([700, 0, 0, 4095, 900, 31])
    b = workloads.Batch(H, KVH, Dh, seqlens, start, 0, num_layer=2, layer_idx=1, slack_tokens=3)
    pl = harness.PagedLayout(b, page_size=64, seed=5) if paged else None
    T = int(seqlens.sum())
    print(f"case rope+write H={H} KVH={KVH} Dh={Dh} rotary_dim={rd} layout={layout} paged={paged} cache_layout={cache_layout}",
          flush=True)
    q = rng.standard_normal((T, H, Dh)).astype(np.float16)
    k = rng.standard_normal((T, KVH, Dh)).astype(np.float16)
    v = rng.standard_normal((T, KVH, Dh)).astype(np.float16)
    ss = b.seqstarts
    cs = pl.table if paged else b.cachestarts
    dq, dk, dv = harness.to_dev(q), harness.to_dev(k), harness.to_dev(v)
    tabs = (harness.to_dev(ss), harness.to_dev(start.astype(np.int64)))
    dcs = harness.to_dev(cs)
    f16 = lambda x: x.cpu().view(torch.int16).numpy()
    results = []
    for fused in (False, True):
        cache, scale = harness.new_slab(b, paged=pl, layout=cache_layout)
        dc, dsc = harness.to_dev(cache), harness.to_dev(scale)
        dqo, dko = torch.zeros_like(dq), torch.zeros_like(dk)
        ra = harness.fill_rope_args(cabi.RopeArgs(), dq, dk, seqlens, start, dqo, dko, ptr=harness.dev_ptr, tables=tabs,
                                    theta=500000.0, rotary_dim=rd, pair_layout=layout)
        w = harness.fill_write_args(cabi.KvWriteArgs(), b, dko, dv, tabs[0], tabs[1], dcs, dc, dsc, ptr=harness.dev_ptr,
                                    paged=pl, layout=cache_layout)
        if fused:
            w.d_current_key = None  # not read
            harness.pkg.check(hiplib.pplhip_rope_kv_write_forward(C.byref(ra), C.byref(w), None), "rope_kv_write")
        else:
            harness.pkg.check(hiplib.pplhip_rope_forward(C.byref(ra), None), "rope_forward")
            harness.pkg.check(hiplib.pplhip_kv_quantize_write(C.byref(w), None), "kv_quantize_write")
        torch.cuda.synchronize()
        results.append((f16(dqo), f16(dko), dc.cpu().numpy(), f16(dsc)))
    for name, x, y in zip(("rotated_query", "rotated_key", "cache", "scale"), results[0], results[1]):
        assert np.array_equal(x, y), f"{name}: the fused launch differs from the two steps"
    assert (results[1][2] != harness.CACHE_FILL).any()
    # the oracle's quantisation of those rotated keys (and of the values)
    ko = results[1][1].view(np.float16)
    cache, scale = harness.new_slab(b, paged=pl, layout=cache_layout)
    wo = harness.fill_write_args(cabi.KvWriteArgs(), b, ko, v, ss, start.astype(np.int64), np.ascontiguousarray(cs), cache,
                                 scale, paged=pl, layout=cache_layout)
    assert olib.oracle_kv_quantize_write(C.byref(wo)) == 0
    assert np.array_equal(cache, results[1][2]) and np.array_equal(scale.view(np.int16), results[1][3])


def test_rope_with_cache_write_checks_that_both_blocks_agree(hiplib):
    q = np.zeros((4, 2, 128), np.float16)
    ptr = lambda t: C.c_void_p(0x1000)
    a = harness.fill_rope_args(cabi.RopeArgs(), q, q, [4], [0], q, q, ptr=ptr)
    w = cabi.KvWriteArgs()
    w.d_current_value, w.d_seqstarts, w.d_cachestarts, w.d_start_pos = ptr(0), a.d_seqstarts, ptr(0), a.d_start_pos
    w.d_cache, w.d_scale = ptr(0), ptr(0)
    w.batch, w.total_new_tokens, w.num_layer, w.num_kv_heads, w.head_dim = 1, 4, 1, 2, 128
    for kk, x in cabi.cache_strides_layout0(1, 2, 128).items():
        setattr(w, kk, x)
    w.total_new_tokens = 5
    assert hiplib.pplhip_rope_kv_write_forward(C.byref(a), C.byref(w), None) == cabi.RC_INVALID_VALUE
    w.total_new_tokens, w.num_kv_heads = 4, 1
    assert hiplib.pplhip_rope_kv_write_forward(C.byref(a), C.byref(w), None) == cabi.RC_INVALID_VALUE
    w.num_kv_heads = 2
    w.d_start_pos = C.c_void_p(0x2000)
    assert hiplib.pplhip_rope_kv_write_forward(C.byref(a), C.byref(w), None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_rope_kv_write_forward(C.byref(a), None, None) == cabi.RC_INVALID_VALUE
