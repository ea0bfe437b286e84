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
                                         (2, 2, 512, 0)])
def test_rope_half_split_layout_vs_oracle(hiplib, olib, H, KVH, Dh, rd):
    """Pairs (i, i + rotary_dim / 2) instead of consecutive channels, out of place and in place (the two halves of a
    pair are handled by two lanes of one wavefront)."""
    rng = np.random.default_rng(21)
    seqlens = np.array([1, 1, 37, 1, 130, 5])
    start = np.array([131071, 0, 0, 4095, 900, 65536])
    T = int(seqlens.sum())
    print(f"case rope half-split H={H} KVH={KVH} Dh={Dh} rotary_dim={rd} T={T}", flush=True)
    q = rng.standard_normal((T, H, Dh)).astype(np.float16)
    k = rng.standard_normal((T, KVH, Dh)).astype(np.float16)
    kw = dict(theta=500000.0, rotary_dim=rd, pair_layout=cabi.ROPE_PAIRS_HALF_SPLIT)
    for inplace in (False, True):
        (qo, ko), (gq, gk) = run_both(hiplib, olib, q, k, seqlens, start, inplace=inplace, **kw)
        close(gq, qo, f"rotated_query in-place={inplace}")
        close(gk, ko, f"rotated_key in-place={inplace}")
        r = rd or Dh
        assert np.array_equal(gq[..., r:], q[..., r:]) and np.array_equal(gk[..., r:], k[..., r:])
    (io, _), _ = run_both(hiplib, olib, q, k, seqlens, start, theta=500000.0, rotary_dim=rd)
    assert not np.array_equal(io, qo)  # not the interleaved layout's result


def test_rope_layout_is_validated(hiplib):
    q = np.zeros((1, 1, 1024), np.float16)
    a = harness.fill_rope_args(cabi.RopeArgs(), q, q, [1], [0], q, q, pair_layout=cabi.ROPE_PAIRS_HALF_SPLIT,
                               ptr=lambda t: C.c_void_p(0x1000))
    assert hiplib.pplhip_rope_forward(C.byref(a), None) == cabi.RC_UNSUPPORTED  # head_dim > 512
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
