"""CPU checks that pin the oracle's RotaryPositionEmbedding / PositionIndex restatement by what the mathematics
fixes: a numpy complex-multiply restatement, rotation invariants, composition and relative-position properties."""
import ctypes as C

import numpy as np
import pytest

import harness
from harness import cabi


def rope_oracle(olib, q, k, seqlens, start_pos, theta=10000.0, rotary_dim=0, bypass_key=0, scaling_type=0,
                scaling_factor=1.0, max_pos=2048, pair_layout=0):
    q, k = np.ascontiguousarray(q), np.ascontiguousarray(k)
    qo, ko = np.zeros_like(q), np.zeros_like(k)
    a = harness.fill_rope_args(cabi.RopeArgs(), q, k, seqlens, start_pos, qo, ko, theta=theta, rotary_dim=rotary_dim,
                               bypass_key=bypass_key, scaling_type=scaling_type, scaling_factor=scaling_factor,
                               max_pos=max_pos, pair_layout=pair_layout)
    assert olib.oracle_rope_forward(C.byref(a)) == 0
    return qo, ko


def close_f16(got, want64, ulps=0.6):
    """got (fp16) is the correctly rounded want64 up to `ulps` units in the last place (the oracle narrows through
    float32, and libm's pow/cos/sin differ from numpy's in the last float64 bits)."""
    ulp = np.spacing(np.abs(want64).astype(np.float16)).astype(np.float64)
    return bool((np.abs(got.astype(np.float64) - want64) <= ulps * ulp + 1e-7).all())


def numpy_rope(x, pos, theta, rotary_dim):
    """x [T, H, D] float64, pos [T]: complex multiply on consecutive channel pairs of the first rotary_dim channels."""
    x = x.astype(np.float64)
    out = x.copy()
    rd = rotary_dim
    inv = theta ** (-np.arange(0, rd, 2, dtype=np.float64) / rd)
    ang = pos[:, None].astype(np.float64) * inv[None, :]
    z = (x[..., 0:rd:2] + 1j * x[..., 1:rd:2]) * np.exp(1j * ang)[:, None, :]
    out[..., 0:rd:2], out[..., 1:rd:2] = z.real, z.imag
    return out


@pytest.mark.parametrize("rotary_dim,Dh", [(0, 128), (64, 128), (0, 64), (32, 80)])
def test_vs_complex_multiply(olib, rotary_dim, Dh):
    rng = np.random.default_rng(5)
    seqlens, start = np.array([1, 5, 1, 17]), np.array([100000, 0, 3, 250])
    T = int(seqlens.sum())
    q = rng.standard_normal((T, 6, Dh)).astype(np.float16)
    k = rng.standard_normal((T, 2, Dh)).astype(np.float16)
    qo, ko = rope_oracle(olib, q, k, seqlens, start, theta=500000.0, rotary_dim=rotary_dim)
    pos = np.concatenate([s + np.arange(n) for n, s in zip(seqlens, start)])
    rd = rotary_dim or Dh
    for got, x in ((qo, q), (ko, k)):
        want = numpy_rope(x, pos, 500000.0, rd)
        assert close_f16(got, want)  # float64 on both sides, one rounding
        assert np.array_equal(got[..., rd:], x[..., rd:])  # pass-through channels untouched


def numpy_rope_half_split(x, pos, theta, rotary_dim):
    """The "rotate_half" restatement: y = x * cos + rotate_half(x) * sin over the first rotary_dim channels, with
    rotate_half(x) = concat(-x[rd/2:], x[:rd/2]) and the angle table repeated for both halves."""
    x = x.astype(np.float64)
    out = x.copy()
    rd = rotary_dim
    inv = theta ** (-np.arange(0, rd, 2, dtype=np.float64) / rd)
    ang = pos[:, None].astype(np.float64) * inv[None, :]
    emb = np.concatenate([ang, ang], axis=-1)[:, None, :]
    xr = x[..., :rd]
    rot = np.concatenate([-xr[..., rd // 2:], xr[..., :rd // 2]], axis=-1)
    out[..., :rd] = xr * np.cos(emb) + rot * np.sin(emb)
    return out


@pytest.mark.parametrize("rotary_dim,Dh", [(0, 128), (64, 128), (0, 64), (32, 80)])
def test_half_split_layout_vs_rotate_half(olib, rotary_dim, Dh):
    rng = np.random.default_rng(15)
    seqlens, start = np.array([1, 5, 1, 17]), np.array([100000, 0, 3, 250])
    T = int(seqlens.sum())
    q = rng.standard_normal((T, 6, Dh)).astype(np.float16)
    k = rng.standard_normal((T, 2, Dh)).astype(np.float16)
    qo, ko = rope_oracle(olib, q, k, seqlens, start, theta=500000.0, rotary_dim=rotary_dim,
                         pair_layout=cabi.ROPE_PAIRS_HALF_SPLIT)
    pos = np.concatenate([s + np.arange(n) for n, s in zip(seqlens, start)])
    rd = rotary_dim or Dh
    for got, x in ((qo, q), (ko, k)):
        assert close_f16(got, numpy_rope_half_split(x, pos, 500000.0, rd))
        assert np.array_equal(got[..., rd:], x[..., rd:])
    # the two layouts are the same rotation up to a fixed permutation of the rotated channels:
    # half-split(x) = P^-1 interleaved(P x), P gathering channels (0, rd/2, 1, rd/2+1, ...)
    perm = np.arange(rd).reshape(2, rd // 2).T.reshape(-1)
    qp = q.copy()
    qp[..., :rd] = q[..., perm]
    inter, _ = rope_oracle(olib, qp, k, seqlens, start, theta=500000.0, rotary_dim=rotary_dim)
    back = inter.copy()
    back[..., perm] = inter[..., :rd]
    assert np.array_equal(back, qo)
    # and they differ as functions of an unpermuted input, so a wrong choice cannot pass unnoticed
    plain, _ = rope_oracle(olib, q, k, seqlens, start, theta=500000.0, rotary_dim=rotary_dim)
    assert not np.array_equal(plain, qo)
    # an unknown layout value is refused
    a = harness.fill_rope_args(cabi.RopeArgs(), q, k, seqlens, start, np.zeros_like(q), np.zeros_like(k), pair_layout=2)
    assert olib.oracle_rope_forward(C.byref(a)) == cabi.RC_INVALID_VALUE


def test_invariants(olib):
    rng = np.random.default_rng(6)
    q = rng.standard_normal((8, 4, 128)).astype(np.float16)
    k = rng.standard_normal((8, 4, 128)).astype(np.float16)
    # position 0 is the identity
    qo, ko = rope_oracle(olib, q, k, [1] * 8, [0] * 8)
    assert np.array_equal(qo, q) and np.array_equal(ko, k)
    # bypass_key leaves the key alone at any position
    qo, ko = rope_oracle(olib, q, k, [8], [77], bypass_key=1)
    assert np.array_equal(ko, k) and not np.array_equal(qo, q)
    # pair norms are preserved (up to the fp16 rounding of the outputs)
    qo, _ = rope_oracle(olib, q, k, [8], [1234])
    n_in = np.hypot(q[..., 0::2].astype(np.float64), q[..., 1::2].astype(np.float64))
    n_out = np.hypot(qo[..., 0::2].astype(np.float64), qo[..., 1::2].astype(np.float64))
    assert np.abs(n_in - n_out).max() < 4e-3
    # q.k depends on the position difference only
    q1, k1 = rope_oracle(olib, q, k, [8], [10])
    q2, k2 = rope_oracle(olib, q, k, [8], [5010])
    d1 = np.einsum("thd,shd->hts", q1.astype(np.float64), k1.astype(np.float64))
    d2 = np.einsum("thd,shd->hts", q2.astype(np.float64), k2.astype(np.float64))
    assert np.abs(d1 - d2).max() < 0.15  # |q.k| ~ 11 with fp16-rounded operands
    # composition: rotating by p1 then by p2 == rotating by p1 + p2 (one extra fp16 rounding in between)
    a1, _ = rope_oracle(olib, q, k, [1] * 8, [300] * 8)
    a2, _ = rope_oracle(olib, a1, k, [1] * 8, [45] * 8)
    a3, _ = rope_oracle(olib, q, k, [1] * 8, [345] * 8)
    assert np.abs(a2.astype(np.float64) - a3.astype(np.float64)).max() < 6e-3


def test_scaling(olib):
    rng = np.random.default_rng(7)
    q = rng.standard_normal((6, 2, 64)).astype(np.float16)
    k = rng.standard_normal((6, 2, 64)).astype(np.float16)
    # linear: position / factor -> same as an unscaled call at the divided positions
    lin, _ = rope_oracle(olib, q, k, [6], [40], scaling_type=cabi.ROPE_SCALING_LINEAR, scaling_factor=4.0)
    pos = (40 + np.arange(6)) / 4.0
    assert close_f16(lin, numpy_rope(q, pos, 10000.0, 64))
    # dynamic: unchanged below max_position_embeddings, NTK-scaled base above it
    dyn, _ = rope_oracle(olib, q, k, [6], [40], scaling_type=cabi.ROPE_SCALING_DYNAMIC, scaling_factor=2.0, max_pos=64)
    none, _ = rope_oracle(olib, q, k, [6], [40])
    assert np.array_equal(dyn, none)
    dyn, _ = rope_oracle(olib, q, k, [6], [100], scaling_type=cabi.ROPE_SCALING_DYNAMIC, scaling_factor=2.0, max_pos=64)
    base = 10000.0 * (2.0 * 106 / 64 - 1.0) ** (64 / 62)
    assert close_f16(dyn, numpy_rope(q, 100 + np.arange(6.0), base, 64))


def test_position_index(olib):
    seqlens, start = np.array([1, 4, 1, 9, 2], np.int64), np.array([7, 0, 100000, 3, 0], np.int64)
    ss = np.concatenate([[0], np.cumsum(seqlens)]).astype(np.int64)
    out = np.full(int(ss[-1]), -1, np.int64)
    assert olib.oracle_position_index(harness._ptr(start), harness._ptr(ss), len(seqlens), harness._ptr(out)) == 0
    want = np.concatenate([s + np.arange(n) for n, s in zip(seqlens, start)])
    assert np.array_equal(out, want)
