"""Pins the oracle's int8 group-8 quantisation rule:
   s = max(fp16(absmax/127), fp16(1e-5)),  q = int8(rint(fp16(x/s)))
against closed forms and an independent numpy float16 restatement over every finite fp16 absmax."""
import numpy as np

EPS_BITS = 0x00A8  # fp16(1e-5)


def oquant(olib, x):
    x = np.ascontiguousarray(x, dtype=np.float16).reshape(-1, 8)
    q = np.empty(x.shape, np.int8)
    s = np.empty(x.shape[0], np.uint16)
    olib.oracle_kv_quantize_groups(x.ctypes.data, q.ctypes.data, s.ctypes.data, x.shape[0])
    return q, s.view(np.float16)


def np_quant(x):
    x = np.asarray(x, dtype=np.float16).reshape(-1, 8)
    a = np.abs(x).max(axis=1)
    s = (a.astype(np.float32) / np.float32(127.0)).astype(np.float16)
    s = np.maximum(s, np.uint16(EPS_BITS).view(np.float16))
    ratio = (x.astype(np.float32) / s.astype(np.float32)[:, None]).astype(np.float16)
    return np.rint(ratio.astype(np.float32)).astype(np.int8), s


def test_eps_constant():
    assert np.float16(1e-5).view(np.uint16) == EPS_BITS


def test_zero_group(olib):
    q, s = oquant(olib, np.zeros(8))
    assert (q == 0).all() and s.view(np.uint16)[0] == EPS_BITS
    q, s = oquant(olib, np.array([0, -0.0, 0, 0, 0, 0, 0, 0]))
    assert (q == 0).all()


def test_single_absmax_maps_to_127(olib):
    finite = np.arange(1, 0x7c00, dtype=np.uint16).view(np.float16)
    big = finite[finite.astype(np.float32) >= 127 * 1.1e-5]  # scale not clamped by eps
    x = np.zeros((big.size, 8), np.float16)
    x[:, 3] = big
    x[:, 5] = -big
    q, s = oquant(olib, x)
    assert (q[:, 3] == 127).all() and (q[:, 5] == -127).all()
    assert (np.delete(q, [3, 5], axis=1) == 0).all()


def test_all_finite_absmax_vs_numpy_restatement(olib):
    finite = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16)  # every non-negative finite half
    a32 = finite.astype(np.float32)
    rng = np.random.default_rng(11)
    cols = [finite, -finite]
    # companions that land on or next to .5 ties of x/s, plus random fractions
    for k in (0, 1, 2, 63, 100, 125, 126):
        cols.append((a32 * np.float32((k + 0.5) / 127.0)).astype(np.float16))
    x = np.stack(cols[:8], axis=1)
    x2 = np.stack([finite] + [(a32 * rng.uniform(-1, 1, a32.size).astype(np.float32)).astype(np.float16)
                              for _ in range(7)], axis=1)
    x3 = np.stack([-finite, cols[8]] + [(a32 * rng.uniform(-1, 1, a32.size).astype(np.float32)).astype(np.float16)
                                        for _ in range(6)], axis=1)
    for xs in (x, x2, x3):
        q, s = oquant(olib, xs)
        qn, sn = np_quant(xs)
        assert np.array_equal(s.view(np.uint16), sn.view(np.uint16))
        assert np.array_equal(q, qn)
        assert np.abs(q.astype(np.int32)).max() <= 127
        # sign symmetry
        qneg, sneg = oquant(olib, -xs)
        assert np.array_equal(qneg, -q) and np.array_equal(sneg.view(np.uint16), s.view(np.uint16))
        # scale is monotone in absmax (rows are ordered by absmax)
        assert (np.diff(s.astype(np.float32)) >= 0).all()
        # reconstruction error <= (1/2 + 1/32) * scale: rint error plus the fp16 rounding of the quotient below 128
        err = np.abs(q.astype(np.float64) * s.astype(np.float64)[:, None] - xs.astype(np.float64))
        assert (err <= (0.5 + 1 / 32) * s.astype(np.float64)[:, None] * (1 + 1e-12)).all()


def test_known_values(olib):
    # absmax 127 -> scale exactly 1, so q = rint(x) with ties to even
    x = np.array([127, -126.5, 0.5, 1.5, 2.5, -0.5, 63.25, -127], np.float16)
    q, s = oquant(olib, x)
    assert s[0] == np.float16(1.0)
    assert q.tolist() == [[127, -126, 0, 2, 2, 0, 63, -127]]
    # the documented double-rounding case: x/s = 126.51 -> fp16 126.5 -> 126 (a direct rint would give 127)
    x = np.array([254, 253.02, 0, 0, 0, 0, 0, 0], np.float16)  # scale exactly 2; 253.02 -> fp16 253.0 -> 126.5 -> 126
    q, s = oquant(olib, x)
    assert s[0] == np.float16(2.0) and q[0, 0] == 127 and q[0, 1] == 126


def test_dequant(olib):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((4096, 8)).astype(np.float16)
    q, s = oquant(olib, x)
    out = np.empty(x.shape, np.float32)
    olib.oracle_kv_dequant_groups(q.ctypes.data, s.ctypes.data, out.ctypes.data, x.shape[0])
    assert np.array_equal(out, q.astype(np.float32) * s.astype(np.float32)[:, None])
