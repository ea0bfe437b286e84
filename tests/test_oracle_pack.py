"""Pins oracle_pack_tables against a brute-force restatement of the host packing loops
(tools/benchmark_llama/generation_state.cc:93-110 for a first step, :162-170 for a decode step)."""
import ctypes as C

import numpy as np

from harness import cabi, workloads


def brute_force(kvlen, newlen, cachestart):
    order = [i for i in range(len(kvlen)) if newlen[i] == 1 and kvlen[i] > 0]
    nd = len(order)
    order += [i for i in range(len(kvlen)) if newlen[i] > 0 and not (newlen[i] == 1 and kvlen[i] > 0)]
    seqstarts, kvstarts = [0], [0]
    for i in order:
        seqstarts.append(seqstarts[-1] + int(newlen[i]))
        kvstarts.append(kvstarts[-1] + int(kvlen[i] + newlen[i]))
    return dict(order=order, nd=nd, seqstarts=seqstarts, kvstarts=kvstarts,
                cachestarts=[int(cachestart[i]) for i in order], start_pos=[int(kvlen[i]) for i in order])


def run_pack(fn, kvlen, newlen, cachestart, advance=0):
    n = len(kvlen)
    out = dict(seqstarts=np.full(n + 1, -7, np.int64), kvstarts=np.full(n + 1, -7, np.int64),
               cachestarts=np.full(n, -7, np.int64), start_pos=np.full(n, -7, np.int64),
               batch_slots=np.full(n, -7, np.int64), header=np.full(6, -7, np.int64))
    a = cabi.PackArgs()
    a.d_slot_kvlen, a.d_slot_newlen, a.d_slot_cachestart = kvlen.ctypes.data, newlen.ctypes.data, cachestart.ctypes.data
    a.num_slots, a.advance_slots = n, advance
    a.d_seqstarts, a.d_kvstarts = out["seqstarts"].ctypes.data, out["kvstarts"].ctypes.data
    a.d_cachestarts, a.d_start_pos = out["cachestarts"].ctypes.data, out["start_pos"].ctypes.data
    a.d_batch_slots, a.d_header = out["batch_slots"].ctypes.data, out["header"].ctypes.data
    assert fn(C.byref(a)) == 0
    return out


def check_against_brute_force(out, kvlen, newlen, cachestart):
    bf = brute_force(kvlen, newlen, cachestart)
    B = len(bf["order"])
    assert out["header"].tolist() == [
        B, bf["nd"], max([int(newlen[i]) for i in bf["order"]], default=0),
        max([int(kvlen[i] + newlen[i]) for i in bf["order"]], default=0), bf["seqstarts"][-1], bf["kvstarts"][-1]]
    assert out["seqstarts"][:B + 1].tolist() == bf["seqstarts"]
    assert out["kvstarts"][:B + 1].tolist() == bf["kvstarts"]
    assert (out["seqstarts"][B + 1:] == bf["seqstarts"][-1]).all()
    assert (out["kvstarts"][B + 1:] == bf["kvstarts"][-1]).all()
    assert out["cachestarts"][:B].tolist() == bf["cachestarts"]
    assert out["start_pos"][:B].tolist() == bf["start_pos"]
    assert out["batch_slots"][:B].tolist() == bf["order"]
    assert (out["batch_slots"][B:] == -1).all()


def test_pack_first_step_matches_reference_first_step(olib):
    # all prefill: prefix sums of prompt lengths, start_pos 0, decoding_batches 0 (generation_state.cc:71-110)
    prompts = np.array([5, 17, 1, 300], np.int64)
    out = run_pack(olib.oracle_pack_tables, np.zeros(4, np.int64), prompts, np.array([0, 100, 200, 300], np.int64))
    assert out["header"].tolist() == [4, 0, 300, 300, 323, 323]
    assert out["seqstarts"].tolist() == [0, 5, 22, 23, 323]
    assert out["start_pos"].tolist() == [0, 0, 0, 0]


def test_pack_random_churn(olib):
    rng = np.random.default_rng(2)
    for n in (1, 2, 7, 64, 256, 1000):
        for _ in range(5):
            kvlen = rng.integers(0, 50, n).astype(np.int64) * (rng.random(n) < 0.7)
            newlen = np.where(rng.random(n) < 0.2, 0, np.where(kvlen > 0, 1, rng.integers(1, 40, n))).astype(np.int64)
            newlen = np.where(rng.random(n) < 0.05, rng.integers(2, 9, n), newlen)  # chunked prefill on live slots
            cs = (np.arange(n) * 1024).astype(np.int64)
            out = run_pack(olib.oracle_pack_tables, kvlen.astype(np.int64), newlen.astype(np.int64), cs)
            check_against_brute_force(out, kvlen, newlen, cs)


def test_churn_schedule_invariants():
    sch = workloads.ChurnSchedule(seed=2, num_slots=64, region=256, lo=8, hi=64)
    prev_after = np.zeros(64, np.int64)
    for _ in range(200):
        kv, nl = sch.next_step()
        assert ((kv == 0) | (kv == prev_after)).all()  # a slot either continues or was reset
        assert (nl[kv > 0] == 1).all() and (nl[kv == 0] >= 8).all()
        assert (kv + nl <= 256).all()
        prev_after = kv + nl


def test_pack_with_advance_moves_the_slot_state(olib):
    """advance_slots = 1: the same tables, and afterwards slot_kvlen += slot_newlen for every active slot
    (generation_state.cc:127-140 grows the kv lengths between steps)."""
    rng = np.random.default_rng(8)
    for n in (1, 5, 64, 300):
        kvlen = (rng.integers(0, 50, n) * (rng.random(n) < 0.7)).astype(np.int64)
        newlen = np.where(rng.random(n) < 0.2, 0, np.where(kvlen > 0, 1, rng.integers(1, 40, n))).astype(np.int64)
        cs = (np.arange(n) * 1024).astype(np.int64)
        plain = run_pack(olib.oracle_pack_tables, kvlen.copy(), newlen, cs)
        state = kvlen.copy()
        moved = run_pack(olib.oracle_pack_tables, state, newlen, cs, advance=1)
        for k in plain:
            assert np.array_equal(plain[k], moved[k]), k
        assert np.array_equal(state, kvlen + np.maximum(newlen, 0))
