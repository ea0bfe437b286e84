"""pplhip_check_tables_host / pplhip_check_tables: the consistency rules of one call's ragged-batch tables. The host
form is exercised on the CPU for every code it can return; the device form (`-m gpu`) must report the same finding
for the same tables -- it only ever reads the tables, so corrupt ones are safe to hand to it."""
import ctypes as C

import numpy as np
import pytest

import harness
from harness import cabi, workloads


def good_batch(paged=False):
    b = workloads.Batch(8, 2, 128, [1, 1, 1, 70, 5], [300, 1, 63, 0, 64], 3, slack_tokens=2, name="tables")
    pl = harness.PagedLayout(b, page_size=64, seed=3) if paged else None
    return b, pl


def tables_of(b, pl):
    t = dict(seqstarts=b.seqstarts.copy(), kvstarts=b.kvstarts.copy(), start_pos=b.start_pos.copy(),
             cachestarts=np.ascontiguousarray(pl.table).copy() if pl else b.cachestarts.copy())
    t["max_slab_tokens"] = pl.slab_tokens if pl else b.max_tokens
    return t


def args_for(b, pl, t, ptr):
    a = cabi.MhcaArgs()
    a.d_seqstarts, a.d_kvstarts = ptr(t["seqstarts"]), ptr(t["kvstarts"])
    a.d_cachestarts, a.d_start_pos = ptr(t["cachestarts"]), ptr(t["start_pos"])
    a.batch, a.decoding_batches = b.batch, b.decoding_batches
    a.max_seqlen, a.max_kvlen, a.total_new_tokens = b.max_seqlen, b.max_kvlen, b.total_new_tokens
    a.cache_mode, a.page_size = (1, pl.page_size) if pl else (0, 128)
    a.cachestart_stride_b = pl.max_pages if pl else 0
    a._refs = [t]
    return a


def host_check(lib, b, pl, t, **over):
    a = args_for(b, pl, t, harness._ptr)
    for k, v in over.items():
        setattr(a, k, v)
    flag = np.full(2, 99, np.int32)
    assert lib.pplhip_check_tables_host(C.byref(a), t["max_slab_tokens"], harness._ptr(flag)) == cabi.RC_SUCCESS
    return int(flag[0]), int(flag[1])


# (name, paged, mutation of the table dict, argument overrides, expected (code, sequence))
def _cases():
    def mut(f):
        return f
    cases = [
        ("consistent", False, lambda t: None, {}, (cabi.TABLES_OK, -1)),
        ("consistent, paged", True, lambda t: None, {}, (cabi.TABLES_OK, -1)),
        ("seqstarts does not start at 0", False, lambda t: t["seqstarts"].__iadd__(1), {"total_new_tokens": 79},
         (cabi.TABLES_BAD_SEQSTARTS, 0)),
        ("seqstarts not increasing", False, lambda t: t["seqstarts"].__setitem__(4, 3), {}, (cabi.TABLES_BAD_SEQSTARTS, 3)),
        ("total_new_tokens differs from seqstarts[batch]", False, lambda t: None, {"total_new_tokens": 77},
         (cabi.TABLES_BAD_SEQSTARTS, 4)),
        ("kvstarts does not start at 0", False, lambda t: t["kvstarts"].__setitem__(0, 1), {}, (cabi.TABLES_BAD_KVSTARTS, 0)),
        ("kv length below the new tokens", False, lambda t: t["kvstarts"].__setitem__(4, t["kvstarts"][3] + 10), {},
         (cabi.TABLES_BAD_KVSTARTS, 3)),
        ("kvlen != start_pos + seqlen", False, lambda t: t["start_pos"].__setitem__(1, 2), {}, (cabi.TABLES_KVLEN_MISMATCH, 1)),
        ("negative start_pos", False, lambda t: t["start_pos"].__setitem__(3, -1), {}, (cabi.TABLES_KVLEN_MISMATCH, 3)),
        ("a decode sequence with two new tokens", False, None, {}, (cabi.TABLES_BAD_DECODE_ORDER, 1)),
        ("more decode sequences than one-token sequences", False, lambda t: None, {"decoding_batches": 4},
         (cabi.TABLES_BAD_DECODE_ORDER, 3)),
        ("max_seqlen too small", False, lambda t: None, {"max_seqlen": 69}, (cabi.TABLES_MAX_EXCEEDED, 3)),
        ("max_kvlen too small", False, lambda t: None, {"max_kvlen": 300}, (cabi.TABLES_MAX_EXCEEDED, 0)),
        ("region runs past the slab", False, lambda t: t["cachestarts"].__setitem__(2, t["max_slab_tokens"] - 63), {},
         (cabi.TABLES_SLAB_RANGE, 2)),
        ("negative cachestart", False, lambda t: t["cachestarts"].__setitem__(4, -1), {}, (cabi.TABLES_SLAB_RANGE, 4)),
        ("a used page outside the slab", True, lambda t: t["cachestarts"].__setitem__((0, 4), t["max_slab_tokens"] - 44), {},
         (cabi.TABLES_SLAB_RANGE, 0)),
        ("an unused page entry is not looked at", True, lambda t: t["cachestarts"].__setitem__((1, 1), -77), {},
         (cabi.TABLES_OK, -1)),
        ("page table row too short", True, lambda t: None, {"cachestart_stride_b": 4}, (cabi.TABLES_PAGE_TABLE_TOO_SHORT, 0)),
        ("two findings: the lowest sequence is reported", False,
         lambda t: (t["start_pos"].__setitem__(4, 0), t["cachestarts"].__setitem__(1, -5)), {}, (cabi.TABLES_SLAB_RANGE, 1)),
    ]
    return cases


def _apply(name, b, pl, t, mutate):
    if name == "a decode sequence with two new tokens":
        # sequence 1 gets two new tokens: every later packed index shifts by one (totals kept consistent otherwise)
        t["seqstarts"][2:] += 1
        t["kvstarts"][2:] += 1
        return {"total_new_tokens": int(t["seqstarts"][-1]), "max_kvlen": b.max_kvlen + 1}
    if name == "page table row too short":
        # the 301-token sequence needs 5 pages of 64; the caller claims rows of 4 entries (the table itself keeps its
        # real row length: entries are only read when the row is long enough)
        t["cachestarts"] = np.ascontiguousarray(t["cachestarts"][:, :4]).copy()
        return {}
    mutate(t)
    return {}


@pytest.mark.parametrize("name,paged,mutate,over,want", _cases(), ids=[c[0] for c in _cases()])
def test_host_check_reports_every_code(hiplib, name, paged, mutate, over, want):
    b, pl = good_batch(paged)
    t = tables_of(b, pl)
    extra = _apply(name, b, pl, t, mutate)
    got = host_check(hiplib, b, pl, t, **{**extra, **over})
    assert got == want, f"{name}: got {got}, want {want}"


def test_check_tables_validates_its_arguments(hiplib):
    b, pl = good_batch()
    t = tables_of(b, pl)
    a = args_for(b, pl, t, harness._ptr)
    flag = np.zeros(2, np.int32)
    assert hiplib.pplhip_check_tables_host(C.byref(a), -1, harness._ptr(flag)) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_check_tables_host(C.byref(a), 10, None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_check_tables_host(None, 10, harness._ptr(flag)) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_check_tables(C.byref(a), 10, None, None) == cabi.RC_INVALID_VALUE  # no launch
    a.cache_mode, a.page_size, a.cachestart_stride_b = 1, 48, 4
    assert hiplib.pplhip_check_tables_host(C.byref(a), 10, harness._ptr(flag)) == cabi.RC_UNSUPPORTED
    a.cache_mode, a.d_start_pos = 0, None
    assert hiplib.pplhip_check_tables_host(C.byref(a), 10, harness._ptr(flag)) == cabi.RC_INVALID_VALUE
    # an empty batch is consistent
    a = args_for(b, pl, t, harness._ptr)
    a.batch = a.decoding_batches = 0
    assert hiplib.pplhip_check_tables_host(C.byref(a), 10, harness._ptr(flag)) == cabi.RC_SUCCESS
    assert tuple(flag) == (cabi.TABLES_OK, -1)


@pytest.mark.gpu
@pytest.mark.parametrize("name,paged,mutate,over,want", _cases(), ids=[c[0] for c in _cases()])
def test_device_check_agrees_with_the_host_check(hiplib, name, paged, mutate, over, want):
    """The device kernel on the same tables (it reads nothing but the tables, so the corrupt ones cannot make it
    touch memory outside them), and on good tables before a real attention call's tables are trusted."""
    import torch
    b, pl = good_batch(paged)
    t = tables_of(b, pl)
    extra = _apply(name, b, pl, t, mutate)
    print(f"case check_tables {name}", flush=True)
    dt = {k: harness.to_dev(v) for k, v in t.items() if k != "max_slab_tokens"}
    dt["max_slab_tokens"] = t["max_slab_tokens"]
    a = args_for(b, pl, dt, harness.dev_ptr)
    for k, v in {**extra, **over}.items():
        setattr(a, k, v)
    flag = torch.full((2,), 99, dtype=torch.int32, device="cuda")
    harness.pkg.check(hiplib.pplhip_check_tables(C.byref(a), t["max_slab_tokens"], harness.dev_ptr(flag), None),
                      "check_tables")
    torch.cuda.synchronize()
    assert tuple(int(x) for x in flag.cpu()) == want


@pytest.mark.gpu
def test_device_check_on_a_large_device_built_batch(hiplib):
    """More sequences than the workgroup has lanes, tables built by pplhip_pack_tables on the device."""
    import torch
    rng = np.random.default_rng(5)
    n = 1000
    kv = rng.integers(0, 900, n).astype(np.int64)
    nl = np.where(kv > 0, 1, rng.integers(1, 120, n)).astype(np.int64)
    nl[rng.random(n) < 0.1] = 0
    cs = (np.arange(n, dtype=np.int64) * 1024)
    d = {k: harness.to_dev(v) for k, v in dict(kv=kv, nl=nl, cs=cs).items()}
    out = {k: torch.zeros(n + 1 if k in ("seqstarts", "kvstarts") else n, dtype=torch.int64, device="cuda")
           for k in ("seqstarts", "kvstarts", "cachestarts", "start_pos", "slots")}
    header = torch.zeros(6, dtype=torch.int64, device="cuda")
    pa = cabi.PackArgs()
    pa.d_slot_kvlen, pa.d_slot_newlen, pa.d_slot_cachestart = (harness.dev_ptr(d[k]) for k in ("kv", "nl", "cs"))
    pa.num_slots = n
    pa.d_seqstarts, pa.d_kvstarts, pa.d_cachestarts = (harness.dev_ptr(out[k]) for k in ("seqstarts", "kvstarts", "cachestarts"))
    pa.d_start_pos, pa.d_batch_slots, pa.d_header = harness.dev_ptr(out["start_pos"]), harness.dev_ptr(out["slots"]), harness.dev_ptr(header)
    harness.pkg.check(hiplib.pplhip_pack_tables(C.byref(pa), None), "pack_tables")
    torch.cuda.synchronize()
    batch, nd, max_seqlen, max_kvlen, total_new, _ = (int(x) for x in header.cpu())
    a = cabi.MhcaArgs()
    a.d_seqstarts, a.d_kvstarts = harness.dev_ptr(out["seqstarts"]), harness.dev_ptr(out["kvstarts"])
    a.d_cachestarts, a.d_start_pos = harness.dev_ptr(out["cachestarts"]), harness.dev_ptr(out["start_pos"])
    a.batch, a.decoding_batches, a.max_seqlen, a.max_kvlen, a.total_new_tokens = batch, nd, max_seqlen, max_kvlen, total_new
    a.cache_mode, a.page_size = 0, 128
    flag = torch.full((2,), 99, dtype=torch.int32, device="cuda")
    harness.pkg.check(hiplib.pplhip_check_tables(C.byref(a), n * 1024, harness.dev_ptr(flag), None), "check_tables")
    torch.cuda.synchronize()
    assert tuple(int(x) for x in flag.cpu()) == (cabi.TABLES_OK, -1)
    # the slab one token too small for the last region that is filled to its end ... (none is): shrink to cut a region
    last_used = int((cs + kv + nl)[nl > 0].max())
    harness.pkg.check(hiplib.pplhip_check_tables(C.byref(a), last_used - 1, harness.dev_ptr(flag), None), "check_tables")
    torch.cuda.synchronize()
    assert int(flag.cpu()[0]) == cabi.TABLES_SLAB_RANGE
