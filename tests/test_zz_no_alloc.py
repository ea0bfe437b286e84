"""pplhip_mhca_forward_noalloc (the entry point that allocates nothing) against pplhip_mhca_forward on the same inputs:
same kernels, same plan, scratch in the library's own device array instead of a caller-owned workspace. Two calls in a
row, the second on a smaller batch, so that whatever the first call left in the shared array must not leak into the
second's results."""
import ctypes as C

import numpy as np
import pytest

import harness
from harness import cabi, workloads

pytestmark = pytest.mark.gpu


def _run_both(hiplib, b, seed):
    import torch
    t = workloads.make_tensors(b, seed=seed)
    print(f"case no-alloc {b.name}: B={b.batch} nd={b.decoding_batches} S={b.total_new_tokens} hist={b.total_hist_tokens}",
          flush=True)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    results = []
    for noalloc in (False, True):
        cache, scale = (harness.to_dev(x) for x in harness.new_slab(b))
        d = {k: harness.to_dev(v) for k, v in t.items()}
        tabs = {k: harness.to_dev(v) for k, v in dict(ss=b.seqstarts, ks=b.kvstarts, cs=b.cachestarts, sp=b.start_pos,
                                                      hs=b.histstarts, z=np.zeros(b.batch, np.int64)).items()}
        w = harness.fill_write_args(cabi.KvWriteArgs(), b, d["hist_key"], d["hist_value"], tabs["hs"], tabs["z"],
                                    tabs["cs"], cache, scale, ptr=harness.dev_ptr)
        harness.pkg.check(hiplib.pplhip_kv_quantize_write(C.byref(w), stream), "history")
        out = torch.zeros((b.total_new_tokens, b.num_heads, b.head_dim), dtype=torch.float16, device="cuda")
        a = harness.fill_mhca_args(cabi.MhcaArgs(), b, d["query"], d["current_key"], d["current_value"], tabs["ss"],
                                   tabs["ks"], tabs["cs"], tabs["sp"], cache, scale, out, ptr=harness.dev_ptr)
        plan = cabi.MhcaPlan()
        harness.pkg.check(hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)), "prepare")
        if noalloc:
            harness.pkg.check(hiplib.pplhip_mhca_forward_noalloc(C.byref(a), C.byref(plan), stream), "forward_noalloc")
        else:
            ws = torch.empty(max(int(plan.workspace_bytes), 256), dtype=torch.uint8, device="cuda")
            harness.pkg.check(hiplib.pplhip_mhca_forward(C.byref(a), C.byref(plan), harness.dev_ptr(ws), stream), "forward")
        torch.cuda.synchronize()
        results.append((out.cpu().view(torch.int16).numpy(), cache.cpu().numpy(), scale.cpu().view(torch.int16).numpy(),
                        int(plan.workspace_bytes)))
    (o0, c0, s0, wsb), (o1, c1, s1, _) = results
    assert wsb > 0  # the call does use scratch: split-k partials of the decode sequences
    assert np.array_equal(c0, c1) and np.array_equal(s0, s1), "int8 cache bytes / fp16 scales differ"
    assert np.array_equal(o0, o1), "outputs differ between the two entry points"


def test_noalloc_matches_forward_on_two_calls_in_a_row(hiplib):
    assert hiplib.pplhip_init() == 0
    # first a mixed batch whose decode sequences span many split-k ranges, then a smaller one (fewer sequences, shorter
    # histories, fewer ranges): stale partial results of the first call lie behind and between the second call's
    big = workloads.Batch(32, 8, 128, [1] * 24 + [200, 64], list(range(3000, 3000 + 24 * 37, 37)) + [0, 0], 24,
                          name="first (larger)")
    small = workloads.Batch(32, 8, 128, [1] * 5 + [40], [900, 17, 2500, 300, 64, 0], 5, name="second (smaller)")
    _run_both(hiplib, big, seed=71)
    _run_both(hiplib, small, seed=72)


def test_noalloc_matches_forward_on_the_general_path(hiplib):
    """head_dim 64: the decode sequences' pieces (general attention path) lie in the scratch array; again two calls
    in a row, the second smaller."""
    assert hiplib.pplhip_init() == 0
    big = workloads.Batch(16, 4, 64, [1] * 12 + [90], list(range(2000, 2000 + 12 * 53, 53)) + [0], 12,
                          name="general, first (larger)")
    small = workloads.Batch(16, 4, 64, [1] * 3 + [20], [700, 130, 1500, 0], 3, name="general, second (smaller)")
    _run_both(hiplib, big, seed=73)
    _run_both(hiplib, small, seed=74)


def test_noalloc_rejects_what_needs_a_caller_workspace(hiplib):
    b = workloads.Batch(32, 8, 128, [1, 1, 512, 512], [100, 900, 4096, 0], 2)
    a = cabi.MhcaArgs()
    fake = lambda t: C.c_void_p(0x1000)
    harness.fill_mhca_args(a, b, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, ptr=fake, cache_prefill=1)
    plan = cabi.MhcaPlan()
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == 0 and plan.prefill_staging == 1
    assert hiplib.pplhip_mhca_forward_noalloc(C.byref(a), C.byref(plan), None) == cabi.RC_OUT_OF_RANGE  # > 16 MiB
    plan.workspace_bytes = 1 << 20
    assert hiplib.pplhip_mhca_forward_noalloc(C.byref(a), C.byref(plan), None) == cabi.RC_UNSUPPORTED  # staging rows
    assert b"caller-owned workspace" in hiplib.pplhip_last_error()
