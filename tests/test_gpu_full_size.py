"""Parity at the baseline's full configuration sizes (the oracle runs on the host cores with OpenMP)."""
import numpy as np
import pytest

import harness
from harness import workloads
from test_gpu_parity import check

pytestmark = pytest.mark.gpu


def test_cfg1_llama2_7b_decode_full():
    b = workloads.cfg1_llama2_7b_decode()
    check(b, workloads.make_tensors(b, seed=0))


def test_cfg2_llama3_8b_mixed_full():
    b = workloads.cfg2_llama3_8b_mixed()
    check(b, workloads.make_tensors(b, seed=1))


def test_cfg3_long_context_reduced_and_property():
    # oracle comparison at 1/8 of the lengths (seconds on the host) ...
    b = workloads.cfg3_long_context(lo=4096, hi=16384)
    check(b, workloads.make_tensors(b, seed=3))
    # ... and at full length a size-independent property: with every cached key equal, softmax is uniform and the
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
