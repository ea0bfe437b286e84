"""The decode kernel keeps its own count of the memory operations in flight (s_waitcnt with hand-derived immediates, so
that a stage's arithmetic runs under the next stage's transfers and a sequence's result stores under the next
sequence's first transfers). The checking build replaces every such wait by a wait for everything in flight. If a count
were too generous the product build would read a stage buffer, a query or a new token before it has landed; the two
builds must therefore agree bit for bit -- outputs, int8 rows and scales -- on batches that take every hand-over: many
short sequences per range (result stores of 4 and of 8 instructions pending), sequences cut by range boundaries, the
token-split workgroups of a single kv head, a paged slab, and decode + prompts in one launch."""
import numpy as np
import pytest

import harness
from harness import workloads

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(11)
    many_short = [int(x) for x in rng.integers(1, 90, 300)]
    ragged = [int(x) for x in rng.integers(1, 3000, 96)]
    yield "many_short_kvh8", workloads.Batch(32, 8, 128, [1] * 300, many_short, 300, name="cw_short"), {}
    yield "ragged_kvh32", workloads.Batch(32, 32, 128, [1] * 96, ragged, 96, name="cw_ragged"), {}
    yield "ragged_kvh8_finest_split", workloads.Batch(32, 8, 128, [1] * 96, ragged, 96, name="cw_split"), dict(split_k=2)
    yield "one_kv_head_token_split", workloads.Batch(8, 1, 128, [1] * 5, [20000, 3, 7000, 64, 33], 5, name="cw_kvh1"), {}
    yield "mixed_launch", workloads.Batch(32, 8, 128, [1] * 40 + [200, 77], ragged[:40] + [0, 0], 40, name="cw_mixed"), {}


@pytest.mark.parametrize("name,b,kw", list(_cases()), ids=[c[0] for c in _cases()])
def test_counted_waits_match_full_waits(name, b, kw):
    check_lib = harness.pkg.load_conservative_waits_library()
    t = workloads.make_tensors(b, seed=17)
    print(f"case {name}: product build", flush=True)
    got = harness.run_device(b, t, **kw)
    print(f"case {name}: checking build (every counted wait replaced by a full wait)", flush=True)
    want = harness.run_device(b, t, lib=check_lib, **kw)
    assert np.array_equal(got["output"].view(np.uint16), want["output"].view(np.uint16))
    assert np.array_equal(got["cache"], want["cache"])
    assert np.array_equal(got["scale"].view(np.uint16), want["scale"].view(np.uint16))


def test_counted_waits_match_full_waits_paged():
    check_lib = harness.pkg.load_conservative_waits_library()
    rng = np.random.default_rng(12)
    b = workloads.Batch(32, 8, 128, [1] * 64, [int(x) for x in rng.integers(1, 1500, 64)], 64, name="cw_paged")
    t = workloads.make_tensors(b, seed=18)
    got = harness.run_device(b, t, paged=harness.PagedLayout(b, page_size=128, seed=3))
    want = harness.run_device(b, t, paged=harness.PagedLayout(b, page_size=128, seed=3), lib=check_lib)
    assert np.array_equal(got["output"].view(np.uint16), want["output"].view(np.uint16))
    assert np.array_equal(got["cache"], want["cache"])
    assert np.array_equal(got["scale"].view(np.uint16), want["scale"].view(np.uint16))
