"""Slab offsets beyond 2^32 bytes. Every kernel folds the plane / head / layer / token offsets of the slab in 64 bits;
a fold that narrowed would be an out-of-range store, so these tests put the sequences at the far end of slabs whose
byte offsets exceed 2^32 and compare with the oracle:
  * cache_layout 3 (L, 2, KVH, MaxT, Dh) with KVH * MaxT * Dh > 2^32: the K -> V plane distance and the upper heads'
    offsets do not fit 32 bits;
  * cache_layout 0 (MaxT, L, 2, KVH, Dh) with num_layer 32, layer_idx 31 and slab tokens beyond 65 536: the token
    offset does not fit 32 bits (65 536 bytes a token).
The oracle runs on a small slab that holds the same sequences (the bytes of a token's rows do not depend on where the
slab keeps them); the device slab is only ever touched on the device: the sequences' rows are gathered there and
compared bit for bit, and every byte outside them must still hold the fill pattern."""
import numpy as np
import pytest

import harness
from harness import cabi, workloads

pytestmark = pytest.mark.gpu


def _device_slab(layout, tokens, L, KVH, Dh):
    import torch
    shape = (tokens, L, 2, KVH, Dh) if layout == 0 else (L, 2, KVH, tokens, Dh)
    cache = torch.full(shape, harness.CACHE_FILL, dtype=torch.int8, device="cuda")
    scale = torch.full(shape[:-1] + (Dh // 8,), 1.0, dtype=torch.float16, device="cuda")  # 0x3c00 = SCALE_FILL
    return cache, scale


def _rows(slab, layout, layer, first, n):
    """[n, 2, KVH, x] rows of slab tokens first .. first + n of one layer"""
    if layout == 0:
        return slab[first:first + n, layer]
    return slab[layer, :, :, first:first + n].permute(2, 0, 1, 3)


def _check(layout, L, layer, tokens_big, H, KVH, Dh, seqlens, start_pos, nd, cache_prefill, staging=None):
    import torch
    small = workloads.Batch(H, KVH, Dh, seqlens, start_pos, nd, num_layer=L, layer_idx=layer, name="large_slab_ref")
    t = workloads.make_tensors(small, seed=2024 + layout + Dh)
    ref = harness.run_oracle(small, t, cache_prefill=cache_prefill)  # layout 0 slab of small.max_tokens tokens
    shift = tokens_big - small.max_tokens  # the same regions, at the far end of the large slab
    big = workloads.Batch(H, KVH, Dh, seqlens, start_pos, nd, num_layer=L, layer_idx=layer, name="large_slab",
                          cachestarts=small.cachestarts + shift)
    assert big.max_tokens == tokens_big
    cache, scale = _device_slab(layout, tokens_big, L, KVH, Dh)
    st = (cabi.cache_strides_layout3(L, KVH, Dh, tokens_big) if layout == 3 else cabi.cache_strides_layout0(L, KVH, Dh))
    far = int(big.cachestarts.max()) * st["cache_stride_s"] + layer * st["cache_stride_l"] + st["cache_stride_kv"] + \
        (KVH - 1) * st["cache_stride_h"]
    assert far > 2 ** 32, "the test must reach past 2^32"
    print(f"case large slab layout={layout} L={L} layer={layer} tokens={tokens_big} Dh={Dh} cache_prefill={cache_prefill} "
          f"staging={staging} farthest row offset {far}", flush=True)
    plans = []
    got = harness.run_device(big, t, cache_prefill=cache_prefill, layout=layout, slab=(cache, scale), plan_out=plans,
                             staging=staging)
    harness.assert_attn_close(got["output"], ref["output_f64"])
    ref_cache = torch.from_numpy(ref["cache"]).cuda()
    ref_scale = torch.from_numpy(ref["scale"].view(np.int16)).cuda()
    touched = 0
    for i in range(big.batch):
        kv = int(big.kvlens[i])
        gc = _rows(cache, layout, layer, int(big.cachestarts[i]), kv)
        gs = _rows(scale.view(torch.int16), layout, layer, int(big.cachestarts[i]), kv)
        assert torch.equal(gc, ref_cache[int(small.cachestarts[i]):int(small.cachestarts[i]) + kv, layer]), \
            f"int8 rows of sequence {i} differ"
        assert torch.equal(gs, ref_scale[int(small.cachestarts[i]):int(small.cachestarts[i]) + kv, layer]), \
            f"fp16 scales of sequence {i} differ"
        touched += int((gc != harness.CACHE_FILL).sum())
    # nothing else was written: the bytes that differ from the fill pattern are all inside the sequences' rows
    assert int((cache != harness.CACHE_FILL).sum()) == touched, "bytes outside the sequences' rows were written"
    assert int((scale.view(torch.int16) != harness.SCALE_FILL).sum()) <= sum(int(k) for k in big.kvlens) * 2 * KVH * (Dh // 8)
    del cache, scale
    torch.cuda.empty_cache()
    return plans[0]


SEQLENS = [1, 1, 1, 1, 1, 200, 70, 129]
START = [700, 31, 2100, 64, 1, 0, 0, 0]


@pytest.mark.parametrize("Dh,KVH,H", [(128, 8, 32), (64, 8, 16)])
def test_layout3_planes_beyond_4gib(Dh, KVH, H):
    """(L, 2, KVH, MaxT, Dh) with KVH * MaxT * Dh > 2^32: tuned kernels (head_dim 128) and general kernels (64)."""
    tokens = (2 ** 32) // (KVH * Dh) + 4099
    plan = _check(3, 1, 0, tokens, H, KVH, Dh, SEQLENS, START, 5, cache_prefill=0)
    assert plan.general_kernel == (0 if Dh == 128 else 1)


@pytest.mark.parametrize("Dh", [128, 64])
def test_layout0_layer_31_of_32_beyond_65536_tokens(Dh):
    """(MaxT, 32, 2, 8, Dh): 65 536 bytes a token at head_dim 128, so tokens beyond 65 536 lie beyond 2^32 bytes."""
    tokens = (2 ** 32) // (32 * 2 * 8 * Dh) + 3001
    _check(0, 32, 31, tokens, 32, 8, Dh, SEQLENS, START, 5, cache_prefill=0)


@pytest.mark.parametrize("layout,staging", [(0, None), (0, 0), (3, None), (3, 0)])
def test_cache_prefill_reads_the_far_end_of_the_slab(layout, staging):
    """Prompts that attend over the slab (cache-prefill with history), on the staged route (the dequantising pass) and
    on the in-kernel route, with the same two oversized slabs."""
    seqlens, start = [1, 1, 600, 300, 260], [900, 17, 1500, 64, 0]  # chunks long enough for the plan to stage them
    if layout == 0:
        tokens, L, layer = (2 ** 32) // 65536 + 5003, 32, 31
    else:
        tokens, L, layer = (2 ** 32) // (8 * 128) + 4099, 1, 0
    plan = _check(layout, L, layer, tokens, 32, 8, 128, seqlens, start, 2, cache_prefill=1, staging=staging)
    assert plan.prefill_staging == (1 if staging is None else 0)
