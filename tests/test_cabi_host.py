"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares, the ctypes
mirrors match the header's field lists, and host-only validation returns the reference's error codes."""
import ctypes as C
import os
import re

import pytest

import harness
from harness import cabi, workloads

HEADER = os.path.join(harness.ROOT, "include", "ppl_llm_kernel_hip.h")
PROBES_HEADER = os.path.join(harness.ROOT, "include", "ppl_llm_kernel_hip_probes.h")


def header_text(path=HEADER):
    with open(path) as f:
        return f.read()


def test_library_exports_every_declared_symbol(hiplib):
    txt = re.sub(r"/\*.*?\*/", "", header_text(), flags=re.S)
    declared = set(re.findall(r"\b(pplhip_[a-z0-9_]+)\s*\(", txt))
    assert declared == set(cabi.PROTOTYPES), declared ^ set(cabi.PROTOTYPES)
    for name in declared:
        assert hasattr(hiplib, name)
    assert hiplib.pplhip_version() >= 100
    assert hiplib.pplhip_last_error() is not None
    assert not any("probe" in name for name in declared)  # the drop-in ABI carries no measurement aids


def test_probe_library_exports_every_declared_symbol(probelib):
    txt = re.sub(r"/\*.*?\*/", "", header_text(PROBES_HEADER), flags=re.S)
    declared = set(re.findall(r"\b(pplhip_[a-z0-9_]+)\s*\(", txt))
    assert declared == set(cabi.PROBE_PROTOTYPES), declared ^ set(cabi.PROBE_PROTOTYPES)
    for name in declared:
        assert hasattr(probelib, name)
    assert probelib.pplhip_probe_last_error() == b""
    assert probelib.pplhip_probe_quantizer(None, None) == cabi.RC_INVALID_VALUE  # host-side check, no device call
    assert b"null counter" in probelib.pplhip_probe_last_error()


@pytest.mark.parametrize("cname,cls", [("pplhip_mhca_args", cabi.MhcaArgs), ("pplhip_mhca_plan", cabi.MhcaPlan),
                                       ("pplhip_kv_write_args", cabi.KvWriteArgs),
                                       ("pplhip_kv_cache_args", cabi.KvCacheArgs), ("pplhip_pack_args", cabi.PackArgs),
                                       ("pplhip_mha_args", cabi.MhaArgs), ("pplhip_rope_args", cabi.RopeArgs)])
def test_ctypes_mirror_matches_header(cname, cls):
    txt = re.sub(r"/\*.*?\*/", "", header_text(), flags=re.S)
    body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), txt, flags=re.S).group(1)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        names.append(re.sub(r"\[.*\]", "", decl.split()[-1].lstrip("*")))
    assert names == [f[0] for f in cls._fields_]


def _valid_args():
    b = workloads.Batch(8, 2, 128, [1, 5], [10, 0], 1)
    a = cabi.MhcaArgs()
    fake = lambda t: C.c_void_p(0x1000)  # prepare never dereferences device pointers
    harness.fill_mhca_args(a, b, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, ptr=fake)
    return a


def test_prepare_accepts_valid_and_sizes_workspace(hiplib):
    a, plan = _valid_args(), cabi.MhcaPlan()
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS
    # 1 decode sequence of 11 tokens: one 128-token piece at most -> 8 ranges (the floor), 2 kv heads per workgroup
    assert plan.decode_num_ranges == 8 and plan.decode_heads_per_block == 2 and plan.decode_waves_per_block == 4
    assert plan.workspace_bytes >= (8 + 1) * 8 * 130 * 4 and plan.workspace_bytes % 256 == 0
    assert plan.prefill_q_tile == 128 and plan.prefill_num_q_tiles == 1
    sizes = []
    for mode in (0, 1, 2):
        a.max_kvlen, a.specify_decoding_attn_split_k = 1000000, mode
        assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS
        assert plan.decode_num_ranges >= 8
        assert plan.workspace_bytes >= (plan.decode_num_ranges + 1) * 8 * 130 * 4
        sizes.append(plan.decode_num_ranges)
    assert sizes[0] < sizes[1] < sizes[2]


@pytest.mark.parametrize("mutate,rc", [
    (lambda a: setattr(a, "d_alibi_slopes", 0x10), cabi.RC_UNSUPPORTED),  # …_kernel.cc:95-98
    (lambda a: setattr(a, "d_scale", None), cabi.RC_UNSUPPORTED),  # …_kernel.cc:100-103
    (lambda a: setattr(a, "d_attn_mask", 0x10), cabi.RC_INVALID_VALUE),  # a mask without its row stride
    (lambda a: (setattr(a, "d_attn_mask", 0x11), setattr(a, "attn_mask_stride_q", 64)), cabi.RC_INVALID_VALUE),
    (lambda a: (setattr(a, "d_attn_mask", 0x10), setattr(a, "attn_mask_stride_q", 64),
                setattr(a, "attn_mask_stride_h", -1)), cabi.RC_INVALID_VALUE),
    (lambda a: setattr(a, "cache_mode", 1), cabi.RC_INVALID_VALUE),  # no 2-d page table: …_kernel.cc:162-166
    (lambda a: setattr(a, "cache_mode", 2), cabi.RC_UNSUPPORTED),
    (lambda a: (setattr(a, "cache_mode", 1), setattr(a, "cachestart_stride_b", 4), setattr(a, "page_size", 96)),
     cabi.RC_UNSUPPORTED),
    (lambda a: (setattr(a, "cache_mode", 1), setattr(a, "cachestart_stride_b", 4), setattr(a, "page_size", 32)),
     cabi.RC_UNSUPPORTED),
    (lambda a: setattr(a, "head_dim", 72), cabi.RC_UNSUPPORTED),  # multiples of 16 up to 256
    (lambda a: setattr(a, "head_dim", 288), cabi.RC_UNSUPPORTED),
    (lambda a: setattr(a, "num_kv_heads", 3), cabi.RC_INVALID_VALUE),
    (lambda a: setattr(a, "layer_idx", 5), cabi.RC_INVALID_VALUE),
    (lambda a: setattr(a, "decoding_batches", 3), cabi.RC_INVALID_VALUE),
    (lambda a: setattr(a, "cache_stride_s", 100), cabi.RC_INVALID_VALUE),
    # offsets inside a stage / tile are 32-bit in the kernels: a token stride of 2^25 elements or more is refused
    (lambda a: setattr(a, "cache_stride_s", 1 << 25), cabi.RC_UNSUPPORTED),
    (lambda a: setattr(a, "d_query", None), cabi.RC_INVALID_VALUE),
    (lambda a: setattr(a, "specify_decoding_attn_split_k", 7), cabi.RC_INVALID_VALUE),
    (lambda a: setattr(a, "specify_decoding_attn_tpb", 128), cabi.RC_INVALID_VALUE),
])
def test_prepare_rejects(hiplib, mutate, rc):
    a, plan = _valid_args(), cabi.MhcaPlan()
    mutate(a)
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == rc
    assert len(hiplib.pplhip_last_error()) > 0


@pytest.mark.parametrize("mutate", [
    lambda a: setattr(a, "head_dim", 64),
    lambda a: setattr(a, "head_dim", 256),
    lambda a: (setattr(a, "num_heads", 34), setattr(a, "num_kv_heads", 2)),  # 17 query heads per kv head
    lambda a: (setattr(a, "d_attn_mask", 0x10), setattr(a, "attn_mask_stride_q", 64)),
])
def test_prepare_routes_other_shapes_to_the_general_kernel(hiplib, mutate):
    """head_dim other than 128, more than 16 query heads per kv head, or an attn_mask: the plan says so and plans no
    split-k ranges; short decode sequences are not cut into pieces and need no workspace, long ones are and do."""
    a, plan = _valid_args(), cabi.MhcaPlan()
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS and plan.general_kernel == 0
    mutate(a)
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS, hiplib.pplhip_last_error()
    assert plan.general_kernel == 1 and plan.workspace_bytes == 0 and plan.decode_num_ranges == 0
    assert plan.general_decode_splits <= 1
    a.max_kvlen = 4096  # 1 decode sequence: 64 pieces of one tile
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS, hiplib.pplhip_last_error()
    assert plan.general_kernel == 1 and plan.general_decode_splits == 64 and plan.decode_num_ranges == 0
    assert plan.workspace_bytes >= 1 * a.num_heads * 64 * (a.head_dim + 2) * 4 and plan.workspace_bytes % 256 == 0
    a.max_kvlen = 1 << 20  # no more than 64 pieces: they grow instead
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS, hiplib.pplhip_last_error()
    assert plan.general_decode_splits == 64
    a.decoding_batches = 0  # no decode sequence, nothing to cut
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS, hiplib.pplhip_last_error()
    assert plan.general_decode_splits <= 1 and plan.workspace_bytes == 0


def test_prepare_plans_head_dim_64_and_32_decode_over_groups_of_kv_heads(hiplib):
    """head_dim 64 (32) with kv heads that are neighbours in the slab and pair up (go in fours): the general plan
    carries the decode kernel's ranges for the decode sequences; anything that breaks the grouping (odd kv heads, more
    than 16 query heads per group, heads apart in the slab, a mask) plans the general decode kernel."""
    def plan_of(H, KVH, Dh, stride_h=None, mask=False):
        b = workloads.Batch(H, KVH, Dh, [1] * 40 + [9], [3000] * 40 + [0], 40)
        a = cabi.MhcaArgs()
        fake = lambda t: C.c_void_p(0x1000)
        harness.fill_mhca_args(a, b, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, ptr=fake, split_k=1)
        if stride_h is not None:
            a.cache_stride_h = stride_h
        if mask:
            a.d_attn_mask, a.attn_mask_stride_q = 0x10, 4096
        plan = cabi.MhcaPlan()
        assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS, hiplib.pplhip_last_error()
        assert plan.general_kernel == 1
        return a, plan

    a, plan = plan_of(32, 8, 64)  # 4 groups of 2 kv heads, 8 query heads each: one workgroup per range
    assert plan.decode_num_ranges == 512 and plan.decode_heads_per_block == 4 and plan.general_decode_splits == 1
    assert plan.workspace_bytes >= (512 + 40) * 32 * 130 * 4 + 512 * 4 and plan.workspace_bytes % 256 == 0
    a, plan = plan_of(32, 8, 32)  # 2 groups of 4 kv heads, 16 query heads each
    assert plan.decode_num_ranges == 512 and plan.decode_heads_per_block == 2
    for args in ((28, 7, 64), (72, 8, 64), (40, 8, 32)):  # odd kv heads; 18 and 20 query heads per group
        a, plan = plan_of(*args)
        assert plan.decode_num_ranges == 0 and plan.general_decode_splits > 1
    a, plan = plan_of(32, 8, 64, stride_h=4096)  # heads apart in the slab (cache_layout 3)
    assert plan.decode_num_ranges == 0
    a, plan = plan_of(32, 8, 64, mask=True)
    assert plan.decode_num_ranges == 0
    a, plan = plan_of(32, 8, 96)
    assert plan.decode_num_ranges == 0


@pytest.mark.parametrize("kvh", [1, 2, 3, 4, 5, 8, 12, 16, 32, 40, 64])
def test_decode_plan_fills_one_round_of_workgroup_slots(hiplib, kvh):
    """The decode launch runs (ranges x groups of <= 4 kv heads) workgroups, two per compute unit: with the default
    knob they must fit the 512 slots of the 256-CU part (that is also what prepare assumes without a device), or a
    nearly empty second round doubles the time; and they must leave fewer slots empty than one more range would take."""
    b = workloads.Batch(kvh * 2, kvh, 128, [1] * 200, [4000] * 200, 200)
    a = cabi.MhcaArgs()
    fake = lambda t: C.c_void_p(0x1000)
    harness.fill_mhca_args(a, b, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, ptr=fake, split_k=1)
    plan = cabi.MhcaPlan()
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS
    groups = kvh // plan.decode_heads_per_block
    assert kvh % plan.decode_heads_per_block == 0 and plan.decode_heads_per_block <= 4
    assert plan.decode_num_ranges >= 8
    assert plan.decode_num_ranges * groups <= 512 or plan.decode_num_ranges == 8
    assert (plan.decode_num_ranges + 1) * groups > 512  # one more range would spill into a second round


def test_cache_prefill_plan_stages_large_chunks_only(hiplib):
    """Cache-prefill: chunks of >= 1024 / (query heads per kv head) new tokens per prompt on average make the plan stage
    the prompts' cached K/V as fp16 rows behind the decode part of the workspace (worst case: every prompt max_kvlen
    long); small chunks, more than 1 GiB of staging rows, or no cache-prefill leave the workspace as it was."""
    fake = lambda t: C.c_void_p(0x1000)

    def plan_of(seqlens, hist, nd, cache_prefill):
        b = workloads.Batch(32, 8, 128, seqlens, hist, nd)
        a = cabi.MhcaArgs()
        harness.fill_mhca_args(a, b, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, ptr=fake, split_k=1, cache_prefill=cache_prefill)
        plan = cabi.MhcaPlan()
        assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS
        return b, plan

    b, base = plan_of([1, 1, 512, 300], [100, 900, 4096, 0], 2, 0)
    assert base.prefill_staging == 0
    b, staged = plan_of([1, 1, 512, 300], [100, 900, 4096, 0], 2, 1)
    assert staged.prefill_staging == 1
    assert staged.prefill_staging_offset_256 * 256 == base.workspace_bytes
    rows = 2 * b.max_kvlen  # two prompts
    assert staged.workspace_bytes == base.workspace_bytes + rows * 2 * 8 * 128 * 2
    _, small = plan_of([1, 1, 100, 200], [100, 900, 4096, 0], 2, 1)  # 150 new tokens per prompt on average x 4 < 1024
    _, small0 = plan_of([1, 1, 100, 200], [100, 900, 4096, 0], 2, 0)
    assert small.prefill_staging == 0 and small.workspace_bytes == small0.workspace_bytes
    _, huge = plan_of([1, 1, 512, 300] + [300] * 30, [100, 900, 16384, 0] + [0] * 30, 2, 1)  # 32 x 16896 rows x 4 KB > 1 GiB
    assert huge.prefill_staging == 0


def test_prepare_accepts_plane_strides_beyond_32_bits(hiplib):
    """cache_layout 3 puts KVH * MaxT * Dh elements between the K and the V plane (multi_head_cache_attention_kernel.cc:
    149-155): more than 4 GiB with a large slab. The kernels carry that distance in 64 bits, so prepare accepts it;
    only the distance between two tokens is limited."""
    a, plan = _valid_args(), cabi.MhcaPlan()
    a.cache_stride_kv, a.cache_stride_l, a.cache_stride_h, a.cache_stride_s = 1 << 33, 1 << 34, 1 << 30, 128
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS
    a.cache_stride_s = (1 << 25) - 16
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS


def test_prepare_accepts_paged_cache(hiplib):
    a, plan = _valid_args(), cabi.MhcaPlan()
    a.cache_mode, a.cachestart_stride_b, a.page_size = 1, 4, 128
    assert hiplib.pplhip_mhca_prepare(C.byref(a), C.byref(plan)) == cabi.RC_SUCCESS


def test_kv_cache_rejects_like_the_reference_stub(hiplib):
    # key_value_cache_kernel.cc:73-96: layout != 0, mode != 0, num_repeat != 1 -> RC_UNSUPPORTED
    for field in ("cache_layout", "cache_mode", "num_repeat"):
        a = cabi.KvCacheArgs()
        a.num_repeat = 1
        setattr(a, field, 3)
        assert hiplib.pplhip_kv_cache_forward(C.byref(a), None) == cabi.RC_UNSUPPORTED


def test_mha_rejects_like_the_reference_wrapper(hiplib):
    def args(**kw):
        a = cabi.MhaArgs()
        for f in ("d_query", "d_key", "d_value", "d_seqstarts", "d_kvstarts", "d_output"):
            setattr(a, f, 0x1000)
        a.is_causal, a.batch, a.max_seqlen, a.max_kvlen = 1, 0, 0, 0  # batch 0: validation only, nothing launched
        a.num_heads, a.num_kv_heads, a.head_dim = 8, 2, 128
        for k, v in kw.items():
            setattr(a, k, v)
        return a
    assert hiplib.pplhip_mha_forward(C.byref(args()), None) == cabi.RC_SUCCESS
    # multi_head_attention_kernel.cc:71-74
    assert hiplib.pplhip_mha_forward(C.byref(args(is_alibi=1)), None) == cabi.RC_UNSUPPORTED
    assert b"is_alibi" in hiplib.pplhip_last_error()
    assert hiplib.pplhip_mha_forward(C.byref(args(d_attn_mask=0x1000)), None) == cabi.RC_INVALID_VALUE  # no stride
    assert hiplib.pplhip_mha_forward(C.byref(args(d_attn_mask=0x1000, attn_mask_stride_q=8)), None) == cabi.RC_SUCCESS
    assert hiplib.pplhip_mha_forward(C.byref(args(head_dim=64)), None) == cabi.RC_SUCCESS
    assert hiplib.pplhip_mha_forward(C.byref(args(head_dim=72)), None) == cabi.RC_UNSUPPORTED
    assert hiplib.pplhip_mha_forward(C.byref(args(num_kv_heads=3)), None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_mha_forward(C.byref(args(batch=1, max_seqlen=4, max_kvlen=2)), None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_mha_forward(C.byref(args(batch=1, max_seqlen=1, max_kvlen=2, d_key=0)), None) == \
        cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_mha_forward(None, None) == cabi.RC_INVALID_VALUE


def test_rope_rejects(hiplib):
    def args(**kw):
        a = cabi.RopeArgs()
        for f in ("d_query", "d_key", "d_start_pos", "d_seqstarts", "d_rotated_query", "d_rotated_key"):
            setattr(a, f, 0x1000)
        a.theta, a.batch, a.total_tokens = 10000.0, 0, 0  # batch 0: validation only, nothing launched
        a.num_heads, a.num_key_heads, a.head_dim, a.scaling_factor = 8, 2, 128, 1.0
        a.max_position_embeddings = 2048
        for k, v in kw.items():
            setattr(a, k, v)
        return a
    assert hiplib.pplhip_rope_forward(C.byref(args()), None) == cabi.RC_SUCCESS
    # rotary_position_embedding_kernel.cc:105-108: "invalid scaling type"
    assert hiplib.pplhip_rope_forward(C.byref(args(scaling_type=3)), None) == cabi.RC_INVALID_VALUE
    assert b"invalid scaling type" in hiplib.pplhip_last_error()
    assert hiplib.pplhip_rope_forward(C.byref(args(rotary_dim=12)), None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_rope_forward(C.byref(args(rotary_dim=256)), None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_rope_forward(C.byref(args(head_dim=100)), None) == cabi.RC_UNSUPPORTED
    assert hiplib.pplhip_rope_forward(C.byref(args(theta=0.0)), None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_rope_forward(C.byref(args(scaling_type=1, scaling_factor=0.0)), None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_rope_forward(C.byref(args(batch=1, total_tokens=1, d_key=0)), None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_position_index(0x1000, 0x1000, -1, 0, 0, 0x1000, None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_position_index(0x1000, 0x1000, 1, 1, 1, None, None) == cabi.RC_INVALID_VALUE
    assert hiplib.pplhip_position_index(0x1000, 0x1000, 0, 0, 0, None, None) == cabi.RC_SUCCESS


def test_pack_rejects_bad_slot_count(hiplib):
    a = cabi.PackArgs()
    for f, _ in cabi.PackArgs._fields_:
        if f.startswith("d_"):
            setattr(a, f, 0x1000)
    a.num_slots = 5000
    assert hiplib.pplhip_pack_tables(C.byref(a), None) == cabi.RC_INVALID_VALUE


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(harness.pkg, "_LIB", None)
    monkeypatch.setattr(harness.pkg, "LIB_PATH", "/nonexistent/libppl_llm_kernel_hip.so")
    with pytest.raises(harness.pkg.LibraryMissing):
        harness.pkg.load_library()


def test_slab_addressing_is_64_bit(probelib):
    """The struct every kernel forms its slab offsets with, compiled for the host, against Python's integers: both
    cache layouts at sizes whose offsets need up to 45 bits, and random strides up to 2^34 elements."""
    import random
    rng = random.Random(7)
    row, srow = C.c_int64(), C.c_int64()
    cases = []
    for L, KVH, Dh, tokens in ((32, 8, 128, 70000), (80, 8, 128, 2 ** 22), (1, 8, 128, 2 ** 22 + 4099), (48, 40, 256, 2 ** 21)):
        for st in (cabi.cache_strides_layout0(L, KVH, Dh), cabi.cache_strides_layout3(L, KVH, Dh, tokens)):
            for _ in range(50):
                cases.append((st["cache_stride_s"], st["cache_stride_l"], st["cache_stride_h"], st["cache_stride_kv"],
                              rng.randrange(L), rng.randrange(tokens), rng.randrange(2), rng.randrange(KVH)))
            cases.append((st["cache_stride_s"], st["cache_stride_l"], st["cache_stride_h"], st["cache_stride_kv"],
                          L - 1, tokens - 1, 1, KVH - 1))
    for _ in range(500):
        cases.append(tuple(16 * rng.randrange(1, 2 ** 30) for _ in range(4)) +
                     (rng.randrange(128), rng.randrange(2 ** 22), rng.randrange(2), rng.randrange(64)))
    beyond = 0
    for ss, sl, sh, skv, layer, tok, kv, head in cases:
        want = tok * ss + layer * sl + kv * skv + head * sh
        if want >= 2 ** 63:
            continue
        assert probelib.pplhip_probe_slab_row(ss, sl, sh, skv, layer, tok, kv, head, C.byref(row), C.byref(srow)) == 0
        assert row.value == want and srow.value == want // 8, (ss, sl, sh, skv, layer, tok, kv, head)
        beyond += want > 2 ** 32
    assert beyond > 400
