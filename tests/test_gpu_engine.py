"""End to end through the llm_hip host engine on the GPU: an ONNX graph with one OPMX node is loaded by the wire reader,
partitioned to the engine, and run by the sequential runtime; results must equal the oracle's (same bar as the C ABI)."""
import ctypes as C

import numpy as np
import pytest

import harness
from ppl_nn_amd import onnx_writer as ow
from harness import cabi, workloads

pytestmark = pytest.mark.gpu


def _i64(*dims):
    return (C.c_int64 * len(dims))(*dims), len(dims)


class Session:
    def __init__(self, eng, model_bytes, configure=(), mm_policy=1):
        self.eng = eng
        self.engine = eng.pplnn_hip_engine_create(0, mm_policy)  # 0 MM_PLAIN, 1 MM_COMPACT, 2 MM_BEST_FIT
        assert self.engine
        for opt, val in configure:
            assert eng.pplnn_hip_engine_configure_u32(self.engine, opt, val) == 0
        self.builder = eng.pplnn_hip_builder_create()
        assert eng.pplnn_hip_builder_load_model(self.builder, model_bytes, len(model_bytes)) == 0
        assert eng.pplnn_hip_builder_set_engine(self.builder, self.engine) == 0
        assert eng.pplnn_hip_builder_preprocess(self.builder) == 0, eng.pplnn_hip_last_error()
        self.rt = eng.pplnn_hip_builder_create_runtime(self.builder)
        assert self.rt, eng.pplnn_hip_last_error()
        self.keep = []

    def input(self, i):
        return self.eng.pplnn_hip_runtime_input(self.rt, i)

    def set_device_tensor(self, i, t):  # borrowed device memory, like the caller-owned KV slab
        tensor = self.input(i)
        dims, n = _i64(*t.shape)
        self.eng.pplnn_hip_tensor_reshape(tensor, dims, n)
        self.eng.pplnn_hip_tensor_set_buffer_ptr(tensor, t.data_ptr())
        self.keep.append(t)

    def set_table(self, i, a):  # copied into an arena buffer of the engine's device
        tensor = self.input(i)
        dims, n = _i64(*a.shape)
        self.eng.pplnn_hip_tensor_reshape(tensor, dims, n)
        a = np.ascontiguousarray(a)
        assert self.eng.pplnn_hip_tensor_copy_from_host(tensor, a.ctypes.data) == 0
        self.keep.append(a)

    def set_host_scalar(self, i, v):  # decoding_batches / max_seqlen / max_kvlen live on the host device
        tensor = self.input(i)
        self.eng.pplnn_hip_tensor_use_host_device(tensor)
        self.eng.pplnn_hip_tensor_reshape(tensor, None, 0)
        a = np.array([v], np.int64)
        assert self.eng.pplnn_hip_tensor_copy_from_host(tensor, a.ctypes.data) == 0

    def output(self, i, dtype):
        tensor = self.eng.pplnn_hip_runtime_output(self.rt, i)
        dims = (C.c_int64 * 8)()
        n = self.eng.pplnn_hip_tensor_dims(tensor, dims, 8)
        out = np.empty(tuple(dims[:n]), dtype)
        assert self.eng.pplnn_hip_tensor_copy_to_host(tensor, out.ctypes.data) == 0
        return out

    def close(self):
        self.eng.pplnn_hip_runtime_destroy(self.rt)
        self.eng.pplnn_hip_builder_destroy(self.builder)
        self.eng.pplnn_hip_engine_destroy(self.engine)


def _prepare_slab(b, t, hiplib):
    """History written through the C ABI into torch-owned slab memory (the caller owns the slab)."""
    import torch
    cache_h, scale_h = harness.new_slab(b)
    cache, scale = harness.to_dev(cache_h), harness.to_dev(scale_h)
    if b.total_hist_tokens:
        hk, hv = harness.to_dev(t["hist_key"]), harness.to_dev(t["hist_value"])
        hs, z, cs = harness.to_dev(b.histstarts), harness.to_dev(np.zeros(b.batch, np.int64)), harness.to_dev(b.cachestarts)
        w = harness.fill_write_args(cabi.KvWriteArgs(), b, hk, hv, hs, z, cs, cache, scale, ptr=harness.dev_ptr)
        harness.pkg.check(hiplib.pplhip_kv_quantize_write(C.byref(w), None), "history")
        torch.cuda.synchronize()
    return cache, scale


@pytest.mark.parametrize("cache_prefill,mm_policy", [(0, 1), (1, 1), (0, 0), (1, 2)])
def test_mhca_graph_through_the_engine(hiplib, cache_prefill, mm_policy):
    import torch
    eng = harness.pkg.load_engine_library()
    b = workloads.Batch(32, 8, 128, [1, 1, 1, 1, 70, 200], [500, 3, 77, 1300, 0, 0], 4, num_layer=2, layer_idx=1,
                        name="engine_mhca")
    t = workloads.make_tensors(b, seed=77)
    ref = harness.run_oracle(b, t, cache_prefill=cache_prefill)
    cache, scale = _prepare_slab(b, t, hiplib)
    s = Session(eng, ow.mhca_model(32, 8, 128, 2, 1), configure=[(1005, cache_prefill)], mm_policy=mm_policy)
    assert eng.pplnn_hip_runtime_input_count(s.rt) == 12 and eng.pplnn_hip_runtime_output_count(s.rt) == 1
    assert eng.pplnn_hip_runtime_set_profiling(s.rt, 1) == 0
    s.set_device_tensor(0, harness.to_dev(t["query"]))
    s.set_device_tensor(1, harness.to_dev(t["current_key"]))
    s.set_device_tensor(2, harness.to_dev(t["current_value"]))
    s.set_table(3, b.seqstarts)
    s.set_table(4, b.kvstarts)
    s.set_table(5, b.cachestarts)
    s.set_table(6, b.start_pos)
    s.set_host_scalar(7, b.decoding_batches)
    s.set_host_scalar(8, b.max_seqlen)
    s.set_host_scalar(9, b.max_kvlen)
    s.set_device_tensor(10, cache)
    s.set_device_tensor(11, scale)
    for _ in range(2):  # the second run reuses arena buffers and must give the same answer
        assert eng.pplnn_hip_runtime_run(s.rt) == 0, eng.pplnn_hip_last_error()
        out = s.output(0, np.float16)
        assert out.shape == (b.total_new_tokens, 32, 128)
        harness.assert_attn_close(out, ref["output_f64"])
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), ref["cache"])
    assert np.array_equal(scale.cpu().view(torch.int16).numpy().view(np.uint16), ref["scale"].view(np.uint16))
    micros, counts = (C.c_uint64 * 4)(), (C.c_uint32 * 4)()
    assert eng.pplnn_hip_runtime_profiling(s.rt, micros, counts, 4) == 1
    assert counts[0] == 2 and micros[0] > 0
    s.close()


@pytest.mark.parametrize("head_dim,mask_rank", [(64, 0), (64, 3), (128, 2), (256, 0), (80, 0), (112, 3)])
def test_mhca_graph_other_head_dims_and_attn_mask(hiplib, head_dim, mask_rank):
    """The same graph with a head_dim other than 128 and / or the optional 13th input attn_mask: the engine reads the
    mask's strides off its shape and the call runs the general kernel."""
    import torch
    from test_oracle_attention import _mask_for
    eng = harness.pkg.load_engine_library()
    b = workloads.Batch(8, 2, head_dim, [1, 1, 70, 130], [500, 3, 0, 0], 2, num_layer=2, layer_idx=1, name="engine_general")
    t = workloads.make_tensors(b, seed=78)
    mask = _mask_for(b, np.random.default_rng(1), per_head=mask_rank == 3) if mask_rank else None
    ref = harness.run_oracle(b, t, mask=mask)
    cache, scale = _prepare_slab(b, t, hiplib)
    s = Session(eng, ow.mhca_model(8, 2, head_dim, 2, 1, mask_rank=mask_rank))
    assert eng.pplnn_hip_runtime_input_count(s.rt) == 12 + (1 if mask_rank else 0)
    for i, name in enumerate(("query", "current_key", "current_value")):
        s.set_device_tensor(i, harness.to_dev(t[name]))
    for i, tab in enumerate((b.seqstarts, b.kvstarts, b.cachestarts, b.start_pos)):
        s.set_table(3 + i, tab)
    for i, v in enumerate((b.decoding_batches, b.max_seqlen, b.max_kvlen)):
        s.set_host_scalar(7 + i, v)
    s.set_device_tensor(10, cache)
    s.set_device_tensor(11, scale)
    if mask_rank:
        s.set_device_tensor(12, harness.to_dev(mask))
    print(f"case {b.name} head_dim={head_dim} mask_rank={mask_rank}", flush=True)
    assert eng.pplnn_hip_runtime_run(s.rt) == 0, eng.pplnn_hip_last_error()
    out = s.output(0, np.float16)
    assert out.shape == (b.total_new_tokens, 8, head_dim)
    harness.assert_attn_close(out, ref["output_f64"])
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), ref["cache"])
    s.close()


def test_engine_error_paths_on_device(hiplib):
    eng = harness.pkg.load_engine_library()
    eng.pplnn_hip_set_log_level(4)
    b = workloads.Batch(8, 2, 128, [1, 5], [10, 0], 1)
    t = workloads.make_tensors(b, seed=5)
    cache, scale = _prepare_slab(b, t, hiplib)

    def run(model, skip=()):
        s = Session(eng, model)
        tensors = [harness.to_dev(t["query"]), harness.to_dev(t["current_key"]), harness.to_dev(t["current_value"])]
        for i in range(3):
            s.set_device_tensor(i, tensors[i])
        for i, a in zip(range(3, 7), (b.seqstarts, b.kvstarts, b.cachestarts, b.start_pos)):
            s.set_table(i, a)
        for i, v in zip(range(7, 10), (b.decoding_batches, b.max_seqlen, b.max_kvlen)):
            s.set_host_scalar(i, v)
        s.set_device_tensor(10, cache)
        if 11 not in skip and eng.pplnn_hip_runtime_input_count(s.rt) > 11:
            s.set_device_tensor(11, scale)
        rc = eng.pplnn_hip_runtime_run(s.rt)
        s.close()
        return rc

    assert run(ow.mhca_model(8, 2, 128, 1, 0)) == 0
    assert run(ow.mhca_model(8, 2, 128, 1, 0, extra_attrs={"is_alibi": 1})) == cabi.RC_UNSUPPORTED  # …_kernel.cc:95-98
    assert run(ow.mhca_model(8, 2, 128, 1, 0, with_scale=False)) == cabi.RC_UNSUPPORTED  # …_kernel.cc:100-103
    assert run(ow.mhca_model(8, 2, 128, 1, 0, extra_attrs={"cache_layout": 2})) == cabi.RC_UNSUPPORTED  # :156-159
    assert run(ow.mhca_model(8, 2, 128, 1, 0, extra_attrs={"cache_mode": 1})) == cabi.RC_INVALID_VALUE  # :163-166
    assert run(ow.mhca_model(8, 2, 128, 1, 0, extra_attrs={"quant_bit": 4, "quant_group": 4})) == cabi.RC_UNSUPPORTED


def test_kv_cache_graph_through_the_engine(hiplib, olib):
    eng = harness.pkg.load_engine_library()
    b = workloads.Batch(4, 4, 128, [1, 6, 1, 40], [9, 0, 3, 0], 0, num_layer=2, layer_idx=1)
    t = workloads.make_tensors(b, seed=9)
    # oracle
    cache_o, scale_o = harness.new_slab(b)
    zeros = np.zeros(b.batch, np.int64)
    w = harness.fill_write_args(cabi.KvWriteArgs(), b, t["hist_key"], t["hist_value"], b.histstarts, zeros, b.cachestarts,
                                cache_o, scale_o)
    assert olib.oracle_kv_quantize_write(C.byref(w)) == 0
    a = cabi.KvCacheArgs()
    ss, ks = b.seqstarts, b.kvstarts
    harness.fill_write_args(a.write, b, t["current_key"], t["current_value"], ss, b.start_pos, b.cachestarts, cache_o, scale_o)
    a.d_kvstarts, a.total_kv_tokens, a.max_kvlen = ks.ctypes.data, int(ks[-1]), b.max_kvlen
    a.num_repeat = 1
    ko, vo = np.zeros((int(ks[-1]), 4, 128), np.float16), np.zeros((int(ks[-1]), 4, 128), np.float16)
    a.d_key_out, a.d_value_out = ko.ctypes.data, vo.ctypes.data
    assert olib.oracle_kv_cache_forward(C.byref(a)) == 0
    # engine
    cache, scale = _prepare_slab(b, t, hiplib)
    s = Session(eng, ow.kv_cache_model(2, 1))
    s.set_device_tensor(0, harness.to_dev(t["current_key"]))
    s.set_device_tensor(1, harness.to_dev(t["current_value"]))
    for i, tab in zip(range(2, 6), (b.seqstarts, b.kvstarts, b.cachestarts, b.start_pos)):
        s.set_table(i, tab)
    s.set_host_scalar(6, b.max_seqlen)
    s.set_host_scalar(7, b.max_kvlen)
    s.set_device_tensor(8, cache)
    s.set_device_tensor(9, scale)
    assert eng.pplnn_hip_runtime_run(s.rt) == 0, eng.pplnn_hip_last_error()
    key, value = s.output(0, np.float16), s.output(1, np.float16)
    assert key.shape == ko.shape  # dim 0 = kvstarts[B], read back like reshape_dynamic_batching_key_value_cache.cc:43-53
    assert np.array_equal(key.view(np.uint16), ko.view(np.uint16)) and np.array_equal(value.view(np.uint16), vo.view(np.uint16))
    s.close()


def _rope_on_oracle(olib, q, k, b, theta):
    qo, ko = np.zeros_like(q), np.zeros_like(k)
    a = harness.fill_rope_args(cabi.RopeArgs(), q, k, b.seqlens, b.start_pos, qo, ko, theta=theta)
    assert olib.oracle_rope_forward(C.byref(a)) == 0
    return qo, ko


def test_rope_then_mhca_graph(hiplib, olib):
    """Two nodes: RotaryPositionEmbedding -> MultiHeadCacheAttention; rotated_query / rotated_key are intermediate
    tensors of the runtime (allocated from the engine's arena, released after the attention node)."""
    import torch
    eng = harness.pkg.load_engine_library()
    b = workloads.Batch(8, 2, 128, [1, 1, 50, 131], [700, 12, 0, 0], 2, num_layer=1, layer_idx=0, name="engine_rope_mhca")
    t = workloads.make_tensors(b, seed=41)
    theta = 500000.0
    # oracle: rotate, then attend (the rotated fp16 tensors are what the attention node sees)
    rq, rk = _rope_on_oracle(olib, t["query"], t["current_key"], b, theta)
    t_rot = dict(t, query=rq, current_key=rk)
    ref = harness.run_oracle(b, t_rot)
    cache, scale = _prepare_slab(b, t, hiplib)
    s = Session(eng, ow.rope_mhca_model(8, 2, 128, 1, 0, theta))
    assert eng.pplnn_hip_runtime_input_count(s.rt) == 12
    s.set_device_tensor(0, harness.to_dev(t["query"]))
    s.set_device_tensor(1, harness.to_dev(t["current_key"]))
    s.set_device_tensor(2, harness.to_dev(t["current_value"]))
    for i, tab in zip(range(3, 7), (b.seqstarts, b.kvstarts, b.cachestarts, b.start_pos)):
        s.set_table(i, tab)
    for i, v in zip(range(7, 10), (b.decoding_batches, b.max_seqlen, b.max_kvlen)):
        s.set_host_scalar(i, v)
    s.set_device_tensor(10, cache)
    s.set_device_tensor(11, scale)
    for _ in range(2):
        assert eng.pplnn_hip_runtime_run(s.rt) == 0, eng.pplnn_hip_last_error()
        out = s.output(0, np.float16)
        # the rotated inputs may differ from the oracle's by one fp16 ulp -> same attention tolerance still holds
        harness.assert_attn_close(out, ref["output_f64"], abs_tol=3e-3)
    torch.cuda.synchronize()
    # the K rows written to the slab are the ROTATED keys
    cache_h = cache.cpu().numpy()
    diff = np.abs(cache_h.astype(np.int32) - ref["cache"].astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.02  # one-ulp differences of the rotation move few int8 codes
    s.close()


@pytest.mark.parametrize("layout", [0, 1])
def test_rope_graph_with_the_engine_pair_layout_option(hiplib, olib, layout):
    """A RotaryPositionEmbedding node alone: ENGINE_CONF_ROPE_PAIR_LAYOUT (1006) selects consecutive-channel or
    half-split pairs for every such node of the engine; each must match the oracle run with the same layout."""
    eng = harness.pkg.load_engine_library()
    rng = np.random.default_rng(43)
    seqlens, start = np.array([1, 9, 130], np.int64), np.array([4000, 0, 77], np.int64)
    T = int(seqlens.sum())
    q = rng.standard_normal((T, 8, 128)).astype(np.float16)
    k = rng.standard_normal((T, 2, 128)).astype(np.float16)
    qo, ko = np.zeros_like(q), np.zeros_like(k)
    a = harness.fill_rope_args(cabi.RopeArgs(), q, k, seqlens, start, qo, ko, theta=500000.0, pair_layout=layout)
    assert olib.oracle_rope_forward(C.byref(a)) == 0
    s = Session(eng, ow.rope_model(ow.rope_attrs(500000.0)), configure=[(1006, layout)])
    s.set_device_tensor(0, harness.to_dev(q))
    s.set_device_tensor(1, harness.to_dev(k))
    s.set_table(2, np.concatenate([[0], np.cumsum(seqlens)]).astype(np.int64))
    s.set_table(3, start)
    s.set_host_scalar(4, int(seqlens.max()))
    assert eng.pplnn_hip_runtime_run(s.rt) == 0, eng.pplnn_hip_last_error()
    for i, want in enumerate((qo, ko)):
        got = s.output(i, np.float16)
        ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float64)
        assert (np.abs(got.astype(np.float64) - want.astype(np.float64)) <= ulp + 1e-6).all()
    s.close()


def test_kv_cache_then_mha_graph_equals_mhca(hiplib):
    import torch
    eng = harness.pkg.load_engine_library()
    b = workloads.Batch(8, 2, 128, [1, 1, 40, 200], [99, 7, 0, 0], 2, num_layer=2, layer_idx=1, name="engine_kvc_mha")
    t = workloads.make_tensors(b, seed=42)
    mhca = harness.run_device(b, t, cache_prefill=1)
    cache, scale = _prepare_slab(b, t, hiplib)
    s = Session(eng, ow.kv_cache_mha_model(8, 2, 128, 2, 1))
    s.set_device_tensor(0, harness.to_dev(t["query"]))
    s.set_device_tensor(1, harness.to_dev(t["current_key"]))
    s.set_device_tensor(2, harness.to_dev(t["current_value"]))
    for i, tab in zip(range(3, 7), (b.seqstarts, b.kvstarts, b.cachestarts, b.start_pos)):
        s.set_table(i, tab)
    for i, v in zip(range(7, 10), (b.decoding_batches, b.max_seqlen, b.max_kvlen)):
        s.set_host_scalar(i, v)
    s.set_device_tensor(10, cache)
    s.set_device_tensor(11, scale)
    assert eng.pplnn_hip_runtime_run(s.rt) == 0, eng.pplnn_hip_last_error()
    out = s.output(0, np.float16)
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), mhca["cache"])
    assert np.abs(out.astype(np.float64) - mhca["output"].astype(np.float64)).max() < 2e-3
    s.close()


def test_position_index_graph(hiplib):
    eng = harness.pkg.load_engine_library()
    seqlens, start = np.array([1, 9, 1, 30], np.int64), np.array([70, 0, 5, 100], np.int64)
    ss = np.concatenate([[0], np.cumsum(seqlens)]).astype(np.int64)
    s = Session(eng, ow.position_index_model())
    s.set_table(0, np.arange(int(ss[-1]), dtype=np.int64))  # token ids: only the shape and type matter
    s.set_table(1, ss)
    s.set_table(2, start)
    s.set_host_scalar(3, int(seqlens.max()))
    assert eng.pplnn_hip_runtime_run(s.rt) == 0, eng.pplnn_hip_last_error()
    out = s.output(0, np.int64)
    assert np.array_equal(out, np.concatenate([p + np.arange(n) for n, p in zip(seqlens, start)]))
    s.close()


def test_paged_mhca_graph_through_the_engine(hiplib):
    """cache_mode 1 through the op: the 2-d cachestarts tensor is the page table, its second extent the table stride."""
    import torch
    eng = harness.pkg.load_engine_library()
    b = workloads.Batch(8, 2, 128, [1, 1, 90], [700, 12, 0], 2, num_layer=1, layer_idx=0, name="engine_paged")
    t = workloads.make_tensors(b, seed=61)
    paged = harness.PagedLayout(b, page_size=128, seed=4)
    ref = harness.run_oracle(b, t, paged=paged)
    # history through the C ABI into the paged slab
    cache_h, scale_h = harness.new_slab(b, paged)
    cache, scale = harness.to_dev(cache_h), harness.to_dev(scale_h)
    hk, hv = harness.to_dev(t["hist_key"]), harness.to_dev(t["hist_value"])
    hs, z, tab = harness.to_dev(b.histstarts), harness.to_dev(np.zeros(b.batch, np.int64)), harness.to_dev(paged.table)
    w = harness.fill_write_args(cabi.KvWriteArgs(), b, hk, hv, hs, z, tab, cache, scale, ptr=harness.dev_ptr, paged=paged)
    harness.pkg.check(hiplib.pplhip_kv_quantize_write(C.byref(w), None), "history")
    torch.cuda.synchronize()
    s = Session(eng, ow.mhca_model(8, 2, 128, 1, 0, extra_attrs={"cache_mode": 1, "page_size": 128}))
    s.set_device_tensor(0, harness.to_dev(t["query"]))
    s.set_device_tensor(1, harness.to_dev(t["current_key"]))
    s.set_device_tensor(2, harness.to_dev(t["current_value"]))
    s.set_table(3, b.seqstarts)
    s.set_table(4, b.kvstarts)
    s.set_table(5, paged.table)
    s.set_table(6, b.start_pos)
    for i, v in zip(range(7, 10), (b.decoding_batches, b.max_seqlen, b.max_kvlen)):
        s.set_host_scalar(i, v)
    s.set_device_tensor(10, cache)
    s.set_device_tensor(11, scale)
    assert eng.pplnn_hip_runtime_run(s.rt) == 0, eng.pplnn_hip_last_error()
    harness.assert_attn_close(s.output(0, np.float16), ref["output_f64"])
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), ref["cache"])
    s.close()


def test_debug_dumps_and_step_replay(hiplib, tmp_path):
    """ENGINE_CONF_TENSOR_DEBUG / ENGINE_CONF_DEBUG_DATA_DIR dump every kernel's outputs as
    <dir>/pplnn_llm_hip_dbg_tensor-<name>-<dims>-<dtype>.dat; a step is replayed from files named
    <name>-<dims>-<dtype>.dat and its outputs saved as pplnn_output-<name>.dat (conventions of tools/pplnn_llm.cc)."""
    import torch
    eng = harness.pkg.load_engine_library()
    b = workloads.Batch(8, 2, 128, [1, 1, 30], [40, 7, 0], 2, name="replay")
    t = workloads.make_tensors(b, seed=71)
    cache, scale = _prepare_slab(b, t, hiplib)
    torch.cuda.synchronize()
    host = dict(query=t["query"], current_key=t["current_key"], current_value=t["current_value"],
                seqstarts=b.seqstarts, kvstarts=b.kvstarts, cachestarts=b.cachestarts, start_pos=b.start_pos,
                decoding_batches=np.array(b.decoding_batches, np.int64), max_seqlen=np.array(b.max_seqlen, np.int64),
                max_kvlen=np.array(b.max_kvlen, np.int64), cache=cache.cpu().numpy(),
                scale=scale.cpu().view(torch.int16).numpy().view(np.float16))
    dt = {np.dtype(np.float16): "fp16", np.dtype(np.int64): "int64", np.dtype(np.int8): "int8"}
    files = []
    for name in ow.MHCA_INPUTS:
        a = np.ascontiguousarray(host[name])
        dims = "scalar" if a.ndim == 0 else "_".join(str(d) for d in a.shape)
        f = tmp_path / f"step0_{name}-{dims}-{dt[a.dtype]}.dat"
        a.tofile(f)
        files.append(str(f))
    dbg = tmp_path / "dbg"
    dbg.mkdir()
    s = Session(eng, ow.rope_mhca_model(8, 2, 128, 1, 0, 10000.0))
    # options are read by kernels at run time from the engine's configuration
    assert eng.pplnn_hip_engine_configure_u32(s.engine, 2, 1) == 0
    assert eng.pplnn_hip_engine_configure_str(s.engine, 3, str(dbg).encode()) == 0
    for i in (7, 8, 9):
        eng.pplnn_hip_tensor_use_host_device(s.input(i))
    assert eng.pplnn_hip_runtime_set_inputs_from_files(s.rt, ",".join(files).encode()) == 0, eng.pplnn_hip_last_error()
    assert eng.pplnn_hip_runtime_run(s.rt) == 0, eng.pplnn_hip_last_error()
    out = s.output(0, np.float16)
    S = b.total_new_tokens
    names = sorted(p.name for p in dbg.iterdir())
    assert names == [f"pplnn_llm_hip_dbg_tensor-attn_output-{S}_8_128-fp16.dat",
                     f"pplnn_llm_hip_dbg_tensor-rotated_key-{S}_2_128-fp16.dat",
                     f"pplnn_llm_hip_dbg_tensor-rotated_query-{S}_8_128-fp16.dat"]
    dumped = np.fromfile(dbg / names[0], np.float16).reshape(S, 8, 128)
    assert np.array_equal(dumped.view(np.uint16), out.view(np.uint16))
    assert eng.pplnn_hip_runtime_save_outputs(s.rt, str(tmp_path).encode()) == 0
    saved = np.fromfile(tmp_path / "pplnn_output-attn_output.dat", np.float16).reshape(S, 8, 128)
    assert np.array_equal(saved.view(np.uint16), out.view(np.uint16))
    # the replayed step equals the same step driven through tensors (RoPE, then attention, against the oracle)
    import oracle
    rq, rk = _rope_on_oracle(oracle.lib(), t["query"], t["current_key"], b, 10000.0)
    ref = harness.run_oracle(b, dict(t, query=rq, current_key=rk))
    harness.assert_attn_close(out, ref["output_f64"], abs_tol=3e-3)
    # error conventions of the loader
    assert eng.pplnn_hip_runtime_set_inputs_from_files(s.rt, files[0].encode()) == cabi.RC_INVALID_VALUE  # count
    bad = list(files)
    bad[0] = str(tmp_path / "query.dat")
    assert eng.pplnn_hip_runtime_set_inputs_from_files(s.rt, ",".join(bad).encode()) == cabi.RC_INVALID_VALUE  # name
    s.close()


def test_engine_debug_options_check_tables_and_sync(hiplib):
    """ENGINE_CONF_DEBUG_CHECK_TABLES (1007): a bad table entry fails the op with RC_INVALID_VALUE before any attention
    kernel is launched (the check reads the tables only, so nothing faults), good tables run as usual; with
    ENGINE_CONF_DEBUG_SYNC_AFTER_OP (1008) every op is followed by a wait for the stream. The slab is poisoned with a
    pattern first: a refused call must leave every byte of it as it was."""
    import torch
    eng = harness.pkg.load_engine_library()
    eng.pplnn_hip_set_log_level(4)
    b = workloads.Batch(8, 2, 128, [1, 1, 70], [300, 9, 0], 2, slack_tokens=1, name="engine_debug")
    t = workloads.make_tensors(b, seed=15)
    ref = harness.run_oracle(b, t)
    cache, scale = _prepare_slab(b, t, hiplib)
    before = cache.clone()

    def run(tables, configure):
        s = Session(eng, ow.mhca_model(8, 2, 128, 1, 0), configure=configure)
        for i, name in enumerate(("query", "current_key", "current_value")):
            s.set_device_tensor(i, harness.to_dev(t[name]))
        for i, tab in enumerate(tables):
            s.set_table(3 + i, tab)
        for i, v in enumerate((b.decoding_batches, b.max_seqlen, b.max_kvlen)):
            s.set_host_scalar(7 + i, v)
        s.set_device_tensor(10, cache)
        s.set_device_tensor(11, scale)
        rc = eng.pplnn_hip_runtime_run(s.rt)
        out = s.output(0, np.float16) if rc == 0 else None
        s.close()
        return rc, out

    good = (b.seqstarts, b.kvstarts, b.cachestarts, b.start_pos)
    past_the_slab = b.cachestarts.copy()
    past_the_slab[2] = b.max_tokens - 3  # the prompt's 70 tokens would run past the end of the cache tensor
    wrong_kvlen = b.start_pos.copy()
    wrong_kvlen[0] = 299
    for name, tables in (("slab range", (b.seqstarts, b.kvstarts, past_the_slab, b.start_pos)),
                         ("kvlen", (b.seqstarts, b.kvstarts, b.cachestarts, wrong_kvlen))):
        print(f"case engine check_tables: {name}", flush=True)
        rc, _ = run(tables, [(1007, 1), (1008, 1)])
        assert rc == cabi.RC_INVALID_VALUE
        assert b"inconsistent tables" in eng.pplnn_hip_last_error()
        torch.cuda.synchronize()
        assert torch.equal(cache, before), "a refused call wrote to the slab"
    rc, out = run(good, [(1007, 1), (1008, 1)])
    assert rc == 0, eng.pplnn_hip_last_error()
    harness.assert_attn_close(out, ref["output_f64"])
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), ref["cache"])


def test_engine_rejects_masks_it_cannot_index(hiplib):
    """attn_mask is indexed unchecked by the kernels: the engine refuses an fp32 mask, one with fewer rows than query
    tokens, and one with fewer columns than the longest sequence has keys."""
    eng = harness.pkg.load_engine_library()
    eng.pplnn_hip_set_log_level(4)
    import torch
    b = workloads.Batch(8, 2, 64, [1, 40], [90, 0], 1, name="engine_mask_checks")
    t = workloads.make_tensors(b, seed=16)
    cache, scale = _prepare_slab(b, t, hiplib)
    S, K = b.total_new_tokens, int(b.kvstarts[-1])

    def run(mask):
        s = Session(eng, ow.mhca_model(8, 2, 64, 1, 0, mask_rank=2))
        for i, name in enumerate(("query", "current_key", "current_value")):
            s.set_device_tensor(i, harness.to_dev(t[name]))
        for i, tab in enumerate((b.seqstarts, b.kvstarts, b.cachestarts, b.start_pos)):
            s.set_table(3 + i, tab)
        for i, v in enumerate((b.decoding_batches, b.max_seqlen, b.max_kvlen)):
            s.set_host_scalar(7 + i, v)
        s.set_device_tensor(10, cache)
        s.set_device_tensor(11, scale)
        s.set_device_tensor(12, mask)
        rc = eng.pplnn_hip_runtime_run(s.rt)
        s.close()
        return rc

    f16 = dict(dtype=torch.float16, device="cuda")
    assert run(torch.zeros((S, (K + 7) // 8 * 8), **f16)) == 0, eng.pplnn_hip_last_error()
    assert run(torch.zeros((S - 1, (K + 7) // 8 * 8), **f16)) == cabi.RC_INVALID_VALUE
    assert run(torch.zeros((S, b.max_kvlen - 1), **f16)) == cabi.RC_INVALID_VALUE
