"""PMX op-parameter blobs (FlatBuffers `OpParam`, llm_cuda_op_params.fbs) of the attention-path ops.

No FlatBuffers package or flatc is available offline, so the engine's reader and writer are checked against a second,
independent implementation written here from the format's specification: `fb_decode` walks any valid buffer, and
`fb_encode_builder_style` lays a buffer out back to front (member table before the root table, vtables directly before
their tables, root offset at the start). On top of that, the committed blobs under tests/golden/ hold the exact bytes
the reference's serialisers produce for three parameter sets, derived field by field from the schema, the generated
Create* call order the reference checks in, and FlatBufferBuilder's published algorithm (tests/golden/README.md); the
engine's writer must reproduce them byte for byte. They were not produced by running flatc or the reference, which is
why the row stays "parity unpinned" against the real tool."""
import ctypes as C
import struct

import pytest

import harness
from ppl_nn_amd import onnx_writer as ow
from harness import cabi

# union OpParamType tags and field lists (name, kind) in schema order: llm_cuda_op_params.fbs:14-23, 31-37, 60-67, 75-88
TAG = {"KeyValueCacheParam": 3, "MultiHeadAttentionParam": 5, "RotaryPositionEmbeddingParam": 8,
       "MultiHeadCacheAttentionParam": 10}
FIELDS = {
    "KeyValueCacheParam": [("num_layer", "i"), ("layer_idx", "i"), ("quant_bit", "i"), ("quant_group", "i"),
                           ("num_repeat", "i"), ("cache_mode", "i"), ("cache_layout", "i"), ("page_size", "i")],
    "MultiHeadAttentionParam": [("num_heads", "i"), ("num_kv_heads", "i"), ("head_dim", "i"), ("is_causal", "?"),
                                ("is_alibi", "?")],
    "RotaryPositionEmbeddingParam": [("bypass_key", "i"), ("rotary_dim", "i"), ("theta", "f"),
                                     ("max_position_embeddings", "i"), ("scaling_type", "I"), ("scaling_factor", "f")],
    "MultiHeadCacheAttentionParam": [("num_heads", "i"), ("num_kv_heads", "i"), ("head_dim", "i"), ("is_causal", "?"),
                                     ("is_alibi", "?"), ("num_layer", "i"), ("layer_idx", "i"), ("quant_bit", "i"),
                                     ("quant_group", "i"), ("cache_mode", "i"), ("cache_layout", "i"), ("page_size", "i")],
}
SIZE = {"i": 4, "I": 4, "f": 4, "?": 1}


def _table(buf, pos):
    (so,) = struct.unpack_from("<i", buf, pos)
    vt = pos - so
    vsize, _tsize = struct.unpack_from("<HH", buf, vt)

    def field(i, kind, default):
        slot = 4 + 2 * i
        if slot + 2 > vsize:
            return default
        (off,) = struct.unpack_from("<H", buf, vt + slot)
        return struct.unpack_from("<" + kind, buf, pos + off)[0] if off else default
    return field


def fb_decode(buf):
    (root,) = struct.unpack_from("<I", buf, 0)
    f = _table(buf, root)
    tag = f(0, "B", 0)
    (so,) = struct.unpack_from("<i", buf, root)
    vt = root - so
    (off,) = struct.unpack_from("<H", buf, vt + 4 + 2)
    vpos = root + off
    member = vpos + struct.unpack_from("<I", buf, vpos)[0]
    name = {v: k for k, v in TAG.items()}[tag]
    g = _table(buf, member)
    return name, {n: g(i, k, False if k == "?" else 0) for i, (n, k) in enumerate(FIELDS[name])}


def fb_encode_builder_style(name, values, force_defaults=False):
    """Back-to-front layout like the official builders: build the tail first, then prepend."""
    fields = FIELDS[name]
    # member table body: fields sorted by size (largest first), as builders add them in call order after alignment
    body = bytearray(4)
    offs = []
    for n, k in fields:
        v = values.get(n, 0)
        if not force_defaults and (v == 0 or v is False):
            offs.append(0)
            continue
        while len(body) % SIZE[k]:
            body.append(0)
        offs.append(len(body))
        body += struct.pack("<" + k, v)
    while len(body) % 4:
        body.append(0)
    vt = struct.pack("<HH", 4 + 2 * len(fields), len(body)) + b"".join(struct.pack("<H", o) for o in offs)
    if len(vt) % 4:
        vt += b"\x00\x00"
    # tail = [member vtable][member table]; the root table and its vtable go in front of it
    root_vt = struct.pack("<HHHH", 8, 12, 8, 4)
    root_body = bytearray(12)
    # buffer: [root off][pad][root vtable][root table][member vtable][member table]
    head = 4 + 4  # root offset + padding word (builders align the whole buffer; any valid padding is allowed)
    root_vt_pos = head
    root_pos = root_vt_pos + len(root_vt)
    member_vt_pos = root_pos + len(root_body)
    member_pos = member_vt_pos + len(vt)
    struct.pack_into("<i", root_body, 0, root_pos - root_vt_pos)
    struct.pack_into("<I", root_body, 4, member_pos - (root_pos + 4))
    struct.pack_into("<B", root_body, 8, TAG[name])
    struct.pack_into("<i", body, 0, member_pos - member_vt_pos)
    return struct.pack("<II", root_pos, 0) + root_vt + bytes(root_body) + vt + bytes(body)


@pytest.fixture(scope="module")
def eng():
    L = harness.pkg.load_engine_library()
    L.pplnn_hip_set_log_level(4)
    return L


def _built(eng, model):
    e = eng.pplnn_hip_engine_create(0, 1)
    b = eng.pplnn_hip_builder_create()
    assert eng.pplnn_hip_builder_load_model(b, model, len(model)) == 0
    assert eng.pplnn_hip_builder_set_engine(b, e) == 0
    assert eng.pplnn_hip_builder_preprocess(b) == 0
    return e, b


def _serialize(eng, b, node):
    buf, n = C.create_string_buffer(512), C.c_uint64()
    assert eng.pplnn_hip_builder_serialize_op(b, node, buf, 512, C.byref(n)) == 0, eng.pplnn_hip_last_error()
    return buf.raw[:n.value]


CASES = [
    ("attn", "MultiHeadCacheAttentionParam",
     lambda: ow.mhca_model(32, 8, 128, 80, 79, extra_attrs={"cache_mode": 1, "cache_layout": 3, "page_size": 256}),
     dict(num_heads=32, num_kv_heads=8, head_dim=128, is_causal=True, is_alibi=False, num_layer=80, layer_idx=79,
          quant_bit=8, quant_group=8, cache_mode=1, cache_layout=3, page_size=256)),
    ("attn", "MultiHeadCacheAttentionParam",  # defaults: num_kv_heads = num_heads, layer 0, is_causal off
     lambda: ow.mhca_model(16, 16, 128, 1, 0, extra_attrs={"is_causal": 0}, drop_attrs=["quant_bit"]),
     dict(num_heads=16, num_kv_heads=16, head_dim=128, is_causal=False, is_alibi=False, num_layer=1, layer_idx=0,
          quant_bit=0, quant_group=8, cache_mode=0, cache_layout=0, page_size=128)),
    ("kvcache", "KeyValueCacheParam", lambda: ow.kv_cache_model(4, 3),
     dict(num_layer=4, layer_idx=3, quant_bit=8, quant_group=8, num_repeat=1, cache_mode=0, cache_layout=0,
          page_size=128)),
    ("mha", "MultiHeadAttentionParam", lambda: ow.mha_model(dict(num_heads=32, head_dim=128, num_kv_heads=8)),
     dict(num_heads=32, num_kv_heads=8, head_dim=128, is_causal=True, is_alibi=False)),
    ("rope", "RotaryPositionEmbeddingParam",
     lambda: ow.rope_model(ow.rope_attrs(500000.0, rotary_dim=64, bypass_key=1, scaling_type="dynamic",
                                         scaling_factor=2.5, max_position_embeddings=8192)),
     dict(bypass_key=1, rotary_dim=64, theta=500000.0, max_position_embeddings=8192, scaling_type=2,
          scaling_factor=2.5)),
]


@pytest.mark.parametrize("node,table,model,want", CASES)
def test_serialized_params_read_back_by_an_independent_reader(eng, node, table, model, want):
    e, b = _built(eng, model())
    blob = _serialize(eng, b, node.encode())
    name, got = fb_decode(blob)
    assert name == table and got == want
    assert struct.unpack_from("<I", blob, 0)[0] % 4 == 0  # tables are 4-byte aligned
    eng.pplnn_hip_builder_destroy(b)
    eng.pplnn_hip_engine_destroy(e)


@pytest.mark.parametrize("node,table,model,want", CASES)
@pytest.mark.parametrize("force_defaults", [False, True])
def test_builder_style_buffers_deserialize_into_the_op(eng, node, table, model, want, force_defaults):
    # start from an op with OTHER parameters, load a blob laid out like the official builders', serialise again
    other = {"attn": lambda: ow.mhca_model(4, 4, 128, 2, 1), "kvcache": lambda: ow.kv_cache_model(9, 1),
             "mha": lambda: ow.mha_model(dict(num_heads=4, head_dim=128)),
             "rope": lambda: ow.rope_model(ow.rope_attrs(10000.0))}[node]
    e, b = _built(eng, other())
    blob = fb_encode_builder_style(table, want, force_defaults=force_defaults)
    assert fb_decode(blob) == (table, want)  # the test's own two halves agree
    assert eng.pplnn_hip_builder_deserialize_op(b, node.encode(), blob, len(blob)) == 0, eng.pplnn_hip_last_error()
    assert fb_decode(_serialize(eng, b, node.encode())) == (table, want)
    eng.pplnn_hip_builder_destroy(b)
    eng.pplnn_hip_engine_destroy(e)


GOLDEN = [
    ("pmx_mhca_llama3_8b_layer5.bin", "attn", "MultiHeadCacheAttentionParam",
     lambda: ow.mhca_model(32, 8, 128, 32, 5, extra_attrs={"page_size": 128}),
     dict(num_heads=32, num_kv_heads=8, head_dim=128, is_causal=True, is_alibi=False, num_layer=32, layer_idx=5,
          quant_bit=8, quant_group=8, cache_mode=0, cache_layout=0, page_size=128)),
    ("pmx_kv_cache_layer3_of_32.bin", "kvcache", "KeyValueCacheParam", lambda: ow.kv_cache_model(32, 3),
     dict(num_layer=32, layer_idx=3, quant_bit=8, quant_group=8, num_repeat=1, cache_mode=0, cache_layout=0,
          page_size=128)),
]


@pytest.mark.parametrize("file,node,table,model,want", GOLDEN)
def test_writer_reproduces_the_golden_blobs_byte_for_byte(eng, file, node, table, model, want):
    import os
    with open(os.path.join(harness.ROOT, "tests", "golden", file), "rb") as f:
        golden = f.read()
    assert fb_decode(golden) == (table, want)  # the fixture itself says what its README says
    e, b = _built(eng, model())
    assert _serialize(eng, b, node.encode()) == golden
    # and it loads: start from other parameters, read the golden blob, write it again
    other = {"attn": lambda: ow.mhca_model(4, 4, 128, 2, 1), "kvcache": lambda: ow.kv_cache_model(9, 1)}[node]
    e2, b2 = _built(eng, other())
    assert eng.pplnn_hip_builder_deserialize_op(b2, node.encode(), golden, len(golden)) == 0
    assert _serialize(eng, b2, node.encode()) == golden
    for x, y in ((b, e), (b2, e2)):
        eng.pplnn_hip_builder_destroy(x)
        eng.pplnn_hip_engine_destroy(y)


def test_golden_blob_with_trailing_defaults_has_a_short_vtable(eng):
    """page_size 0 never leaves the ONNX parser (its default is 128), so this fixture is checked at the byte level
    only: absent trailing fields shorten the vtable instead of being stored as zero slots, and the reader returns the
    schema defaults for them."""
    import os
    with open(os.path.join(harness.ROOT, "tests", "golden", "pmx_mhca_trailing_defaults.bin"), "rb") as f:
        golden = f.read()
    name, got = fb_decode(golden)
    assert name == "MultiHeadCacheAttentionParam" and got["page_size"] == 0 and got["quant_group"] == 8
    (root,) = struct.unpack_from("<I", golden, 0)
    member = root + 8 + struct.unpack_from("<I", golden, root + 8)[0]
    (so,) = struct.unpack_from("<i", golden, member)
    assert struct.unpack_from("<H", golden, member - so)[0] == 4 + 2 * 9  # slots num_heads .. quant_group
    e, b = _built(eng, ow.mhca_model(4, 4, 128, 2, 1))
    assert eng.pplnn_hip_builder_deserialize_op(b, b"attn", golden, len(golden)) == 0
    assert _serialize(eng, b, b"attn") == golden
    eng.pplnn_hip_builder_destroy(b)
    eng.pplnn_hip_engine_destroy(e)


def test_golden_script_is_reproducible():
    import importlib.util
    import os
    path = os.path.join(harness.ROOT, "tests", "golden", "make_pmx_golden.py")
    spec = importlib.util.spec_from_file_location("make_pmx_golden", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    for name, blob in mod.CASES.items():
        with open(os.path.join(os.path.dirname(path), name), "rb") as f:
            assert f.read() == blob, name


def test_malformed_and_mismatched_blobs_are_rejected(eng):
    e, b = _built(eng, ow.mhca_model(8, 2, 128, 1, 0))
    good = _serialize(eng, b, b"attn")
    for bad in (b"", good[:3], good[:10], good[:-6], b"\xff" * 40):
        assert eng.pplnn_hip_builder_deserialize_op(b, b"attn", bad, len(bad)) == cabi.RC_INVALID_VALUE
    wrong_member = fb_encode_builder_style("KeyValueCacheParam", dict(num_layer=1))
    assert eng.pplnn_hip_builder_deserialize_op(b, b"attn", wrong_member, len(wrong_member)) == cabi.RC_INVALID_VALUE
    assert eng.pplnn_hip_builder_deserialize_op(b, b"nope", good, len(good)) == cabi.RC_NOT_FOUND
    assert eng.pplnn_hip_builder_deserialize_op(b, b"attn", good, len(good)) == 0
    eng.pplnn_hip_builder_destroy(b)
    eng.pplnn_hip_engine_destroy(e)


def test_op_without_parameters_writes_nothing(eng):
    e, b = _built(eng, ow.position_index_model())
    assert _serialize(eng, b, b"posidx") == b""  # position_index_op.cc:44-46
    eng.pplnn_hip_builder_destroy(b)
    eng.pplnn_hip_engine_destroy(e)
