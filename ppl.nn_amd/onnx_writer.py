"""Minimal ONNX ModelProto writer (protobuf wire format by hand; no onnx / protobuf package needed).
Field numbers follow onnx.proto: ModelProto{ir_version=1, graph=7, opset_import=8}, GraphProto{node=1, name=2,
input=11, output=12}, NodeProto{input=1, output=2, name=3, op_type=4, attribute=5, domain=7},
AttributeProto{name=1, f=2, i=3, s=4, ints=8, type=20}, ValueInfoProto{name=1, type=2}, GraphProto.initializer=5 with
TensorProto{dims=1, data_type=2, name=8, raw_data=9}."""
import struct

FLOAT, INT8, INT64, FLOAT16 = 1, 3, 7, 10


def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        out.append(b | (0x80 if v else 0))
        if not v:
            return bytes(out)


def _key(field, wt):
    return _varint((field << 3) | wt)


def _ld(field, payload):
    return _key(field, 2) + _varint(len(payload)) + payload


def _str(field, s):
    return _ld(field, s.encode())


def _int(field, v):
    return _key(field, 0) + _varint(v)


def attr_int(name, v):
    return _str(1, name) + _int(3, v) + _int(20, 2)


def attr_float(name, v):
    return _str(1, name) + _key(2, 5) + struct.pack("<f", v) + _int(20, 1)


def attr_ints(name, vs):
    return _str(1, name) + b"".join(_int(8, v) for v in vs) + _int(20, 7)


def initializer(name, elem_type, dims, raw):
    """TensorProto with raw little-endian data."""
    return b"".join(_int(1, d) for d in dims) + _int(2, elem_type) + _str(8, name) + _ld(9, bytes(raw))


def value_info(name, elem_type, dims):
    """dims: ints, or strings for symbolic dimensions."""
    shape = b"".join(_ld(1, _int(1, d) if isinstance(d, int) else _str(2, d)) for d in dims)
    tensor = _int(1, elem_type) + _ld(2, shape)
    return _str(1, name) + _ld(2, _ld(1, tensor))


def node(op_type, inputs, outputs, name="", domain="", attrs=()):
    b = b"".join(_str(1, i) for i in inputs) + b"".join(_str(2, o) for o in outputs)
    if name:
        b += _str(3, name)
    b += _str(4, op_type) + b"".join(_ld(5, a) for a in attrs)
    if domain:
        b += _str(7, domain)
    return b


def model(nodes, inputs, outputs, opsets, graph_name="g", initializers=()):
    graph = b"".join(_ld(1, n) for n in nodes) + _str(2, graph_name) + b"".join(_ld(5, t) for t in initializers) + \
        b"".join(_ld(11, i) for i in inputs) + b"".join(_ld(12, o) for o in outputs)
    m = _int(1, 8) + _ld(7, graph)
    for domain, version in opsets:
        m += _ld(8, (_str(1, domain) if domain else b"") + _int(2, version))
    return m


MHCA_INPUTS = ["query", "current_key", "current_value", "seqstarts", "kvstarts", "cachestarts", "start_pos",
               "decoding_batches", "max_seqlen", "max_kvlen", "cache", "scale"]


def mhca_model(num_heads, num_kv_heads, head_dim, num_layer, layer_idx, extra_attrs=(), drop_attrs=(), with_scale=True,
               domain="opmx.dynamic_batching", opsets=None, mask_rank=0):
    """mask_rank 2 or 3 appends the optional 13th input `attn_mask` ([tokens, keys] or [heads, tokens, keys])."""
    attrs = dict(num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, num_layer=num_layer,
                 layer_idx=layer_idx, quant_bit=8, quant_group=8)
    attrs.update(dict(extra_attrs))
    for k in drop_attrs:
        attrs.pop(k)
    names = list(MHCA_INPUTS) if with_scale else MHCA_INPUTS[:-1]
    if mask_rank:
        names.append("attn_mask")
    n = node("MultiHeadCacheAttention", names, ["attn_output"], name="attn", domain=domain,
             attrs=[attr_int(k, v) for k, v in attrs.items()])
    types = {"query": FLOAT16, "current_key": FLOAT16, "current_value": FLOAT16, "cache": INT8, "scale": FLOAT16,
             "attn_mask": FLOAT16}
    ranks = {"query": 3, "current_key": 3, "current_value": 3, "seqstarts": 1, "kvstarts": 1, "cachestarts": 1,
             "start_pos": 1, "decoding_batches": 0, "max_seqlen": 0, "max_kvlen": 0, "cache": 5, "scale": 5,
             "attn_mask": mask_rank}
    ins = [value_info(x, types.get(x, INT64), ["d%d" % i for i in range(ranks[x])]) for x in names]
    outs = [value_info("attn_output", FLOAT16, ["s", "h", "d"])]
    return model([n], ins, outs, opsets if opsets is not None else [("", 11), (domain, 1)])


KVC_INPUTS = ["current_key", "current_value", "seqstarts", "kvstarts", "cachestarts", "start_pos", "max_seqlen",
              "max_kvlen", "cache", "scale"]


def kv_cache_model(num_layer, layer_idx, extra_attrs=()):
    attrs = dict(num_layer=num_layer, layer_idx=layer_idx, quant_bit=8, quant_group=8)
    attrs.update(dict(extra_attrs))
    n = node("KeyValueCache", KVC_INPUTS, ["key", "value"], name="kvcache", domain="opmx.dynamic_batching",
             attrs=[attr_int(k, v) for k, v in attrs.items()])
    types = {"current_key": FLOAT16, "current_value": FLOAT16, "cache": INT8, "scale": FLOAT16}
    ranks = {"current_key": 3, "current_value": 3, "seqstarts": 1, "kvstarts": 1, "cachestarts": 1, "start_pos": 1,
             "max_seqlen": 0, "max_kvlen": 0, "cache": 5, "scale": 5}
    ins = [value_info(x, types.get(x, INT64), ["d%d" % i for i in range(ranks[x])]) for x in KVC_INPUTS]
    outs = [value_info("key", FLOAT16, ["t", "h", "d"]), value_info("value", FLOAT16, ["t", "h", "d"])]
    return model([n], ins, outs, [("", 11), ("opmx.dynamic_batching", 1)])


def attr_string(name, v):
    return _str(1, name) + _ld(4, v.encode()) + _int(20, 3)


DB = "opmx.dynamic_batching"
_TYPES = {"query": FLOAT16, "key": FLOAT16, "value": FLOAT16, "current_key": FLOAT16, "current_value": FLOAT16,
          "cache": INT8, "scale": FLOAT16}
_RANKS = {"query": 3, "key": 3, "value": 3, "current_key": 3, "current_value": 3, "seqstarts": 1, "kvstarts": 1,
          "cachestarts": 1, "start_pos": 1, "decoding_batches": 0, "max_seqlen": 0, "max_kvlen": 0, "cache": 5,
          "scale": 5, "sequence": 1}


def _inputs(names):
    return [value_info(x, _TYPES.get(x, INT64), ["d%d" % i for i in range(_RANKS[x])]) for x in names]


def rope_attrs(theta=10000.0, drop_theta=False, scaling_type=None, **ints):
    attrs = [] if drop_theta else [attr_float("theta", theta)]
    attrs += [attr_float(k, v) if isinstance(v, float) else attr_int(k, v) for k, v in ints.items()]
    if scaling_type is not None:
        attrs.append(attr_string("scaling_type", scaling_type))
    return attrs


def rope_model(attrs):
    names = ["query", "key", "seqstarts", "start_pos", "max_seqlen"]
    n = node("RotaryPositionEmbedding", names, ["rotated_query", "rotated_key"], name="rope", domain=DB, attrs=attrs)
    outs = [value_info("rotated_query", FLOAT16, ["s", "h", "d"]), value_info("rotated_key", FLOAT16, ["s", "h", "d"])]
    return model([n], _inputs(names), outs, [("", 11), (DB, 1)])


ROPE_MHCA_INPUTS = ["query", "key", "current_value", "seqstarts", "kvstarts", "cachestarts", "start_pos",
                    "decoding_batches", "max_seqlen", "max_kvlen", "cache", "scale"]


def rope_mhca_model(num_heads, num_kv_heads, head_dim, num_layer, layer_idx, theta):
    """RotaryPositionEmbedding feeding MultiHeadCacheAttention: rotated_query / rotated_key are intermediate tensors."""
    rope = node("RotaryPositionEmbedding", ["query", "key", "seqstarts", "start_pos", "max_seqlen"],
                ["rotated_query", "rotated_key"], name="rope", domain=DB, attrs=rope_attrs(theta))
    attrs = dict(num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, num_layer=num_layer,
                 layer_idx=layer_idx, quant_bit=8, quant_group=8)
    attn = node("MultiHeadCacheAttention",
                ["rotated_query", "rotated_key"] + ROPE_MHCA_INPUTS[2:], ["attn_output"], name="attn", domain=DB,
                attrs=[attr_int(k, v) for k, v in attrs.items()])
    outs = [value_info("attn_output", FLOAT16, ["s", "h", "d"])]
    return model([rope, attn], _inputs(ROPE_MHCA_INPUTS), outs, [("", 11), (DB, 1)])


KVC_MHA_INPUTS = ["query", "current_key", "current_value", "seqstarts", "kvstarts", "cachestarts", "start_pos",
                  "decoding_batches", "max_seqlen", "max_kvlen", "cache", "scale"]


def kv_cache_mha_model(num_heads, num_kv_heads, head_dim, num_layer, layer_idx, mha_extra=()):
    """KeyValueCache feeding MultiHeadAttention: the two-op spelling of MultiHeadCacheAttention."""
    kvc = node("KeyValueCache", KVC_INPUTS, ["key", "value"], name="kvcache", domain=DB,
               attrs=[attr_int(k, v) for k, v in dict(num_layer=num_layer, layer_idx=layer_idx, quant_bit=8,
                                                      quant_group=8).items()])
    attrs = dict(num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim)
    attrs.update(dict(mha_extra))
    mha = node("MultiHeadAttention", ["query", "key", "value", "seqstarts", "kvstarts", "decoding_batches", "max_seqlen",
                                      "max_kvlen"], ["attn_output"], name="mha", domain=DB,
               attrs=[attr_int(k, v) for k, v in attrs.items()])
    outs = [value_info("attn_output", FLOAT16, ["s", "h", "d"])]
    return model([kvc, mha], _inputs(KVC_MHA_INPUTS), outs, [("", 11), (DB, 1)])


def mha_model(attrs):
    names = ["query", "key", "value", "seqstarts", "kvstarts", "decoding_batches", "max_seqlen", "max_kvlen"]
    n = node("MultiHeadAttention", names, ["attn_output"], name="mha", domain=DB,
             attrs=[attr_int(k, v) for k, v in attrs.items()])
    return model([n], _inputs(names), [value_info("attn_output", FLOAT16, ["s", "h", "d"])], [("", 11), (DB, 1)])


def position_index_model():
    names = ["sequence", "seqstarts", "start_pos", "max_seqlen"]
    n = node("PositionIndex", names, ["position_idx"], name="posidx", domain=DB)
    return model([n], _inputs(names), [value_info("position_idx", INT64, ["s"])], [("", 11), (DB, 1)])


def attention_fp32_model(head_dim, rank=3, opset=11):
    """The attention subgraph the x86 engine runs per sequence, fp32: Transpose(K) -> MatMul(Q, K^T) -> Mul by the
    initializer 1/sqrt(head_dim) -> Add of an additive mask -> Softmax over the keys -> MatMul with V.
    rank 3: query / key / value [heads, L, head_dim]; rank 4: [kv_heads, heads per kv head | 1, L, head_dim] (MatMul's
    batch broadcasting shares a kv head among its query heads). mask [Lq, Lk], -inf where a query must not look."""
    lead = ["h"] if rank == 3 else ["g", "r"]
    perm = list(range(rank - 2)) + [rank - 1, rank - 2]
    nodes = [
        node("Transpose", ["key"], ["key_t"], name="transpose_k", attrs=[attr_ints("perm", perm)]),
        node("MatMul", ["query", "key_t"], ["scores"], name="qk"),
        node("Mul", ["scores", "scale"], ["scaled"], name="scale_scores"),
        node("Add", ["scaled", "mask"], ["masked"], name="add_mask"),
        node("Softmax", ["masked"], ["probs"], name="softmax", attrs=[attr_int("axis", -1)]),
        node("MatMul", ["probs", "value"], ["attn_output"], name="pv"),
    ]
    ins = [value_info("query", FLOAT, lead + ["lq", head_dim]), value_info("key", FLOAT, lead + ["lk", head_dim]),
           value_info("value", FLOAT, lead + ["lk", head_dim]), value_info("mask", FLOAT, ["lq", "lk"])]
    outs = [value_info("attn_output", FLOAT, lead + ["lq", head_dim])]
    scale = initializer("scale", FLOAT, [], struct.pack("<f", 1.0 / (head_dim ** 0.5)))
    return model(nodes, ins, outs, [("", opset)], graph_name="attention_fp32", initializers=[scale])
