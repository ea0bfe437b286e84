// ONNX model loading without libprotobuf: a hand-written reader of the protobuf wire format for exactly the fields the
// reference loader consumes (src/ppl/nn/models/onnx/model_parser.cc:52-96, graph_parser.cc:47-316, utils.h:129-142;
// field numbers from src/ppl/nn/models/onnx/proto/onnx.proto), plus the op-parameter parsers of
//   src/ppl/nn/models/onnx/parsers/opmx/parse_multi_head_cache_attention_param.cc:13-45
//   src/ppl/nn/models/onnx/parsers/opmx/parse_key_value_cache_param.cc:27-48
// registered like src/ppl/nn/models/onnx/param_parser_manager.cc:353-368.
#include <mutex>

#include "params.h"

using namespace ppl::common;

namespace ppl { namespace nn { namespace onnx {

namespace {

// ---- wire format
struct Reader final {
    const uint8_t* p;
    const uint8_t* end;
    bool ok = true;
    Reader(const void* b, uint64_t n) : p((const uint8_t*)b), end((const uint8_t*)b + n) {}
    bool Done() const { return p >= end || !ok; }
    uint64_t Varint() {
        uint64_t v = 0;
        for (int shift = 0; shift < 64; shift += 7) {
            if (p >= end) {
                ok = false;
                return 0;
            }
            const uint8_t b = *p++;
            v |= (uint64_t)(b & 0x7f) << shift;
            if (!(b & 0x80)) return v;
        }
        ok = false;
        return 0;
    }
    // returns field number, sets wire type; for length-delimited fields `sub` covers the payload
    uint32_t Next(uint32_t* wt, Reader* sub, uint64_t* scalar) {
        const uint64_t key = Varint();
        if (!ok) return 0;
        *wt = (uint32_t)(key & 7);
        switch (*wt) {
            case 0: *scalar = Varint(); break;
            case 1:
                if (end - p < 8) { ok = false; return 0; }
                memcpy(scalar, p, 8);
                p += 8;
                break;
            case 2: {
                const uint64_t n = Varint();
                if (!ok || (uint64_t)(end - p) < n) { ok = false; return 0; }
                *sub = Reader(p, n);
                p += n;
                break;
            }
            case 5: {
                if (end - p < 4) { ok = false; return 0; }
                uint32_t v;
                memcpy(&v, p, 4);
                *scalar = v;
                p += 4;
                break;
            }
            default: ok = false; return 0;
        }
        return (uint32_t)(key >> 3);
    }
    std::string Str() const { return std::string((const char*)p, end - p); }
};

struct PbAttr final {
    std::string name;
    int64_t i = 0;
    float f = 0;
    std::string s;
    std::vector<int64_t> ints;
    bool has_i = false, has_f = false;
};

struct PbNode final {
    std::vector<std::string> inputs, outputs;
    std::string name, op_type, domain;
    std::vector<PbAttr> attrs;
};

bool ParseAttr(Reader r, PbAttr* a) {
    while (!r.Done()) {
        uint32_t wt; Reader sub(nullptr, 0); uint64_t v = 0;
        const uint32_t f = r.Next(&wt, &sub, &v);
        if (!r.ok) return false;
        if (f == 1 && wt == 2) a->name = sub.Str();
        else if (f == 2 && wt == 5) { uint32_t u = (uint32_t)v; memcpy(&a->f, &u, 4); a->has_f = true; }
        else if (f == 3 && wt == 0) { a->i = (int64_t)v; a->has_i = true; }
        else if (f == 4 && wt == 2) a->s = sub.Str();
        else if (f == 8 && wt == 2) { while (!sub.Done()) a->ints.push_back((int64_t)sub.Varint()); } // packed ints
        else if (f == 8 && wt == 0) a->ints.push_back((int64_t)v);
    }
    return r.ok;
}

bool ParseNode(Reader r, PbNode* n) {
    while (!r.Done()) {
        uint32_t wt; Reader sub(nullptr, 0); uint64_t v = 0;
        const uint32_t f = r.Next(&wt, &sub, &v);
        if (!r.ok) return false;
        if (wt != 2) continue;
        switch (f) {
            case 1: n->inputs.push_back(sub.Str()); break;
            case 2: n->outputs.push_back(sub.Str()); break;
            case 3: n->name = sub.Str(); break;
            case 4: n->op_type = sub.Str(); break;
            case 5: { PbAttr a; if (!ParseAttr(sub, &a)) return false; n->attrs.push_back(a); break; }
            case 7: n->domain = sub.Str(); break;
            default: break;
        }
    }
    return r.ok;
}

datatype_t ConvertOnnxDataType(int64_t t) { // src/ppl/nn/models/onnx/utils.cc:36-63
    switch (t) {
        case 1: return DATATYPE_FLOAT32;
        case 2: return DATATYPE_UINT8;
        case 3: return DATATYPE_INT8;
        case 4: return DATATYPE_UINT16;
        case 5: return DATATYPE_INT16;
        case 6: return DATATYPE_INT32;
        case 7: return DATATYPE_INT64;
        case 9: return DATATYPE_BOOL;
        case 10: return DATATYPE_FLOAT16;
        case 11: return DATATYPE_FLOAT64;
        case 12: return DATATYPE_UINT32;
        case 13: return DATATYPE_UINT64;
        case 16: return DATATYPE_BFLOAT16;
        default: return DATATYPE_UNKNOWN;
    }
}

// ValueInfoProto{name=1, type=2{tensor_type=1{elem_type=1, shape=2{dim=1{dim_value=1|dim_param=2}}}}}
bool ParseValueInfo(Reader r, std::string* name, ir::Shape* shape) {
    while (!r.Done()) {
        uint32_t wt; Reader sub(nullptr, 0); uint64_t v = 0;
        const uint32_t f = r.Next(&wt, &sub, &v);
        if (!r.ok) return false;
        if (f == 1 && wt == 2) *name = sub.Str();
        else if (f == 2 && wt == 2) {
            Reader type = sub;
            while (!type.Done()) {
                uint32_t wt2; Reader tt(nullptr, 0); uint64_t v2 = 0;
                const uint32_t f2 = type.Next(&wt2, &tt, &v2);
                if (!type.ok) return false;
                if (f2 != 1 || wt2 != 2) continue; // tensor_type only
                while (!tt.Done()) {
                    uint32_t wt3; Reader sh(nullptr, 0); uint64_t v3 = 0;
                    const uint32_t f3 = tt.Next(&wt3, &sh, &v3);
                    if (!tt.ok) return false;
                    if (f3 == 1 && wt3 == 0) shape->data_type = ConvertOnnxDataType((int64_t)v3);
                    else if (f3 == 2 && wt3 == 2) {
                        while (!sh.Done()) {
                            uint32_t wt4; Reader dim(nullptr, 0); uint64_t v4 = 0;
                            const uint32_t f4 = sh.Next(&wt4, &dim, &v4);
                            if (!sh.ok) return false;
                            if (f4 != 1 || wt4 != 2) continue;
                            int64_t dv = INVALID_DIM_VALUE; // symbolic unless dim_value is present
                            while (!dim.Done()) {
                                uint32_t wt5; Reader x(nullptr, 0); uint64_t v5 = 0;
                                const uint32_t f5 = dim.Next(&wt5, &x, &v5);
                                if (!dim.ok) return false;
                                if (f5 == 1 && wt5 == 0) dv = (int64_t)v5;
                            }
                            shape->dims.push_back(dv);
                        }
                    }
                }
            }
        }
    }
    return r.ok;
}

// TensorProto{dims=1, data_type=2, name=8, raw_data=9, float_data=4, int32_data=5, int64_data=7}
bool ParseInitializer(Reader r, std::string* name, ir::Shape* shape, ir::Constant* c) {
    std::vector<float> floats;
    std::vector<int64_t> int64s;
    std::vector<int32_t> int32s;
    bool has_raw = false;
    auto packed_or_single = [](uint32_t wt, Reader sub, uint64_t v, auto&& push) {
        if (wt == 2) {
            while (!sub.Done()) push(sub.Varint());
        } else {
            push(v);
        }
    };
    while (!r.Done()) {
        uint32_t wt; Reader sub(nullptr, 0); uint64_t v = 0;
        const uint32_t f = r.Next(&wt, &sub, &v);
        if (!r.ok) return false;
        switch (f) {
            case 1: packed_or_single(wt, sub, v, [&](uint64_t x) { shape->dims.push_back((int64_t)x); }); break;
            case 2: shape->data_type = ConvertOnnxDataType((int64_t)v); break;
            case 4:
                if (wt == 2) { floats.resize((sub.end - sub.p) / 4); memcpy(floats.data(), sub.p, floats.size() * 4); }
                else { uint32_t u = (uint32_t)v; float x; memcpy(&x, &u, 4); floats.push_back(x); }
                break;
            case 5: packed_or_single(wt, sub, v, [&](uint64_t x) { int32s.push_back((int32_t)x); }); break;
            case 7: packed_or_single(wt, sub, v, [&](uint64_t x) { int64s.push_back((int64_t)x); }); break;
            case 8: *name = sub.Str(); break;
            case 9: c->data = sub.Str(); has_raw = true; break;
            case 13: case 14: return false; // external data is not supported on this path
            default: break;
        }
    }
    if (!has_raw) {
        if (!floats.empty()) c->data.assign((const char*)floats.data(), floats.size() * 4);
        else if (!int64s.empty()) c->data.assign((const char*)int64s.data(), int64s.size() * 8);
        else if (!int32s.empty()) { // fp16 / int8 / bool may arrive widened in int32_data (models/onnx/utils.cc:148-314)
            const uint32_t sz = GetSizeOfDataType(shape->data_type);
            for (auto x : int32s) c->data.append((const char*)&x, sz ? (sz < 4 ? sz : 4) : 4);
        }
    }
    return r.ok;
}

// ---- attribute access with the reference's contract: returns false and stores the default when absent
template <typename T>
bool GetNodeAttr(const PbNode& n, const char* key, T* value, T dft) {
    for (auto& a : n.attrs) {
        if (a.name == key) {
            *value = std::is_floating_point<T>::value ? (T)a.f : (T)a.i;
            return true;
        }
    }
    *value = dft;
    return false;
}

struct ParserInfo final {
    std::function<std::shared_ptr<ir::Attr>()> create_param; // may be empty for ops without attributes
    std::function<RetCode(const PbNode&, const ir::Node&, ir::Attr*)> parse_param;
};

RetCode ParseMultiHeadCacheAttentionParam(const PbNode& pb, const ir::Node& node, ir::Attr* arg) {
    const std::string& node_name = node.name;
    auto param = static_cast<opmx::MultiHeadCacheAttentionParam*>(arg);
    if (!GetNodeAttr(pb, "num_heads", &param->num_heads, -1)) { LOG(ERROR) << node_name << ": missing num_heads"; return RC_INVALID_VALUE; }
    if (!GetNodeAttr(pb, "head_dim", &param->head_dim, -1)) { LOG(ERROR) << node_name << ": missing head_dim"; return RC_INVALID_VALUE; }
    if (!GetNodeAttr(pb, "num_layer", &param->num_layer, -1)) { LOG(ERROR) << node_name << ": missing num_layer"; return RC_INVALID_VALUE; }
    if (!GetNodeAttr(pb, "layer_idx", &param->layer_idx, -1)) { LOG(ERROR) << node_name << ": missing layer_idx"; return RC_INVALID_VALUE; }
    int32_t is_causal, is_alibi;
    GetNodeAttr(pb, "is_causal", &is_causal, 1);
    param->is_causal = is_causal;
    GetNodeAttr(pb, "is_alibi", &is_alibi, 0);
    param->is_alibi = is_alibi;
    GetNodeAttr(pb, "num_kv_heads", &param->num_kv_heads, param->num_heads);
    GetNodeAttr(pb, "quant_bit", &param->quant_bit, 0);
    GetNodeAttr(pb, "quant_group", &param->quant_group, 8);
    GetNodeAttr(pb, "cache_mode", &param->cache_mode, 0);
    GetNodeAttr(pb, "cache_layout", &param->cache_layout, 0);
    GetNodeAttr(pb, "page_size", &param->page_size, 128);
    return RC_SUCCESS;
}

RetCode ParseKeyValueCacheParam(const PbNode& pb, const ir::Node& node, ir::Attr* arg) {
    const std::string& node_name = node.name;
    auto param = static_cast<opmx::KeyValueCacheParam*>(arg);
    if (!GetNodeAttr(pb, "num_layer", &param->num_layer, -1)) { LOG(ERROR) << node_name << ": missing num_layer"; return RC_INVALID_VALUE; }
    if (!GetNodeAttr(pb, "layer_idx", &param->layer_idx, -1)) { LOG(ERROR) << node_name << ": missing layer_idx"; return RC_INVALID_VALUE; }
    GetNodeAttr(pb, "quant_bit", &param->quant_bit, 0);
    GetNodeAttr(pb, "quant_group", &param->quant_group, 8);
    GetNodeAttr(pb, "num_repeat", &param->num_repeat, 1);
    GetNodeAttr(pb, "cache_mode", &param->cache_mode, 0);
    GetNodeAttr(pb, "cache_layout", &param->cache_layout, 0);
    GetNodeAttr(pb, "page_size", &param->page_size, 128);
    return RC_SUCCESS;
}

// models/onnx/parsers/opmx/parse_multi_head_attention_param.cc:10-31
RetCode ParseMultiHeadAttentionParam(const PbNode& pb, const ir::Node& node, ir::Attr* arg) {
    const std::string& node_name = node.name;
    auto param = static_cast<opmx::MultiHeadAttentionParam*>(arg);
    if (!GetNodeAttr(pb, "num_heads", &param->num_heads, -1)) { LOG(ERROR) << node_name << ": missing num_heads"; return RC_INVALID_VALUE; }
    if (!GetNodeAttr(pb, "head_dim", &param->head_dim, -1)) { LOG(ERROR) << node_name << ": missing head_dim"; return RC_INVALID_VALUE; }
    int32_t is_causal, is_alibi;
    GetNodeAttr(pb, "is_causal", &is_causal, 1);
    param->is_causal = is_causal;
    GetNodeAttr(pb, "is_alibi", &is_alibi, 0);
    param->is_alibi = is_alibi;
    GetNodeAttr(pb, "num_kv_heads", &param->num_kv_heads, param->num_heads);
    return RC_SUCCESS;
}

// models/onnx/parsers/opmx/parse_rotary_position_embedding_param.cc:10-41
RetCode ParseRotaryPositionEmbeddingParam(const PbNode& pb, const ir::Node& node, ir::Attr* arg) {
    const std::string& node_name = node.name;
    auto param = static_cast<opmx::RotaryPositionEmbeddingParam*>(arg);
    if (!GetNodeAttr(pb, "theta", &param->theta, -1.0f)) { LOG(ERROR) << node_name << ": missing theta"; return RC_INVALID_VALUE; }
    GetNodeAttr(pb, "bypass_key", &param->bypass_key, 0);
    GetNodeAttr(pb, "rotary_dim", &param->rotary_dim, 0);
    GetNodeAttr(pb, "scaling_factor", &param->scaling_factor, 1.0f);
    GetNodeAttr(pb, "max_position_embeddings", &param->max_position_embeddings, 2048);
    std::string scaling_type;
    for (auto& a : pb.attrs)
        if (a.name == "scaling_type") scaling_type = a.s;
    if (scaling_type == "") {
        param->scaling_type = opmx::RotaryPositionEmbeddingParam::SCALING_TYPE_NONE;
    } else if (scaling_type == "linear") {
        param->scaling_type = opmx::RotaryPositionEmbeddingParam::SCALING_TYPE_LINEAR;
    } else if (scaling_type == "dynamic") {
        param->scaling_type = opmx::RotaryPositionEmbeddingParam::SCALING_TYPE_DYNAMIC;
    } else {
        LOG(ERROR) << "unsupported scaling_type: " << scaling_type;
        return RC_UNSUPPORTED;
    }
    return RC_SUCCESS;
}

// models/onnx/parsers/onnx/parse_softmax_param.cc:26-32: the default axis depends on the opset
RetCode ParseSoftmaxParam(const PbNode& pb, const ir::Node& node, ir::Attr* arg) {
    auto param = static_cast<ppl::nn::onnx::SoftmaxParam*>(arg);
    GetNodeAttr(pb, "axis", &param->axis, node.type.version >= 13 ? -1 : 1);
    return RC_SUCCESS;
}

// models/onnx/parsers/onnx/parse_transpose_param.cc: `perm`, empty = reverse the dimensions
RetCode ParseTransposeParam(const PbNode& pb, const ir::Node&, ir::Attr* arg) {
    auto param = static_cast<ppl::nn::onnx::TransposeParam*>(arg);
    for (auto& a : pb.attrs)
        if (a.name == "perm") param->perm.assign(a.ints.begin(), a.ints.end());
    return RC_SUCCESS;
}

utils::OpInfoManager<ParserInfo>& ParamParserManager() {
    static utils::OpInfoManager<ParserInfo> mgr;
    static std::once_flag once;
    std::call_once(once, [] {
        auto reg = [&](const char* domain, const char* type, uint64_t first, uint64_t last, const ParserInfo& info) {
            if (last < first) { // same reaction as param_parser_manager.cc:111-124
                LOG(ERROR) << "register op[" << domain << ":" << type << "] failed: invalid version range";
                exit(-1);
            }
            mgr.Register(domain, type, utils::VersionRange{first, last}, info);
        };
        reg("opmx.dynamic_batching", "MultiHeadCacheAttention", 1, 1,
            {[] { return std::make_shared<opmx::MultiHeadCacheAttentionParam>(); }, ParseMultiHeadCacheAttentionParam});
        reg("opmx.dynamic_batching", "KeyValueCache", 1, 1,
            {[] { return std::make_shared<opmx::KeyValueCacheParam>(); }, ParseKeyValueCacheParam});
        reg("opmx.dynamic_batching", "MultiHeadAttention", 1, 1,
            {[] { return std::make_shared<opmx::MultiHeadAttentionParam>(); }, ParseMultiHeadAttentionParam});
        reg("opmx.dynamic_batching", "RotaryPositionEmbedding", 1, 1,
            {[] { return std::make_shared<opmx::RotaryPositionEmbeddingParam>(); }, ParseRotaryPositionEmbeddingParam});
        reg("opmx.dynamic_batching", "PositionIndex", 1, 1, {nullptr, nullptr}); // no attributes
        // the ONNX ops of the attention subgraph the x86 engine runs (param_parser_manager.cc: same version ranges)
        reg("", "Softmax", 1, 16, {[] { return std::make_shared<ppl::nn::onnx::SoftmaxParam>(); }, ParseSoftmaxParam});
        reg("", "Transpose", 1, 16, {[] { return std::make_shared<ppl::nn::onnx::TransposeParam>(); }, ParseTransposeParam});
        reg("", "MatMul", 1, 16, {nullptr, nullptr});
        reg("", "Mul", 7, 16, {nullptr, nullptr});
        reg("", "Add", 7, 16, {nullptr, nullptr});
    });
    return mgr;
}

} // namespace

RetCode ParseModel(const char* buf, uint64_t size, ir::Graph* graph) {
    Reader model(buf, size);
    std::map<std::string, uint64_t> opsets; // domain -> max version (model_parser.cc:52-62)
    Reader graph_pb(nullptr, 0);
    bool has_graph = false;
    while (!model.Done()) {
        uint32_t wt; Reader sub(nullptr, 0); uint64_t v = 0;
        const uint32_t f = model.Next(&wt, &sub, &v);
        if (!model.ok) break;
        if (f == 7 && wt == 2) { graph_pb = sub; has_graph = true; }
        else if (f == 8 && wt == 2) {
            std::string domain; uint64_t version = 0;
            Reader os = sub;
            while (!os.Done()) {
                uint32_t wt2; Reader s2(nullptr, 0); uint64_t v2 = 0;
                const uint32_t f2 = os.Next(&wt2, &s2, &v2);
                if (!os.ok) break;
                if (f2 == 1 && wt2 == 2) domain = s2.Str();
                else if (f2 == 2 && wt2 == 0) version = v2;
            }
            auto it = opsets.find(domain);
            if (it == opsets.end() || it->second < version) opsets[domain] = version;
        }
    }
    if (!model.ok || !has_graph) {
        LOG(ERROR) << "parse onnx model failed: malformed ModelProto";
        return RC_INVALID_VALUE;
    }

    graph->topo = std::make_shared<ir::GraphTopo>();
    graph->data = std::make_shared<ir::GraphData>();
    auto topo = graph->topo.get();
    auto data = graph->data.get();

    std::vector<PbNode> nodes;
    std::vector<std::pair<std::string, ir::Shape>> inputs, outputs;
    Reader g = graph_pb;
    while (!g.Done()) {
        uint32_t wt; Reader sub(nullptr, 0); uint64_t v = 0;
        const uint32_t f = g.Next(&wt, &sub, &v);
        if (!g.ok) break;
        if (wt != 2) continue;
        switch (f) {
            case 1: { PbNode n; if (!ParseNode(sub, &n)) { g.ok = false; break; } nodes.push_back(n); break; }
            case 2: topo->name = sub.Str(); break;
            case 5: { // initializer
                std::string name; ir::Shape shape; ir::Constant c;
                if (!ParseInitializer(sub, &name, &shape, &c)) {
                    LOG(ERROR) << "parse initializer failed (external data is unsupported)";
                    return RC_UNSUPPORTED;
                }
                const edgeid_t eid = topo->AddEdge(name);
                topo->constants.push_back(eid);
                data->shapes[eid] = shape;
                data->constants[eid] = c;
                break;
            }
            case 11: { std::string name; ir::Shape s; if (!ParseValueInfo(sub, &name, &s)) { g.ok = false; break; } inputs.emplace_back(name, s); break; }
            case 12: { std::string name; ir::Shape s; if (!ParseValueInfo(sub, &name, &s)) { g.ok = false; break; } outputs.emplace_back(name, s); break; }
            case 14: LOG(ERROR) << "quantization_annotation is not supported"; return RC_UNSUPPORTED; // model_parser.cc:74-77
            default: break;
        }
    }
    if (!g.ok) {
        LOG(ERROR) << "parse onnx model failed: malformed GraphProto";
        return RC_INVALID_VALUE;
    }

    for (auto& in : inputs) {
        const edgeid_t eid = topo->AddEdge(in.first);
        bool is_const = false;
        for (auto c : topo->constants) is_const |= (c == eid);
        if (is_const) continue; // graph inputs that are initialisers stay constants (graph_parser.cc:114-143)
        topo->inputs.push_back(eid);
        data->shapes[eid] = in.second;
    }

    uint32_t anonymous = 0;
    for (auto& pb : nodes) {
        ir::Node node;
        node.id = (nodeid_t)topo->nodes.size();
        node.name = pb.name.empty() ? "ppl_anonymous_node_" + std::to_string(anonymous++) : pb.name;
        auto os = opsets.find(pb.domain);
        if (os == opsets.end()) { // graph_parser.cc:166-172
            LOG(ERROR) << "opset of domain[" << pb.domain << "] for node[" << node.name << "] is not imported";
            return RC_NOT_FOUND;
        }
        node.type.domain = pb.domain;
        node.type.name = pb.op_type;
        node.type.version = os->second;
        for (auto& in : pb.inputs) {
            if (in.empty()) { node.inputs.push_back(INVALID_EDGEID); continue; } // optional slot left empty
            const edgeid_t eid = topo->AddEdge(in);
            topo->edges[eid].consumers.push_back(node.id);
            node.inputs.push_back(eid);
        }
        for (auto& out : pb.outputs) {
            const edgeid_t eid = topo->AddEdge(out);
            topo->edges[eid].producer = node.id;
            node.outputs.push_back(eid);
        }
        auto info = ParamParserManager().Find(node.type.domain, node.type.name, node.type.version);
        if (info && info->create_param) {
            auto param = info->create_param();
            const RetCode rc = info->parse_param(pb, node, param.get());
            if (rc != RC_SUCCESS) {
                LOG(ERROR) << "parse attr of node[" << node.name << "] failed: " << GetRetCodeStr(rc);
                return rc;
            }
            data->attrs[node.id] = param;
        }
        topo->nodes.push_back(node);
    }
    for (auto& out : outputs) {
        const edgeid_t eid = topo->FindEdge(out.first);
        if (eid == INVALID_EDGEID) {
            LOG(ERROR) << "graph output[" << out.first << "] is not produced by any node";
            return RC_NOT_FOUND;
        }
        topo->outputs.push_back(eid);
        data->shapes[eid] = out.second;
    }
    return RC_SUCCESS;
}

}}} // namespace ppl::nn::onnx
