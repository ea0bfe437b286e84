// PMX op-parameter blobs of the attention-path ops: the FlatBuffers tables of
//   src/ppl/nn/engines/llm_cuda/pmx/schema/llm_cuda_op_params.fbs:14-23 (KeyValueCacheParam), :31-37
//   (MultiHeadAttentionParam), :60-67 (RotaryPositionEmbeddingParam), :75-88 (MultiHeadCacheAttentionParam), wrapped in
//   `table OpParam { value: OpParamType; }` (:123-145), as written and read by the ops' SerializeData / DeserializeData
//   (e.g. ops/opmx/dynamic_batching/multi_head_cache_attention_op.cc:55-94).
// The FlatBuffers library is not used: the wire format is small enough to state directly.
//   buffer  = [uoffset32 -> root table] ...
//   table   = [soffset32: table position - vtable position] [inline fields ...]
//   vtable  = [u16 vtable bytes] [u16 table bytes] [u16 offset of field i inside the table, 0 = absent -> default] ...
//   a union = two fields: the u8 type tag, then a uoffset32 (relative to its own position) to the member table
// Scalars equal to their default (0 / false / 0.0f for every field of these tables) are left out by writers and read
// back as the default, which is what the reference's generated accessors do.
#ifndef PPLNN_LLM_HIP_PMX_PARAMS_H_
#define PPLNN_LLM_HIP_PMX_PARAMS_H_

#include <cstring>
#include <string>
#include <vector>

#include "params.h"

namespace ppl { namespace nn { namespace pmx {

using ppl::common::RetCode;

// union OpParamType, in schema order (llm_cuda_op_params.fbs:123-139); NONE = 0
enum OpParamType : uint8_t {
    OpParamType_NONE = 0,
    OpParamType_ColumnParallelLinearParam = 1,
    OpParamType_GELUParam = 2,
    OpParamType_KeyValueCacheParam = 3,
    OpParamType_LayerNormParam = 4,
    OpParamType_MultiHeadAttentionParam = 5,
    OpParamType_ParallelEmbeddingParam = 6,
    OpParamType_RMSNormParam = 7,
    OpParamType_RotaryPositionEmbeddingParam = 8,
    OpParamType_RowParallelLinearParam = 9,
    OpParamType_MultiHeadCacheAttentionParam = 10,
};

// ---- writer: one member table of 4-byte and 1-byte scalar fields, wrapped in OpParam
class TableWriter final {
public:
    void AddI32(int field, int32_t v) { if (v != 0) Add(field, &v, 4); }
    void AddU32(int field, uint32_t v) { if (v != 0) Add(field, &v, 4); }
    void AddF32(int field, float v) { if (v != 0.0f) Add(field, &v, 4); }
    void AddBool(int field, bool v) { if (v) { uint8_t b = 1; Add(field, &b, 1); } }

    // [root uoffset][OpParam vtable][OpParam table][member vtable][member table]
    std::string Finish(OpParamType type, int num_fields) const {
        std::string out;
        auto put16 = [&](uint16_t v) { out.append((const char*)&v, 2); };
        auto put32 = [&](uint32_t v) { out.append((const char*)&v, 4); };
        auto align4 = [&] { while (out.size() & 3) out.push_back(0); };
        put32(0); // root offset, patched below
        // OpParam: field 0 = value_type (u8), field 1 = value (uoffset32)
        const size_t root_vt = out.size();
        put16(8);
        put16(12);
        put16(8); // value_type at table + 8
        put16(4); // value at table + 4
        align4();
        const size_t root_tab = out.size();
        put32((uint32_t)(int32_t)(root_tab - root_vt));
        const size_t value_pos = out.size();
        put32(0); // patched
        out.push_back((char)type);
        align4();
        // member table: 4-byte fields first, then the bools
        std::vector<uint16_t> offs(num_fields, 0);
        std::string body(4, '\0'); // soffset placeholder
        for (int pass = 0; pass < 2; ++pass)
            for (auto& f : fields_)
                if ((f.size == 4) == (pass == 0)) {
                    offs[f.field] = (uint16_t)body.size();
                    body.append(f.bytes, f.size);
                }
        while (body.size() & 3) body.push_back(0);
        const size_t vt = out.size();
        put16((uint16_t)(4 + 2 * num_fields));
        put16((uint16_t)body.size());
        for (auto o : offs) put16(o);
        align4();
        const size_t tab = out.size();
        const uint32_t so = (uint32_t)(int32_t)(tab - vt);
        memcpy(&body[0], &so, 4);
        out += body;
        const uint32_t rel = (uint32_t)(tab - value_pos), root = (uint32_t)root_tab;
        memcpy(&out[value_pos], &rel, 4);
        memcpy(&out[0], &root, 4);
        return out;
    }

private:
    struct Field {
        int field;
        int size;
        char bytes[4];
    };
    void Add(int field, const void* v, int size) {
        Field f;
        f.field = field;
        f.size = size;
        memcpy(f.bytes, v, size);
        fields_.push_back(f);
    }
    std::vector<Field> fields_;
};

// ---- reader with bounds checks (the reference trusts the buffer; a truncated blob must not read out of range here)
class TableReader final {
public:
    TableReader() {}
    // positions the reader on the member table of an OpParam buffer; false if malformed
    bool Open(const void* base, uint64_t size, OpParamType* type) {
        base_ = (const uint8_t*)base;
        size_ = size;
        uint32_t root;
        if (!Get(0, &root) || !SetTable(root)) return false;
        uint8_t tag = 0;
        const uint32_t type_pos = FieldPos(0), value_pos = FieldPos(1);
        if (type_pos && !Get(type_pos, &tag)) return false;
        *type = (OpParamType)tag;
        if (tag == OpParamType_NONE || !value_pos) return false;
        uint32_t rel;
        if (!Get(value_pos, &rel)) return false;
        return SetTable((uint64_t)value_pos + rel);
    }
    int32_t I32(int field) { return Scalar<int32_t>(field); }
    uint32_t U32(int field) { return Scalar<uint32_t>(field); }
    float F32(int field) { return Scalar<float>(field); }
    bool Bool(int field) { return Scalar<uint8_t>(field) != 0; }
    bool Ok() const { return ok_; } // false once a field that is present pointed outside the buffer

private:
    template <typename T>
    T Scalar(int field) {
        T v = 0;
        const uint32_t p = FieldPos(field);
        if (p && !Get(p, &v)) ok_ = false;
        return v;
    }
    template <typename T>
    bool Get(uint64_t pos, T* v) const {
        if (pos + sizeof(T) > size_) return false;
        memcpy(v, base_ + pos, sizeof(T));
        return true;
    }
    bool SetTable(uint64_t pos) {
        int32_t so;
        if (!Get(pos, &so)) return false;
        const int64_t vt = (int64_t)pos - so;
        uint16_t vsize;
        if (vt < 0 || !Get((uint64_t)vt, &vsize) || vsize < 4 || (uint64_t)vt + vsize > size_) return false;
        table_ = (uint32_t)pos;
        vtable_ = (uint32_t)vt;
        vsize_ = vsize;
        return true;
    }
    uint32_t FieldPos(int field) const { // absolute position of the field's bytes, 0 when absent
        const uint32_t slot = 4 + 2 * (uint32_t)field;
        if (slot + 2 > vsize_) return 0;
        uint16_t off = 0;
        Get(vtable_ + slot, &off);
        return off ? table_ + off : 0;
    }
    const uint8_t* base_ = nullptr;
    uint64_t size_ = 0;
    uint32_t table_ = 0, vtable_ = 0;
    uint16_t vsize_ = 0;
    bool ok_ = true;
};

inline RetCode CheckRead(const TableReader& r) {
    if (r.Ok()) return ppl::common::RC_SUCCESS;
    LOG(ERROR) << "op param buffer is truncated";
    return ppl::common::RC_INVALID_VALUE;
}

// ---- the four tables, field ids in schema order
inline std::string SerializeOpParam(const opmx::MultiHeadCacheAttentionParam& p) {
    TableWriter w;
    w.AddI32(0, p.num_heads);
    w.AddI32(1, p.num_kv_heads);
    w.AddI32(2, p.head_dim);
    w.AddBool(3, p.is_causal);
    w.AddBool(4, p.is_alibi);
    w.AddI32(5, p.num_layer);
    w.AddI32(6, p.layer_idx);
    w.AddI32(7, p.quant_bit);
    w.AddI32(8, p.quant_group);
    w.AddI32(9, p.cache_mode);
    w.AddI32(10, p.cache_layout);
    w.AddI32(11, p.page_size);
    return w.Finish(OpParamType_MultiHeadCacheAttentionParam, 12);
}
inline std::string SerializeOpParam(const opmx::KeyValueCacheParam& p) {
    TableWriter w;
    w.AddI32(0, p.num_layer);
    w.AddI32(1, p.layer_idx);
    w.AddI32(2, p.quant_bit);
    w.AddI32(3, p.quant_group);
    w.AddI32(4, p.num_repeat);
    w.AddI32(5, p.cache_mode);
    w.AddI32(6, p.cache_layout);
    w.AddI32(7, p.page_size);
    return w.Finish(OpParamType_KeyValueCacheParam, 8);
}
inline std::string SerializeOpParam(const opmx::MultiHeadAttentionParam& p) {
    TableWriter w;
    w.AddI32(0, p.num_heads);
    w.AddI32(1, p.num_kv_heads);
    w.AddI32(2, p.head_dim);
    w.AddBool(3, p.is_causal);
    w.AddBool(4, p.is_alibi);
    return w.Finish(OpParamType_MultiHeadAttentionParam, 5);
}
inline std::string SerializeOpParam(const opmx::RotaryPositionEmbeddingParam& p) {
    TableWriter w;
    w.AddI32(0, p.bypass_key);
    w.AddI32(1, p.rotary_dim);
    w.AddF32(2, p.theta);
    w.AddI32(3, p.max_position_embeddings);
    w.AddU32(4, (uint32_t)p.scaling_type);
    w.AddF32(5, p.scaling_factor);
    return w.Finish(OpParamType_RotaryPositionEmbeddingParam, 6);
}

inline RetCode OpenAs(const void* base, uint64_t size, OpParamType want, TableReader* r) {
    OpParamType got = OpParamType_NONE;
    if (!base || !r->Open(base, size, &got)) {
        LOG(ERROR) << "malformed op param buffer of " << size << " bytes";
        return ppl::common::RC_INVALID_VALUE;
    }
    if (got != want) {
        LOG(ERROR) << "op param buffer holds union member " << (int)got << ", expected " << (int)want;
        return ppl::common::RC_INVALID_VALUE;
    }
    return ppl::common::RC_SUCCESS;
}
inline RetCode DeserializeOpParam(const void* base, uint64_t size, opmx::MultiHeadCacheAttentionParam* p) {
    TableReader r;
    auto rc = OpenAs(base, size, OpParamType_MultiHeadCacheAttentionParam, &r);
    if (rc != ppl::common::RC_SUCCESS) return rc;
    p->num_heads = r.I32(0);
    p->num_kv_heads = r.I32(1);
    p->head_dim = r.I32(2);
    p->is_causal = r.Bool(3);
    p->is_alibi = r.Bool(4);
    p->num_layer = r.I32(5);
    p->layer_idx = r.I32(6);
    p->quant_bit = r.I32(7);
    p->quant_group = r.I32(8);
    p->cache_mode = r.I32(9);
    p->cache_layout = r.I32(10);
    p->page_size = r.I32(11);
    return CheckRead(r);
}
inline RetCode DeserializeOpParam(const void* base, uint64_t size, opmx::KeyValueCacheParam* p) {
    TableReader r;
    auto rc = OpenAs(base, size, OpParamType_KeyValueCacheParam, &r);
    if (rc != ppl::common::RC_SUCCESS) return rc;
    p->num_layer = r.I32(0);
    p->layer_idx = r.I32(1);
    p->quant_bit = r.I32(2);
    p->quant_group = r.I32(3);
    p->num_repeat = r.I32(4);
    p->cache_mode = r.I32(5);
    p->cache_layout = r.I32(6);
    p->page_size = r.I32(7);
    return CheckRead(r);
}
inline RetCode DeserializeOpParam(const void* base, uint64_t size, opmx::MultiHeadAttentionParam* p) {
    TableReader r;
    auto rc = OpenAs(base, size, OpParamType_MultiHeadAttentionParam, &r);
    if (rc != ppl::common::RC_SUCCESS) return rc;
    p->num_heads = r.I32(0);
    p->num_kv_heads = r.I32(1);
    p->head_dim = r.I32(2);
    p->is_causal = r.Bool(3);
    p->is_alibi = r.Bool(4);
    return CheckRead(r);
}
inline RetCode DeserializeOpParam(const void* base, uint64_t size, opmx::RotaryPositionEmbeddingParam* p) {
    TableReader r;
    auto rc = OpenAs(base, size, OpParamType_RotaryPositionEmbeddingParam, &r);
    if (rc != ppl::common::RC_SUCCESS) return rc;
    p->bypass_key = r.I32(0);
    p->rotary_dim = r.I32(1);
    p->theta = r.F32(2);
    p->max_position_embeddings = r.I32(3);
    p->scaling_type = (int32_t)r.U32(4);
    p->scaling_factor = r.F32(5);
    return CheckRead(r);
}

}}} // namespace ppl::nn::pmx

#endif
