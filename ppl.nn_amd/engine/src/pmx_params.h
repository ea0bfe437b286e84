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

// ---- writer: one member table of 4-byte and 1-byte scalar fields, wrapped in OpParam. The bytes are laid out the
// way the reference's serialisers lay them out, i.e. the way flatbuffers::FlatBufferBuilder does when driven by the
// generated Create*Param / CreateOpParam / FinishOpParamBuffer functions (pmx/generated/
// llm_cuda_op_params_generated.h:1042-1070, 1545-1553, 1654-1658): the buffer grows downwards; the 4-byte fields are
// added in reverse schema order, then the 1-byte fields in reverse order; a scalar equal to its default is not
// written; every write is aligned to its size counted from the END of the buffer; a table ends with its soffset and a
// vtable just long enough for the highest field present; the root offset comes last, i.e. first in memory.
class TableWriter final {
public:
    void AddI32(int field, int32_t v) { if (v != 0) Add(field, &v, 4); }
    void AddU32(int field, uint32_t v) { if (v != 0) Add(field, &v, 4); }
    void AddF32(int field, float v) { if (v != 0.0f) Add(field, &v, 4); }
    void AddBool(int field, bool v) { if (v) { uint8_t b = 1; Add(field, &b, 1); } }

    std::string Finish(OpParamType type, int /*num_fields*/) const {
        Down b;
        // member table
        uint32_t start = b.Size();
        for (int size = 4; size >= 1; size -= 3) // 4-byte fields, then 1-byte fields
            for (int field = 63; field >= 0; --field)
                for (auto& f : fields_)
                    if (f.field == field && f.size == size) b.AddElement(4 + 2 * field, f.bytes, size);
        const uint32_t member = b.EndTable(start);
        // OpParam { value_type: u8 (slot 4), value: offset (slot 6) }: the offset is added first
        start = b.Size();
        const uint32_t rel = b.ReferTo(member);
        b.AddElement(6, &rel, 4);
        const uint8_t tag = (uint8_t)type;
        b.AddElement(4, &tag, 1);
        const uint32_t root = b.EndTable(start);
        // Finish(root): pad so that the whole buffer is a multiple of the largest alignment used, then the root offset
        b.Pad((4 - (b.Size() + 4) % 4) % 4);
        const uint32_t root_rel = b.ReferTo(root);
        b.Push(&root_rel, 4);
        return b.bytes;
    }

private:
    struct Down final { // bytes written so far, in memory order: a write prepends; offsets count from the end
        std::string bytes;
        std::vector<std::pair<int, uint32_t>> slots; // (vtable slot, offset) of the table being built
        uint32_t Size() const { return (uint32_t)bytes.size(); }
        void Pad(size_t n) { bytes.insert(0, n, '\0'); }
        void Align(size_t n) { Pad((n - bytes.size() % n) % n); }
        uint32_t Push(const void* v, int size) {
            Align(size);
            bytes.insert(0, (const char*)v, size);
            return Size();
        }
        void AddElement(int slot, const void* v, int size) { slots.emplace_back(slot, Push(v, size)); }
        uint32_t ReferTo(uint32_t off) {
            Align(4);
            return Size() - off + 4;
        }
        uint32_t EndTable(uint32_t start) {
            const int32_t zero = 0;
            const uint32_t table = Push(&zero, 4); // soffset, patched below
            int max_slot = 2;
            for (auto& s : slots) max_slot = s.first > max_slot ? s.first : max_slot;
            std::string vt(max_slot + 2, '\0');
            const uint16_t vt_bytes = (uint16_t)vt.size(), table_bytes = (uint16_t)(table - start);
            memcpy(&vt[0], &vt_bytes, 2);
            memcpy(&vt[2], &table_bytes, 2);
            for (auto& s : slots) {
                const uint16_t pos = (uint16_t)(table - s.second);
                memcpy(&vt[s.first], &pos, 2);
            }
            bytes.insert(0, vt);
            slots.clear();
            const int32_t so = (int32_t)(Size() - table); // the vtable sits right in front of its table
            memcpy(&bytes[bytes.size() - table], &so, 4);
            return table;
        }
    };
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
