// Op parameter structs, field for field as in the reference:
//   src/ppl/nn/params/opmx/multi_head_cache_attention_param.h:10-38
//   src/ppl/nn/params/opmx/key_value_cache_param.h:10-30
//   src/ppl/nn/params/opmx/multi_head_attention_param.h:10-26
//   src/ppl/nn/params/opmx/rotary_position_embedding_param.h:10-36
//   src/ppl/nn/params/onnx/softmax_param.h, transpose_param.h (the ONNX ops of the x86 attention subgraph)
#ifndef PPLNN_LLM_HIP_PARAMS_H_
#define PPLNN_LLM_HIP_PARAMS_H_

#include "core.h"

#include <cmath>

namespace ppl { namespace nn { namespace opmx {

struct MultiHeadCacheAttentionParam final : public ir::Attr {
    int32_t num_heads = 0;
    int32_t num_kv_heads = 0;
    int32_t head_dim = 0;
    bool is_causal = true;
    bool is_alibi = false;
    int32_t num_layer = 0;
    int32_t layer_idx = 0;
    int32_t quant_bit = 0;
    int32_t quant_group = 8;
    int32_t cache_mode = 0;
    int32_t cache_layout = 0;
    int32_t page_size = 128;
    bool operator==(const MultiHeadCacheAttentionParam& p) const {
        return num_heads == p.num_heads && num_kv_heads == p.num_kv_heads && head_dim == p.head_dim &&
            is_causal == p.is_causal && is_alibi == p.is_alibi && num_layer == p.num_layer && layer_idx == p.layer_idx &&
            quant_bit == p.quant_bit && quant_group == p.quant_group && cache_mode == p.cache_mode &&
            cache_layout == p.cache_layout && (cache_mode == 0 || page_size == p.page_size);
    }
};

struct KeyValueCacheParam final : public ir::Attr {
    int32_t num_layer = 0;
    int32_t layer_idx = 0;
    int32_t quant_bit = 0;
    int32_t quant_group = 8;
    int32_t num_repeat = 1;
    int32_t cache_mode = 0;
    int32_t cache_layout = 0;
    int32_t page_size = 128;
    bool operator==(const KeyValueCacheParam& p) const {
        return num_layer == p.num_layer && layer_idx == p.layer_idx && quant_bit == p.quant_bit &&
            quant_group == p.quant_group && num_repeat == p.num_repeat && cache_mode == p.cache_mode &&
            cache_layout == p.cache_layout && (cache_mode == 0 || page_size == p.page_size);
    }
};

struct MultiHeadAttentionParam final : public ir::Attr {
    int32_t num_heads = 0;
    int32_t num_kv_heads = 0;
    int32_t head_dim = 0;
    bool is_causal = true;
    bool is_alibi = false;
    bool operator==(const MultiHeadAttentionParam& p) const {
        return num_heads == p.num_heads && num_kv_heads == p.num_kv_heads && head_dim == p.head_dim &&
            is_causal == p.is_causal && is_alibi == p.is_alibi;
    }
};

struct RotaryPositionEmbeddingParam final : public ir::Attr {
    enum { SCALING_TYPE_NONE = 0, SCALING_TYPE_LINEAR = 1, SCALING_TYPE_DYNAMIC = 2 };
    int32_t bypass_key = 0;
    int32_t rotary_dim = 0;
    float theta = 10000.0f;
    int32_t max_position_embeddings = 2048;
    int32_t scaling_type = SCALING_TYPE_NONE;
    float scaling_factor = 1.0f;
    bool operator==(const RotaryPositionEmbeddingParam& p) const {
        return bypass_key == p.bypass_key && fabs(theta - p.theta) <= 1e-05 && rotary_dim == p.rotary_dim &&
            scaling_type == p.scaling_type &&
            (scaling_type == SCALING_TYPE_NONE || max_position_embeddings == p.max_position_embeddings) &&
            (scaling_type == SCALING_TYPE_NONE || fabs(scaling_factor - p.scaling_factor) <= 1e-05);
    }
};

}}} // namespace ppl::nn::opmx

namespace ppl { namespace nn { namespace onnx {

struct SoftmaxParam final : public ir::Attr {
    int32_t axis = 1;
    bool operator==(const SoftmaxParam& p) const { return axis == p.axis; }
};

struct TransposeParam final : public ir::Attr {
    std::vector<int32_t> perm;
    bool operator==(const TransposeParam& p) const { return perm == p.perm; }
};

}}} // namespace ppl::nn::onnx

#endif
