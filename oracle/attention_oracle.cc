// TEST INFRASTRUCTURE ONLY. Scalar CPU restatement of the dynamic-batching attention path.
// Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this library; the product
// (the HIP kernel library and the llm_hip engine) never links, imports or calls it.
//
// What it restates (the arithmetic itself lives in the un-vendored dependency `ppl.llm.kernel.cuda`,
// fetched from GitHub branch `master` by cmake/deps.cmake:290-304, so it is absent from the reference tree):
//   * argument meaning, tensor order, strides      src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/
//                                                   multi_head_cache_attention_kernel.cc:27-41, 136-212
//   * KeyValueCache I/O contract                    .../dynamic_batching/key_value_cache_kernel.cc:26-110 and
//                                                   src/ppl/nn/oputils/opmx/reshape_dynamic_batching_key_value_cache.cc:26-53
//   * table semantics (seqstarts/kvstarts/...)      tools/benchmark_llama/generation_state.cc:60-192
//   * prefill reads fp16 K/V unless cache-prefill   include/ppl/nn/engines/llm_cuda/options.h:139-149
//
// PARITY STATUS (no reference test, fixture or golden vector covers any opmx op, and the reference cannot be
// built or run offline, so each function is pinned by mathematics instead -- see tests/test_oracle_*.py):
//   oracle_kv_quantize_*   rule DEFINED here (published text: "INT8 groupwise", fp16 absmax/127 scale per group
//                          of 8); pinned by closed forms + a numpy restatement over all finite fp16 absmax values.
//                          Bit pattern of the absent CUDA kernel: parity unpinned.
//   oracle_mhca_forward    pinned against a float64 numpy softmax(QK^T/sqrt(d)+mask)V, closed forms
//                          (kvlen 1, equal keys, dominant key), GQA==MHA, decode == last prefill row, NaN poison.
//   oracle_mha_forward     pinned against the same float64 textbook routine (explicit K/V, kvlen >= seqlen offsets)
//                          and by the identity MHCA == MHA applied to KeyValueCache's outputs.
//   oracle_rope_forward    pinned by rotation invariants (pair norms, position 0 = identity, R(p1+p2) = R(p1)R(p2),
//                          q.k depends on the position difference only) and a numpy complex-multiply restatement;
//                          pair convention and NTK formula of the absent kernel: parity unpinned.
//   oracle_position_index  pinned by a Python loop.
//   oracle_kv_cache_forward pinned by |dequant(quant(x)) - x| <= scale/2 and row-order checks.
//   oracle_pack_tables     pinned against a brute-force Python loop written from generation_state.cc.

#include "../include/ppl_llm_kernel_hip.h"
#include "fp16_soft.h"

#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <vector>

using oracle::float_to_half;
using oracle::half_to_float;

namespace {

const int kGroup = 8;

inline uint16_t eps_half() {
    return float_to_half(1e-5f); // 0x00a8, a binary16 subnormal ~= 1.0014e-5
}

// One group of 8 channels. Rule:
//   a = max |x_i|                         (exact in binary16)
//   s = max(fp16_rne(float(a) / 127.0f), fp16_rne(1e-5f))
//   q_i = int8(rint_ties_even(float(fp16_rne(float(x_i) / float(s)))))
void quantize_group(const uint16_t* x, int8_t* q, uint16_t* scale) {
    float amax = 0.f;
    for (int i = 0; i < kGroup; ++i) {
        float v = fabsf(half_to_float(x[i]));
        if (v > amax) amax = v; // NaN never wins; inf does
    }
    uint16_t s = float_to_half(amax / 127.0f);
    const uint16_t e = eps_half();
    if (half_to_float(s) < half_to_float(e)) s = e;
    const float sf = half_to_float(s);
    for (int i = 0; i < kGroup; ++i) {
        const float ratio = half_to_float(float_to_half(half_to_float(x[i]) / sf));
        float r = nearbyintf(ratio); // default rounding mode: ties to even
        if (!(r >= -128.f)) r = -128.f; // also catches NaN
        if (r > 127.f) r = 127.f;
        q[i] = (int8_t)r;
    }
    *scale = s;
}

struct CacheView {
    int8_t* cache;
    uint16_t* scale;
    int64_t ss, sl, sh, skv;
    int layer;
    int8_t* row(int64_t tok, int kv, int head) const {
        return cache + tok * ss + layer * sl + kv * skv + head * sh;
    }
    uint16_t* srow(int64_t tok, int kv, int head) const {
        return scale + (tok * ss + layer * sl + kv * skv + head * sh) / kGroup;
    }
};

// Slab token of token j of sequence b: contiguous region (cache_mode 0) or page table (cache_mode 1) laid out as
// tools/benchmark_llama/generation_state.cc:111-117 fills it: cachestarts[b][p] = first slab token of page p.
inline int64_t slab_token(const int64_t* cachestarts, int cache_mode, int page_size, int64_t stride_b, int64_t b,
                          int64_t j) {
    if (cache_mode == 0) return cachestarts[b] + j;
    return cachestarts[b * stride_b + j / page_size] + j % page_size;
}

void write_new_tokens(const pplhip_kv_write_args* a) {
    CacheView cv{(int8_t*)a->d_cache, (uint16_t*)a->d_scale, a->cache_stride_s, a->cache_stride_l,
                 a->cache_stride_h, a->cache_stride_kv, a->layer_idx};
    const uint16_t* src[2] = {(const uint16_t*)a->d_current_key, (const uint16_t*)a->d_current_value};
    const int KVH = a->num_kv_heads, Dh = a->head_dim;
    for (int64_t b = 0; b < a->batch; ++b) {
        const int64_t s0 = a->d_seqstarts[b], s1 = a->d_seqstarts[b + 1];
        for (int64_t t = s0; t < s1; ++t) {
            const int64_t tok = slab_token(a->d_cachestarts, a->cache_mode, a->page_size, a->cachestart_stride_b, b,
                                           a->d_start_pos[b] + (t - s0));
            for (int kv = 0; kv < 2; ++kv)
                for (int h = 0; h < KVH; ++h) {
                    const uint16_t* x = src[kv] + (t * KVH + h) * Dh;
                    int8_t* q = cv.row(tok, kv, h);
                    uint16_t* s = cv.srow(tok, kv, h);
                    for (int g = 0; g < Dh / kGroup; ++g) quantize_group(x + g * kGroup, q + g * kGroup, s + g);
                }
        }
    }
}

inline void dequant_row(const int8_t* q, const uint16_t* s, int Dh, double* out) {
    for (int d = 0; d < Dh; ++d) out[d] = (double)q[d] * (double)half_to_float(s[d / kGroup]);
}

} // namespace

extern "C" {

void oracle_half_to_float(const uint16_t* h, float* f, int64_t n) {
    for (int64_t i = 0; i < n; ++i) f[i] = half_to_float(h[i]);
}
void oracle_float_to_half(const float* f, uint16_t* h, int64_t n) {
    for (int64_t i = 0; i < n; ++i) h[i] = float_to_half(f[i]);
}

// n_groups groups of 8 binary16 values -> int8 bytes + one binary16 scale per group.
void oracle_kv_quantize_groups(const uint16_t* x, int8_t* q, uint16_t* scale, int64_t n_groups) {
    for (int64_t g = 0; g < n_groups; ++g) quantize_group(x + g * kGroup, q + g * kGroup, scale + g);
}

// q (int8) * scale (binary16) -> float32 (exact product of the two, rounded once to float32).
void oracle_kv_dequant_groups(const int8_t* q, const uint16_t* scale, float* out, int64_t n_groups) {
    for (int64_t g = 0; g < n_groups; ++g)
        for (int i = 0; i < kGroup; ++i) out[g * kGroup + i] = (float)q[g * kGroup + i] * half_to_float(scale[g]);
}

// The additive attention mask (null: none): the entry for head h, packed query token `qtok` and packed key `key`.
// Layout as the C ABI header defines it for pplhip_mhca_args.
static inline double mask_value(const uint16_t* mask, int64_t stride_h, int64_t stride_q, int h, int64_t qtok,
                                int64_t key) {
    return mask ? (double)half_to_float(mask[h * stride_h + qtok * stride_q + key]) : 0.0;
}

// All pointers in the argument blocks are HOST pointers here.
int oracle_kv_quantize_write(const pplhip_kv_write_args* a) {
    if (a->head_dim % kGroup) return PPLHIP_RC_INVALID_VALUE;
    write_new_tokens(a);
    return PPLHIP_RC_SUCCESS;
}

// Write-then-attend. out_f64 (optional) receives the un-rounded double results, [S, H, Dh].
int oracle_mhca_forward(const pplhip_mhca_args* a, double* out_f64) {
    const int H = a->num_heads, KVH = a->num_kv_heads, Dh = a->head_dim;
    if (H <= 0 || KVH <= 0 || H % KVH || Dh % kGroup) return PPLHIP_RC_INVALID_VALUE;
    if (a->d_alibi_slopes || (a->cache_mode != 0 && a->cache_mode != 1)) return PPLHIP_RC_UNSUPPORTED;
    if (a->d_attn_mask && (a->attn_mask_stride_q <= 0 || a->attn_mask_stride_h < 0)) return PPLHIP_RC_INVALID_VALUE;
    pplhip_kv_write_args w;
    memset(&w, 0, sizeof(w));
    w.d_current_key = a->d_current_key;
    w.d_current_value = a->d_current_value;
    w.d_seqstarts = a->d_seqstarts;
    w.d_cachestarts = a->d_cachestarts;
    w.d_start_pos = a->d_start_pos;
    w.batch = a->batch;
    w.total_new_tokens = a->total_new_tokens;
    w.layer_idx = a->layer_idx;
    w.num_layer = a->num_layer;
    w.num_kv_heads = KVH;
    w.head_dim = Dh;
    w.cache_stride_s = a->cache_stride_s;
    w.cache_stride_l = a->cache_stride_l;
    w.cache_stride_h = a->cache_stride_h;
    w.cache_stride_kv = a->cache_stride_kv;
    w.d_cache = a->d_cache;
    w.d_scale = a->d_scale;
    w.cache_mode = a->cache_mode;
    w.page_size = a->page_size;
    w.cachestart_stride_b = a->cachestart_stride_b;
    write_new_tokens(&w);

    CacheView cv{(int8_t*)a->d_cache, (uint16_t*)a->d_scale, a->cache_stride_s, a->cache_stride_l,
                 a->cache_stride_h, a->cache_stride_kv, a->layer_idx};
    const uint16_t* Q = (const uint16_t*)a->d_query;
    const uint16_t* CK = (const uint16_t*)a->d_current_key;
    const uint16_t* CV = (const uint16_t*)a->d_current_value;
    uint16_t* O = (uint16_t*)a->d_output;
    const int rep = H / KVH;
    const double sm_scale = 1.0 / sqrt((double)Dh);
    const uint16_t* mask = (const uint16_t*)a->d_attn_mask;

#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int64_t b = 0; b < a->batch; ++b) {
        for (int h = 0; h < H; ++h) {
            const int kvh = h / rep;
            const int64_t s0 = a->d_seqstarts[b], seqlen = a->d_seqstarts[b + 1] - s0;
            const bool from_cache = (b < a->decoding_batches) || a->enable_cache_prefill;
            // A prefill sequence of a call without cache-prefill attends over the fp16 rows it brings: exactly seqlen
            // keys, query t seeing keys 0..t. Cached history (start_pos > 0) is not looked at on that path; kvstarts
            // only places the sequence's columns in an attn_mask.
            const int64_t sp = from_cache ? a->d_start_pos[b] : 0;
            const int64_t kvlen = from_cache ? a->d_kvstarts[b + 1] - a->d_kvstarts[b] : seqlen;
            // materialise this (sequence, kv head)'s keys and values as doubles
            std::vector<double> K((size_t)kvlen * Dh), V((size_t)kvlen * Dh);
            for (int64_t j = 0; j < kvlen; ++j) {
                if (from_cache) {
                    const int64_t tok =
                        slab_token(a->d_cachestarts, a->cache_mode, a->page_size, a->cachestart_stride_b, b, j);
                    dequant_row(cv.row(tok, 0, kvh), cv.srow(tok, 0, kvh), Dh, &K[j * Dh]);
                    dequant_row(cv.row(tok, 1, kvh), cv.srow(tok, 1, kvh), Dh, &V[j * Dh]);
                } else {
                    // fp16 path: key j of the sequence is packed row seqstarts[b] + j
                    const uint16_t* kr = CK + ((s0 + j) * KVH + kvh) * Dh;
                    const uint16_t* vr = CV + ((s0 + j) * KVH + kvh) * Dh;
                    for (int d = 0; d < Dh; ++d) {
                        K[j * Dh + d] = half_to_float(kr[d]);
                        V[j * Dh + d] = half_to_float(vr[d]);
                    }
                }
            }
            std::vector<double> p((size_t)kvlen), acc(Dh), q(Dh);
            for (int64_t t = 0; t < seqlen; ++t) {
                const uint16_t* qr = Q + ((s0 + t) * H + h) * Dh;
                for (int d = 0; d < Dh; ++d) q[d] = half_to_float(qr[d]);
                const int64_t last = a->is_causal ? std::min<int64_t>(sp + t, kvlen - 1) : kvlen - 1;
                double m = -INFINITY;
                for (int64_t j = 0; j <= last; ++j) {
                    double s = 0;
                    for (int d = 0; d < Dh; ++d) s += q[d] * K[j * Dh + d];
                    p[j] = s * sm_scale + mask_value(mask, a->attn_mask_stride_h, a->attn_mask_stride_q, h, s0 + t,
                                                     a->d_kvstarts[b] + j);
                    m = std::max(m, p[j]);
                }
                double l = 0;
                for (int64_t j = 0; j <= last; ++j) {
                    p[j] = m == -INFINITY ? 0.0 : exp(p[j] - m); // every key masked out: no distribution, zeros
                    l += p[j];
                }
                std::fill(acc.begin(), acc.end(), 0.0);
                for (int64_t j = 0; j <= last; ++j)
                    for (int d = 0; d < Dh; ++d) acc[d] += p[j] * V[j * Dh + d];
                for (int d = 0; d < Dh; ++d) {
                    const double o = l > 0 ? acc[d] / l : 0.0;
                    const int64_t idx = ((s0 + t) * H + h) * Dh + d;
                    if (out_f64) out_f64[idx] = o;
                    O[idx] = float_to_half((float)o);
                }
            }
        }
    }
    return PPLHIP_RC_SUCCESS;
}

// MultiHeadAttention (no cache): explicit packed fp16 key/value rows indexed by kvstarts; the queries of a sequence
// are its last seqlen keys. Argument meaning follows the call at
// src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/multi_head_attention_kernel.cc:105-127.
int oracle_mha_forward(const pplhip_mha_args* a, double* out_f64) {
    const int H = a->num_heads, KVH = a->num_kv_heads, Dh = a->head_dim;
    if (H <= 0 || KVH <= 0 || H % KVH) return PPLHIP_RC_INVALID_VALUE;
    if (a->is_alibi) return PPLHIP_RC_UNSUPPORTED;
    if (a->d_attn_mask && (a->attn_mask_stride_q <= 0 || a->attn_mask_stride_h < 0)) return PPLHIP_RC_INVALID_VALUE;
    const uint16_t* Q = (const uint16_t*)a->d_query;
    const uint16_t* Kp = (const uint16_t*)a->d_key;
    const uint16_t* Vp = (const uint16_t*)a->d_value;
    uint16_t* O = (uint16_t*)a->d_output;
    const int rep = H / KVH;
    const double sm_scale = 1.0 / sqrt((double)Dh);
    const uint16_t* mask = (const uint16_t*)a->d_attn_mask;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int64_t b = 0; b < a->batch; ++b) {
        for (int h = 0; h < H; ++h) {
            const int kvh = h / rep;
            const int64_t s0 = a->d_seqstarts[b], seqlen = a->d_seqstarts[b + 1] - s0;
            const int64_t k0 = a->d_kvstarts[b], kvlen = a->d_kvstarts[b + 1] - k0;
            const int64_t sp = kvlen - seqlen;
            std::vector<double> p((size_t)kvlen), acc(Dh), q(Dh);
            for (int64_t t = 0; t < seqlen; ++t) {
                const uint16_t* qr = Q + ((s0 + t) * H + h) * Dh;
                for (int d = 0; d < Dh; ++d) q[d] = half_to_float(qr[d]);
                const int64_t last = a->is_causal ? std::min<int64_t>(sp + t, kvlen - 1) : kvlen - 1;
                double m = -INFINITY;
                for (int64_t j = 0; j <= last; ++j) {
                    const uint16_t* kr = Kp + ((k0 + j) * KVH + kvh) * Dh;
                    double s = 0;
                    for (int d = 0; d < Dh; ++d) s += q[d] * (double)half_to_float(kr[d]);
                    p[j] = s * sm_scale + mask_value(mask, a->attn_mask_stride_h, a->attn_mask_stride_q, h, s0 + t, k0 + j);
                    m = std::max(m, p[j]);
                }
                double l = 0;
                for (int64_t j = 0; j <= last; ++j) {
                    p[j] = m == -INFINITY ? 0.0 : exp(p[j] - m);
                    l += p[j];
                }
                std::fill(acc.begin(), acc.end(), 0.0);
                for (int64_t j = 0; j <= last; ++j) {
                    const uint16_t* vr = Vp + ((k0 + j) * KVH + kvh) * Dh;
                    for (int d = 0; d < Dh; ++d) acc[d] += p[j] * (double)half_to_float(vr[d]);
                }
                for (int d = 0; d < Dh; ++d) {
                    const double o = l > 0 ? acc[d] / l : 0.0;
                    const int64_t idx = ((s0 + t) * H + h) * Dh + d;
                    if (out_f64) out_f64[idx] = o;
                    O[idx] = float_to_half((float)o);
                }
            }
        }
    }
    return PPLHIP_RC_SUCCESS;
}

// RotaryPositionEmbedding over a ragged batch, float64 throughout, one rounding to binary16 at the end.
// Argument meaning follows src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/
// rotary_position_embedding_kernel.cc:110-132; the angle position * theta^(-2i/rotary_dim) of pair i and the linear /
// dynamic-NTK position scaling restate the published algorithm of the absent kernel library; which channels form a
// pair (consecutive, or i with i + rotary_dim/2) is the caller's pair_layout: parity unpinned against the absent
// kernel's exact bits and against its choice of layout.
int oracle_rope_forward(const pplhip_rope_args* a) {
    const int Dh = a->head_dim, rd = a->rotary_dim == 0 ? Dh : a->rotary_dim;
    if (Dh <= 0 || rd % 2 || rd > Dh) return PPLHIP_RC_INVALID_VALUE;
    if (a->pair_layout != PPLHIP_ROPE_PAIRS_INTERLEAVED && a->pair_layout != PPLHIP_ROPE_PAIRS_HALF_SPLIT)
        return PPLHIP_RC_INVALID_VALUE;
    const bool half_split = a->pair_layout == PPLHIP_ROPE_PAIRS_HALF_SPLIT;
    const uint16_t* Q = (const uint16_t*)a->d_query;
    const uint16_t* K = (const uint16_t*)a->d_key;
    uint16_t* QO = (uint16_t*)a->d_rotated_query;
    uint16_t* KO = (uint16_t*)a->d_rotated_key;
    for (int64_t b = 0; b < a->batch; ++b) {
        const int64_t s0 = a->d_seqstarts[b], seqlen = a->d_seqstarts[b + 1] - s0, sp = a->d_start_pos[b];
        double theta = (double)a->theta;
        if (a->scaling_type == PPLHIP_ROPE_SCALING_DYNAMIC) {
            const double total = (double)(sp + seqlen), maxp = (double)a->max_position_embeddings;
            if (total > maxp) {
                const double f = (double)a->scaling_factor;
                theta *= pow(f * total / maxp - (f - 1.0), (double)rd / (double)(rd - 2));
            }
        }
        for (int64_t t = 0; t < seqlen; ++t) {
            double pos = (double)(sp + t);
            if (a->scaling_type == PPLHIP_ROPE_SCALING_LINEAR) pos /= (double)a->scaling_factor;
            for (int which = 0; which < 2; ++which) {
                const int heads = which ? a->num_key_heads : a->num_heads;
                const uint16_t* src = which ? K : Q;
                uint16_t* dst = which ? KO : QO;
                const bool bypass = which && a->bypass_key;
                for (int h = 0; h < heads; ++h) {
                    const int64_t off = ((s0 + t) * heads + h) * Dh;
                    for (int c = 0; c < Dh; ++c) dst[off + c] = src[off + c]; // channels past rotary_dim, bypassed keys
                    if (bypass) continue;
                    for (int i = 0; i < rd / 2; ++i) {
                        // pair i: consecutive channels, or channel i with channel i + rotary_dim / 2
                        const int lo = half_split ? i : 2 * i, hi = half_split ? i + rd / 2 : 2 * i + 1;
                        const double ang = pos * pow(theta, -2.0 * i / (double)rd);
                        const double c = cos(ang), sn = sin(ang);
                        const double x0 = half_to_float(src[off + lo]), x1 = half_to_float(src[off + hi]);
                        dst[off + lo] = float_to_half((float)(x0 * c - x1 * sn));
                        dst[off + hi] = float_to_half((float)(x1 * c + x0 * sn));
                    }
                }
            }
        }
    }
    return PPLHIP_RC_SUCCESS;
}

// PositionIndex: position of every packed token (position_index_kernel.cc:60-67 for the argument meaning).
int oracle_position_index(const int64_t* start_pos, const int64_t* seqstarts, int64_t batch, int64_t* out) {
    for (int64_t b = 0; b < batch; ++b)
        for (int64_t t = seqstarts[b]; t < seqstarts[b + 1]; ++t) out[t] = start_pos[b] + (t - seqstarts[b]);
    return PPLHIP_RC_SUCCESS;
}

// KeyValueCache op: write, then emit dequantised rows in batch order as binary16 (one rounding of q*scale).
int oracle_kv_cache_forward(const pplhip_kv_cache_args* a) {
    if (a->num_repeat != 1 || a->cache_mode != 0 || a->cache_layout != 0) return PPLHIP_RC_UNSUPPORTED;
    const pplhip_kv_write_args* w = &a->write;
    write_new_tokens(w);
    CacheView cv{(int8_t*)w->d_cache, (uint16_t*)w->d_scale, w->cache_stride_s, w->cache_stride_l,
                 w->cache_stride_h, w->cache_stride_kv, w->layer_idx};
    const int KVH = w->num_kv_heads, Dh = w->head_dim;
    uint16_t* outs[2] = {(uint16_t*)a->d_key_out, (uint16_t*)a->d_value_out};
    for (int64_t b = 0; b < w->batch; ++b) {
        const int64_t k0 = a->d_kvstarts[b], kvlen = a->d_kvstarts[b + 1] - k0;
        for (int64_t j = 0; j < kvlen; ++j) {
            const int64_t tok = w->d_cachestarts[b] + j;
            for (int kv = 0; kv < 2; ++kv)
                for (int h = 0; h < KVH; ++h) {
                    const int8_t* q = cv.row(tok, kv, h);
                    const uint16_t* s = cv.srow(tok, kv, h);
                    uint16_t* o = outs[kv] + ((k0 + j) * KVH + h) * Dh;
                    for (int d = 0; d < Dh; ++d)
                        o[d] = float_to_half((float)q[d] * half_to_float(s[d / kGroup]));
                }
        }
    }
    return PPLHIP_RC_SUCCESS;
}

// Table rebuild: stable compaction (decode first, then prefill), prefix sums, maxima.
// Follows tools/benchmark_llama/generation_state.cc:93-110 (prefix sums, start_pos, cachestarts) and :162-170.
int oracle_pack_tables(const pplhip_pack_args* a) {
    const int n = a->num_slots;
    int64_t b = 0, max_seq = 0, max_kv = 0;
    a->d_seqstarts[0] = 0;
    a->d_kvstarts[0] = 0;
    int64_t decoding = 0;
    for (int pass = 0; pass < 2; ++pass) {
        for (int i = 0; i < n; ++i) {
            const int64_t nl = a->d_slot_newlen[i], kl = a->d_slot_kvlen[i];
            if (nl <= 0) continue;
            const bool is_decode = (nl == 1 && kl > 0);
            if ((pass == 0) != is_decode) continue;
            a->d_seqstarts[b + 1] = a->d_seqstarts[b] + nl;
            a->d_kvstarts[b + 1] = a->d_kvstarts[b] + kl + nl;
            a->d_cachestarts[b] = a->d_slot_cachestart[i];
            a->d_start_pos[b] = kl;
            a->d_batch_slots[b] = i;
            max_seq = std::max(max_seq, nl);
            max_kv = std::max(max_kv, kl + nl);
            ++b;
        }
        if (pass == 0) decoding = b;
    }
    for (int64_t i = b; i < n; ++i) {
        a->d_seqstarts[i + 1] = a->d_seqstarts[b];
        a->d_kvstarts[i + 1] = a->d_kvstarts[b];
        a->d_cachestarts[i] = 0;
        a->d_start_pos[i] = 0;
        a->d_batch_slots[i] = -1;
    }
    a->d_header[0] = b;
    a->d_header[1] = decoding;
    a->d_header[2] = max_seq;
    a->d_header[3] = max_kv;
    a->d_header[4] = a->d_seqstarts[b];
    a->d_header[5] = a->d_kvstarts[b];
    if (a->advance_slots) { // the slot state moves on in the same call (generation_state.cc:127-140: kv lengths grow)
        int64_t* kv = const_cast<int64_t*>(a->d_slot_kvlen);
        for (int i = 0; i < n; ++i)
            if (a->d_slot_newlen[i] > 0) kv[i] += a->d_slot_newlen[i];
    }
    return PPLHIP_RC_SUCCESS;
}

} // extern "C"
