// The attention kernel for everything the specialised kernels (decode.hip, prefill.hip: head_dim 128, at most 16 query
// heads per kv head, no mask) do not take: any head_dim that is a multiple of 32 up to 256, any number of query heads
// per kv head, and an additive attn_mask. One kernel serves decode sequences, prompts and MultiHeadAttention.
//
// Rows of a workgroup are (query token, query head of the kv head) pairs of ONE (sequence, kv head): row r of the
// sequence is token r / rep, head kvh * rep + r % rep, so the K/V tile a workgroup stages in LDS is shared by all query
// heads of its kv head, and a decode sequence (one token) fills rep rows of a tile instead of one. 64 rows per
// workgroup, 16 per wave. Per K/V tile: S^T = K Q^T and O^T += V^T P^T with v_mfma_f32_16x16x16_f16, a query row
// living in the 16 lanes' same column throughout (row statistics are per lane, reductions only over the four 16-lane
// groups); P never leaves registers (the result layout of the first product is the B operand layout of the second);
// V^T operands come from row-major V through ds_read_b64_tr_b16. K/V come from the int8 slab (dequantised on the way
// into LDS, value = fp16(float(q) * float(scale)) as everywhere) or from packed fp16 rows.
// The next K/V tile is requested from memory before the current one is computed. No split of long sequences: this
// path is for coverage, the tuned kernels for speed.
#include "common.h"

namespace pplhip {

typedef short short4_t __attribute__((ext_vector_type(4)));

struct GenericParams {
    const half_t* q; // [S, H, DH]
    const half_t* k16; // packed fp16 rows [*, KVH, DH]: current_key (prompts of a call without cache-prefill) or MHA's key
    const half_t* v16;
    const int64_t* seqstarts;
    const int64_t* kvstarts;
    const int64_t* k16_starts; // row of a sequence's first key in k16 / v16: seqstarts or kvstarts
    const int8_t* cache; // int8 slab and scales (null for MultiHeadAttention)
    const half_t* scale;
    PageMap pages;
    CacheAddr addr;
    const half_t* mask; // additive, or null: mask[h * stride_h + (seqstarts[b] + t) * stride_q + kvstarts[b] + j]
    int64_t mask_stride_h, mask_stride_q;
    half_t* out; // [S, H, DH]
    int32_t batch, num_heads, kv_heads, rep;
    int32_t first_fp16_seq; // sequences [0, first_fp16_seq) read the slab, the others the fp16 rows
    int32_t is_causal;
    int32_t tiles_max; // row tiles of the longest sequence
    float scale_log2; // log2(e) / sqrt(DH)
};

constexpr int kGenRows = 64;
constexpr float kLog2e = 1.4426950408889634f;

template <int DH>
__global__ __launch_bounds__(256) void generic_attention_kernel(const GenericParams p) {
    constexpr int BN = DH <= 128 ? 64 : 32; // kv tokens per tile
    constexpr int LDK = DH + 8; // halves per LDS row (padding spreads the rows over the banks)
    constexpr int KC = DH / 16;
    constexpr int TB = BN / 16;
    __shared__ __attribute__((aligned(16))) half_t Ks[BN * LDK];
    __shared__ __attribute__((aligned(16))) half_t Vs[BN * LDK];

    const int64_t blk = blockIdx.x;
    const int tile = (int)(blk % p.tiles_max);
    const int64_t rest = blk / p.tiles_max;
    const int kvh = (int)(rest % p.kv_heads);
    const int b = (int)(rest / p.kv_heads);
    const int64_t s0 = p.seqstarts[b];
    const int64_t L = p.seqstarts[b + 1] - s0;
    const int64_t kv_first = p.kvstarts[b];
    const int64_t kvlen = p.kvstarts[b + 1] - kv_first;
    const int64_t rows = L * p.rep;
    const int64_t row0 = (int64_t)tile * kGenRows;
    if (row0 >= rows || kvlen <= 0) return;
    const int64_t sp = kvlen > L ? kvlen - L : 0;
    const bool from_slab = b < p.first_fp16_seq;
    const int64_t k16_row0 = from_slab ? 0 : p.k16_starts[b];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r_lane = lane & 15, g = lane >> 4;
    const int64_t my_row_raw = row0 + wave * 16 + r_lane;
    const bool valid = my_row_raw < rows;
    const int64_t my_row = valid ? my_row_raw : rows - 1;
    const int64_t tok = my_row / p.rep;
    const int head = kvh * p.rep + (int)(my_row - tok * p.rep);
    // keys 0 .. row_limit are visible to this lane's row
    const int64_t all = kvlen - 1;
    const int64_t row_limit = !valid ? -1 : (p.is_causal ? (sp + tok < all ? sp + tok : all) : all);
    const int64_t last_row = (row0 + kGenRows - 1 < rows - 1) ? row0 + kGenRows - 1 : rows - 1;
    const int64_t kv_end = p.is_causal ? ((sp + last_row / p.rep + 1 < kvlen) ? sp + last_row / p.rep + 1 : kvlen) : kvlen;

    // Q^T as the B operand of the score product: channels 16 * kc + 4 * g .. + 3 of the lane's row
    half4_t qf[KC];
    {
        const half_t* qp = p.q + ((s0 + tok) * p.num_heads + head) * DH + 4 * g;
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) qf[kc] = *reinterpret_cast<const half4_t*>(qp + 16 * kc);
    }
    const half_t* mrow =
        p.mask ? p.mask + (int64_t)head * p.mask_stride_h + (s0 + tok) * p.mask_stride_q + kv_first : nullptr;

    float m_run = -INFINITY, l_part = 0.f;
    float4_t o[KC];
#pragma unroll
    for (int i = 0; i < KC; ++i) o[i] = float4_t{0.f, 0.f, 0.f, 0.f};

    // A thread's share of a K/V tile: NCH 16-byte chunks (one quantisation group each) of K and of V, as they come from
    // memory. The next tile's are requested before the current tile is computed and go to LDS (dequantised) when it is
    // their turn, so part of a tile's memory latency passes under the arithmetic of the one before. (Two tiles ahead
    // measured slower: 263 against 243 us on 120 decode sequences of head_dim 64.)
    constexpr int CH = DH / 8; // chunks per row
    constexpr int NCH = (BN * CH + 255) / 256; // (the last pass is partial for head_dim 160 and 224)
    struct RawChunk {
        uint4 k, v; // fp16 source: 8 halves each; slab: .x/.y = 8 int8, .z = the group's scale (fp16 bits)
    };
    RawChunk raw[NCH];
    // contiguous slab region: the sequence's first slab token, looked up once
    const int64_t seq_tok0 = from_slab && p.pages.page_shift == 0 ? p.pages.cachestarts[b] : 0;
    auto fetch = [&](int64_t kv0) {
#pragma unroll
        for (int n = 0; n < NCH; ++n) {
            const int c = tid + 256 * n;
            const int r = c / CH, ch = c - r * CH;
            const int64_t j = kv0 + r;
            raw[n].k = raw[n].v = make_uint4(0, 0, 0, 0);
            if (c < BN * CH && j < kvlen) {
                if (from_slab) {
                    const int64_t t_slab = p.pages.page_shift == 0 ? seq_tok0 + j : p.pages.token(b, j);
                    const int64_t rk = p.addr.row(t_slab, 0, kvh), rv = p.addr.row(t_slab, 1, kvh);
                    const uint2 qk = *reinterpret_cast<const uint2*>(p.cache + rk + ch * 8);
                    const uint2 qv = *reinterpret_cast<const uint2*>(p.cache + rv + ch * 8);
                    uint16_t sk, sv;
                    __builtin_memcpy(&sk, &p.scale[rk / kQuantGroup + ch], 2);
                    __builtin_memcpy(&sv, &p.scale[rv / kQuantGroup + ch], 2);
                    raw[n].k = make_uint4(qk.x, qk.y, sk, 0);
                    raw[n].v = make_uint4(qv.x, qv.y, sv, 0);
                } else {
                    const int64_t off = ((k16_row0 + j) * p.kv_heads + kvh) * DH + ch * 8;
                    raw[n].k = *reinterpret_cast<const uint4*>(p.k16 + off);
                    raw[n].v = *reinterpret_cast<const uint4*>(p.v16 + off);
                }
            }
        }
    };
    auto dequant = [&](const uint4& x) { // slab chunk -> 8 halves, fp16(float(q) * float(scale)) as everywhere
        half_t sc;
        const uint16_t bits = (uint16_t)x.z;
        __builtin_memcpy(&sc, &bits, 2);
        const float sf = (float)sc;
        const uint32_t w[2] = {x.x, x.y};
        half8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (half_t)((float)(int)(int8_t)((w[i >> 2] >> (8 * (i & 3))) & 0xff) * sf);
        return o;
    };
    auto stash = [&]() {
#pragma unroll
        for (int n = 0; n < NCH; ++n) {
            const int c = tid + 256 * n;
            if (c >= BN * CH) break;
            const int r = c / CH, ch = c - r * CH;
            half8_t kx, vx;
            if (from_slab) {
                kx = dequant(raw[n].k);
                vx = dequant(raw[n].v);
            } else {
                __builtin_memcpy(&kx, &raw[n].k, 16);
                __builtin_memcpy(&vx, &raw[n].v, 16);
            }
            *reinterpret_cast<half8_t*>(&Ks[r * LDK + ch * 8]) = kx;
            *reinterpret_cast<half8_t*>(&Vs[r * LDK + ch * 8]) = vx;
        }
    };
    // a wave none of whose 16 rows exists (a decode sequence fills rep rows of the tile's 64) only helps to stage the
    // tiles: its arithmetic would be thrown away, and it would take the matrix cores from the waves that have rows
    const bool wave_has_rows = row0 + wave * 16 < rows;
    fetch(0);
    for (int64_t kv0 = 0; kv0 < kv_end; kv0 += BN) {
        __syncthreads(); // everybody has finished reading the previous tile
        stash();
        if (kv0 + BN < kv_end) fetch(kv0 + BN);
        __syncthreads();
        if (!wave_has_rows) continue;

        // ---- scores of the lane's row against tokens kv0 + 16 * tb + 4 * g + i, in the exp2 domain
        float s[TB][4];
        float mx = -INFINITY;
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kc = 0; kc < KC; ++kc) {
                const half4_t a = *reinterpret_cast<const half4_t*>(&Ks[(16 * tb + r_lane) * LDK + 16 * kc + 4 * g]);
                acc = __builtin_amdgcn_mfma_f32_16x16x16f16(a, qf[kc], acc, 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t j = kv0 + 16 * tb + 4 * g + i;
                float v = acc[i] * p.scale_log2;
                if (j <= row_limit) {
                    if (mrow) v += (float)mrow[j] * kLog2e;
                } else {
                    v = -INFINITY;
                }
                s[tb][i] = v;
                mx = fmaxf(mx, v);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        // a row that has seen nothing but masked keys so far keeps max -inf: its probabilities are zero, not NaN
        const float alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m_run - m_new);
        half4_t pf[TB];
        float psum = 0.f;
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = m_new == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(s[tb][i] - m_new);
                const half_t h = (half_t)e;
                pf[tb][i] = h;
                psum += (float)h; // the sum of what the second product multiplies
            }
        }
        l_part = l_part * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int db = 0; db < KC; ++db) {
            o[db] *= alpha;
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) {
                // V^T operand: lane (block g, j) receives channel 16 * db + j of tokens 16 * tb + 4 * g .. + 3 when
                // lane 4 * i + c of the block addresses token 16 * tb + 4 * g + i, channels 16 * db + 4 * c .. + 3
                const half_t* src = &Vs[(16 * tb + 4 * g + (r_lane >> 2)) * LDK + 16 * db + 4 * (r_lane & 3)];
                const short4_t raw =
                    __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)src);
                half4_t a;
                __builtin_memcpy(&a, &raw, 8);
                o[db] = __builtin_amdgcn_mfma_f32_16x16x16f16(a, pf[tb], o[db], 0, 0, 0);
            }
        }
    }
    float l = l_part;
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    if (!valid) return;
    // a row whose keys were all masked out has no distribution: zeros
    const float inv_l = l > 0.f ? 1.0f / l : 0.f;
    half_t* dst = p.out + ((s0 + tok) * p.num_heads + head) * DH + 4 * g;
#pragma unroll
    for (int db = 0; db < KC; ++db) {
        const half4_t r = {(half_t)(o[db][0] * inv_l), (half_t)(o[db][1] * inv_l), (half_t)(o[db][2] * inv_l),
                           (half_t)(o[db][3] * inv_l)};
        *reinterpret_cast<half4_t*>(dst + 16 * db) = r;
    }
}

template <int DH>
static void launch_one(const GenericParams& p, int64_t blocks, hipStream_t stream) {
    hipLaunchKernelGGL(generic_attention_kernel<DH>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
}

bool generic_head_dim_supported(int head_dim) {
    return head_dim >= 32 && head_dim <= 256 && head_dim % 32 == 0;
}

static pplhip_retcode launch_generic(GenericParams& p, int head_dim, int64_t max_seqlen, hipStream_t stream) {
    if (!generic_head_dim_supported(head_dim))
        PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "head_dim %d: must be a multiple of 32 between 32 and 256", head_dim);
    p.scale_log2 = kLog2e / sqrtf((float)head_dim);
    const int64_t tiles = (max_seqlen * p.rep + kGenRows - 1) / kGenRows;
    if (tiles <= 0 || p.batch <= 0) return PPLHIP_RC_SUCCESS;
    const int64_t blocks = tiles * p.kv_heads * (int64_t)p.batch;
    if (tiles > 0x7fffffffLL || blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "attention: too many row tiles");
    p.tiles_max = (int32_t)tiles;
    switch (head_dim) {
        case 32: launch_one<32>(p, blocks, stream); break;
        case 64: launch_one<64>(p, blocks, stream); break;
        case 96: launch_one<96>(p, blocks, stream); break;
        case 128: launch_one<128>(p, blocks, stream); break;
        case 160: launch_one<160>(p, blocks, stream); break;
        case 192: launch_one<192>(p, blocks, stream); break;
        case 224: launch_one<224>(p, blocks, stream); break;
        default: launch_one<256>(p, blocks, stream); break;
    }
    PPLHIP_CHECK_LAUNCH("generic_attention");
    return PPLHIP_RC_SUCCESS;
}

// MultiHeadCacheAttention through the general kernel; the new tokens are already in the slab.
pplhip_retcode launch_generic_mhca(const pplhip_mhca_args* a, hipStream_t stream) {
    GenericParams p;
    p.q = (const half_t*)a->d_query;
    p.k16 = (const half_t*)a->d_current_key;
    p.v16 = (const half_t*)a->d_current_value;
    p.seqstarts = a->d_seqstarts;
    p.kvstarts = a->d_kvstarts;
    p.k16_starts = a->d_seqstarts;
    p.cache = (const int8_t*)a->d_cache;
    p.scale = (const half_t*)a->d_scale;
    p.pages = PageMap{a->d_cachestarts, a->cachestart_stride_b, page_shift_of(a->cache_mode, a->page_size)};
    p.addr = CacheAddr{a->cache_stride_s, a->cache_stride_l, a->cache_stride_h, a->cache_stride_kv, a->layer_idx};
    p.mask = (const half_t*)a->d_attn_mask;
    p.mask_stride_h = a->attn_mask_stride_h;
    p.mask_stride_q = a->attn_mask_stride_q;
    p.out = (half_t*)a->d_output;
    p.batch = (int32_t)a->batch;
    p.num_heads = a->num_heads;
    p.kv_heads = a->num_kv_heads;
    p.rep = a->num_heads / a->num_kv_heads;
    // decode sequences always attend over the slab; prompts only in a cache-prefill call (otherwise over the fp16 rows
    // they bring, like the specialised path)
    p.first_fp16_seq = a->enable_cache_prefill ? (int32_t)a->batch : (int32_t)a->decoding_batches;
    p.is_causal = a->is_causal;
    const int64_t max_rows_tokens = a->batch > a->decoding_batches ? a->max_seqlen : 1;
    return launch_generic(p, a->head_dim, max_rows_tokens, stream);
}

pplhip_retcode launch_generic_mha(const pplhip_mha_args* a, hipStream_t stream) {
    GenericParams p;
    p.q = (const half_t*)a->d_query;
    p.k16 = (const half_t*)a->d_key;
    p.v16 = (const half_t*)a->d_value;
    p.seqstarts = a->d_seqstarts;
    p.kvstarts = a->d_kvstarts;
    p.k16_starts = a->d_kvstarts;
    p.cache = nullptr;
    p.scale = nullptr;
    p.pages = PageMap{nullptr, 0, 0};
    p.addr = CacheAddr{0, 0, 0, 0, 0};
    p.mask = (const half_t*)a->d_attn_mask;
    p.mask_stride_h = a->attn_mask_stride_h;
    p.mask_stride_q = a->attn_mask_stride_q;
    p.out = (half_t*)a->d_output;
    p.batch = (int32_t)a->batch;
    p.num_heads = a->num_heads;
    p.kv_heads = a->num_kv_heads;
    p.rep = a->num_heads / a->num_kv_heads;
    p.first_fp16_seq = 0;
    p.is_causal = a->is_causal;
    return launch_generic(p, a->head_dim, a->max_seqlen, stream);
}

} // namespace pplhip
