// Causal prefill attention over ragged packed sequences (flash-attention style, fp16 MFMA, fp32 online softmax).
//
// Roofline: fp16 MFMA. One workgroup (4 wavefronts) owns 128 query rows of one (sequence, query head); each wave
// owns 32 of them. K/V tiles of 64 tokens are staged in LDS once per workgroup and shared by the 4 waves; grouped
// query heads map to their kv head by integer division. Everything is computed transposed so that probabilities
// never leave registers:
//   S^T = K * Q^T    v_mfma_f32_32x32x8_f16, A = K tile from LDS (8 B per lane per MFMA), B = Q^T held in registers
//                    -> lane (n = lane & 31, hb = lane >> 5) owns query row n and kv tokens {8*(r/4) + 4*hb + r%4}
//   O^T += V^T * P^T A = V^T: a lane reads 4 tokens x 4 channels from LDS (row-major, conflict-free) and transposes
//                    them in registers with v_perm; B = P^T is exactly the layout the score registers already have.
// Softmax statistics are per lane column, so rescaling O^T needs no cross-lane traffic; one shuffle per tile
// combines the two half-waves' maxima. Tiles entirely above the causal diagonal are skipped, the heaviest query
// tiles are scheduled first.
//
// K/V source: the fp16 current_key/current_value of the sequence (default), or the int8 slab dequantised on the way
// into LDS (cache-prefill: supports start_pos > 0, i.e. chunked prefill / prompt cache).
#include "common.h"

namespace pplhip {

constexpr int kPDh = 128;
constexpr int kBM = 128; // query rows per workgroup
constexpr int kBN = 64; // kv tokens per tile
constexpr int kLdsRow = kPDh * 2 + 8; // bytes per LDS row: 256 B of fp16 + 8 B pad -> 8-byte reads hit distinct banks

struct PrefillParams {
    const half_t* q;
    const half_t* k;
    const half_t* v;
    const int8_t* cache;
    const half_t* scale;
    const int64_t* seqstarts;
    const int64_t* kvstarts;
    const int64_t* cachestarts;
    const int64_t* start_pos;
    half_t* out;
    CacheAddr addr;
    int32_t first_seq; // = decoding_batches
    int32_t num_heads, kv_heads, rep;
    int32_t is_causal;
    float score_scale; // log2(e) / sqrt(Dh)
};

__device__ inline uint32_t pf_as_u32(half2_t h) {
    uint32_t u;
    __builtin_memcpy(&u, &h, 4);
    return u;
}

template <bool FROM_CACHE>
__device__ inline void load_kv_tile(const PrefillParams& p, char* lds_k, char* lds_v, int64_t j0, int64_t kvlen,
                                    int64_t s0, int64_t tok0, int kvh) {
    const int tid = threadIdx.x;
    if (!FROM_CACHE) {
        // 64 rows x 256 B per tensor; thread -> (row = tid/16 + 16*pass, 16 B column chunk tid%16)
        const int col = tid & 15;
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int row = (tid >> 4) + 16 * pass;
            const int64_t j = j0 + row;
            uint4 kx = make_uint4(0, 0, 0, 0), vx = make_uint4(0, 0, 0, 0);
            if (j < kvlen) {
                const int64_t off = ((s0 + j) * p.kv_heads + kvh) * kPDh + col * 8;
                kx = *reinterpret_cast<const uint4*>(p.k + off);
                vx = *reinterpret_cast<const uint4*>(p.v + off);
            }
            uint2* dk = reinterpret_cast<uint2*>(lds_k + row * kLdsRow + col * 16);
            uint2* dv = reinterpret_cast<uint2*>(lds_v + row * kLdsRow + col * 16);
            dk[0] = make_uint2(kx.x, kx.y);
            dk[1] = make_uint2(kx.z, kx.w);
            dv[0] = make_uint2(vx.x, vx.y);
            dv[1] = make_uint2(vx.z, vx.w);
        }
    } else {
        // int8 slab: 64 rows x 128 B (+ 32 B of scales) per tensor; thread -> (row = tid/4, 32-channel quarter tid%4)
        const int row = tid >> 2, quarter = tid & 3;
        const int64_t j = j0 + row;
#pragma unroll
        for (int kv = 0; kv < 2; ++kv) {
            char* dst = (kv ? lds_v : lds_k) + row * kLdsRow + quarter * 64;
            uint32_t w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            half_t sc[4] = {(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
            if (j < kvlen) {
                const int64_t r = p.addr.row(tok0 + j, kv, kvh);
                const uint4 a = *reinterpret_cast<const uint4*>(p.cache + r + quarter * 32);
                const uint4 b = *reinterpret_cast<const uint4*>(p.cache + r + quarter * 32 + 16);
                const uint2 s = *reinterpret_cast<const uint2*>(p.scale + r / kQuantGroup + quarter * 4);
                w[0] = a.x, w[1] = a.y, w[2] = a.z, w[3] = a.w, w[4] = b.x, w[5] = b.y, w[6] = b.z, w[7] = b.w;
                __builtin_memcpy(sc, &s, 8);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                half_t o[8];
                const float sf = (float)sc[g];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int qi = (int)(int8_t)((w[2 * g + (i >> 2)] >> (8 * (i & 3))) & 0xff);
                    o[i] = (half_t)((float)qi * sf);
                }
                uint2 lo, hi;
                __builtin_memcpy(&lo, &o[0], 8);
                __builtin_memcpy(&hi, &o[4], 8);
                reinterpret_cast<uint2*>(dst + g * 16)[0] = lo;
                reinterpret_cast<uint2*>(dst + g * 16)[1] = hi;
            }
        }
    }
}

template <bool FROM_CACHE>
__global__ __launch_bounds__(256, 2) void prefill_attention_kernel(const PrefillParams p) {
    __shared__ __attribute__((aligned(16))) char lds_k[kBN * kLdsRow];
    __shared__ __attribute__((aligned(16))) char lds_v[kBN * kLdsRow];

    const int b = p.first_seq + blockIdx.z;
    const int head = blockIdx.y;
    const int kvh = head / p.rep;
    const int64_t s0 = p.seqstarts[b];
    const int64_t L = p.seqstarts[b + 1] - s0;
    const int64_t sp = FROM_CACHE ? p.start_pos[b] : 0;
    const int64_t kvlen = FROM_CACHE ? (p.kvstarts[b + 1] - p.kvstarts[b]) : L;
    const int64_t tok0 = FROM_CACHE ? p.cachestarts[b] : 0;
    const int ntiles = (int)((L + kBM - 1) / kBM);
    if ((int)blockIdx.x >= ntiles) return;
    const int qt = ntiles - 1 - blockIdx.x; // heaviest (latest) query tiles first
    const int64_t q0 = (int64_t)qt * kBM;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 31;
    const int hb = lane >> 5;
    const int64_t row = q0 + 32 * wave + n; // this lane's query row inside the sequence
    const bool row_ok = row < L;

    // Q^T as the B operand: qB[kk] = Q[row][8*kk + 4*hb .. +3]
    half4_t qB[16];
    {
        const half_t* qp = p.q + ((s0 + (row_ok ? row : 0)) * p.num_heads + head) * kPDh + 4 * hb;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            uint2 x = *reinterpret_cast<const uint2*>(qp + 8 * kk);
            if (!row_ok) x = make_uint2(0, 0);
            __builtin_memcpy(&qB[kk], &x, 8);
        }
    }

    float16_t oT[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oT[i][r] = 0.f;
    float m_run = -INFINITY, l_part = 0.f;

    // keys visible to the last row of this workgroup's tile
    const int64_t last_row = (q0 + kBM < L ? q0 + kBM : L) - 1;
    int64_t kv_end = p.is_causal ? sp + last_row + 1 : kvlen;
    if (kv_end > kvlen) kv_end = kvlen;
    const int64_t wave_last_vis = p.is_causal ? sp + q0 + 32 * wave + 31 : kvlen; // last key any row of this wave sees
    const int64_t wave_first_vis = p.is_causal ? sp + q0 + 32 * wave : kvlen; // keys <= this are seen by all its rows

    for (int64_t j0 = 0; j0 < kv_end; j0 += kBN) {
        __syncthreads();
        load_kv_tile<FROM_CACHE>(p, lds_k, lds_v, j0, kvlen, s0, tok0, kvh);
        __syncthreads();
        if (j0 > wave_last_vis) continue; // the whole tile is above this wave's diagonal (wave-uniform)

        // ---- S^T tiles: 2 x (32 kv tokens x 32 query rows)
        float16_t sT[2];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            float16_t acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
            const char* kr = lds_k + (32 * blk + n) * kLdsRow + 8 * hb;
#pragma unroll
            for (int kk = 0; kk < 16; ++kk) {
                half4_t a;
                const uint2 x = *reinterpret_cast<const uint2*>(kr + 16 * kk);
                __builtin_memcpy(&a, &x, 8);
                acc = __builtin_amdgcn_mfma_f32_32x32x8f16(a, qB[kk], acc, 0, 0, 0);
            }
            sT[blk] = acc;
        }
        const bool need_mask = (j0 + kBN - 1 > wave_first_vis) || (j0 + kBN > kvlen);
        const int64_t vis = p.is_causal ? sp + row : kvlen; // last visible key of this lane's row
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float s = sT[blk][r] * p.score_scale;
                if (need_mask) {
                    const int64_t j = j0 + 32 * blk + 8 * (r >> 2) + 4 * hb + (r & 3);
                    if (j > vis || j >= kvlen) s = -INFINITY;
                }
                sT[blk][r] = s;
            }

        // ---- online softmax for this lane's query row
        float mx = -INFINITY;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sT[blk][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        // key 0 is visible to every row, so m_new is finite from the first tile on; rows past the sequence end have
        // all-zero queries and stay finite as well
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
        half4_t pB[8];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float pe[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    pe[e] = __builtin_amdgcn_exp2f(sT[blk][4 * g + e] - m_new);
                    psum += pe[e];
                }
                pB[4 * blk + g] = half4_t{(half_t)pe[0], (half_t)pe[1], (half_t)pe[2], (half_t)pe[3]};
            }
        l_part = l_part * alpha + psum;
#pragma unroll
        for (int i = 0; i < 4; ++i) oT[i] *= alpha;

        // ---- O^T += V^T * P^T, 8 tokens per MFMA k-block
#pragma unroll
        for (int jb = 0; jb < 8; ++jb) {
            uint2 vr[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                vr[e] = *reinterpret_cast<const uint2*>(lds_v + (8 * jb + 4 * hb + e) * kLdsRow + 8 * n);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
                const uint32_t a01 = __builtin_amdgcn_perm((i < 2) ? vr[1].x : vr[1].y, (i < 2) ? vr[0].x : vr[0].y, sel);
                const uint32_t a23 = __builtin_amdgcn_perm((i < 2) ? vr[3].x : vr[3].y, (i < 2) ? vr[2].x : vr[2].y, sel);
                const uint2 packed = make_uint2(a01, a23);
                half4_t a;
                __builtin_memcpy(&a, &packed, 8);
                oT[i] = __builtin_amdgcn_mfma_f32_32x32x8f16(a, pB[jb], oT[i], 0, 0, 0);
            }
        }
    }

    const float l_tot = l_part + __shfl_xor(l_part, 32);
    if (!row_ok) return;
    const float inv = 1.0f / l_tot;
    // lane (row n, hb) holds, in oT[i][r], channel 4 * (8*(r/4) + 4*hb + r%4) + i
    half_t* op = p.out + ((s0 + row) * p.num_heads + head) * kPDh;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int ch = 4 * (8 * (r >> 2) + 4 * hb + (r & 3));
        const half4_t o = {(half_t)(oT[0][r] * inv), (half_t)(oT[1][r] * inv), (half_t)(oT[2][r] * inv),
                           (half_t)(oT[3][r] * inv)};
        uint2 packed;
        __builtin_memcpy(&packed, &o, 8);
        *reinterpret_cast<uint2*>(op + ch) = packed;
    }
}

pplhip_retcode launch_prefill(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, hipStream_t stream) {
    const int npre = (int)(a->batch - a->decoding_batches);
    if (npre <= 0 || plan->prefill_num_q_tiles <= 0) return PPLHIP_RC_SUCCESS;
    PrefillParams p;
    p.q = (const half_t*)a->d_query;
    p.k = (const half_t*)a->d_current_key;
    p.v = (const half_t*)a->d_current_value;
    p.cache = (const int8_t*)a->d_cache;
    p.scale = (const half_t*)a->d_scale;
    p.seqstarts = a->d_seqstarts;
    p.kvstarts = a->d_kvstarts;
    p.cachestarts = a->d_cachestarts;
    p.start_pos = a->d_start_pos;
    p.out = (half_t*)a->d_output;
    p.addr = CacheAddr{a->cache_stride_s, a->cache_stride_l, a->cache_stride_h, a->cache_stride_kv, a->layer_idx};
    p.first_seq = (int32_t)a->decoding_batches;
    p.num_heads = a->num_heads;
    p.kv_heads = a->num_kv_heads;
    p.rep = a->num_heads / a->num_kv_heads;
    p.is_causal = a->is_causal;
    p.score_scale = 1.4426950408889634f / sqrtf((float)a->head_dim);
    if (npre > 65535) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "prefill: more than 65535 prefill sequences in one call");
    const dim3 grid(plan->prefill_num_q_tiles, a->num_heads, npre);
    if (a->enable_cache_prefill)
        hipLaunchKernelGGL(prefill_attention_kernel<true>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(prefill_attention_kernel<false>, grid, dim3(256), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("prefill_attention");
    return PPLHIP_RC_SUCCESS;
}

} // namespace pplhip
