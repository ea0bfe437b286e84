// Decode attention over the int8 group-8 KV slab (one new token per sequence), split along the cached tokens.
//
// Roofline: HBM. Each cached token costs 2 * KVH * (Dh + Dh/4) bytes and is read exactly once; arithmetic
// intensity is 1.6 .. 12.8 flop/B, so the kernel is organised around streaming bytes, and the contraction is put
// on the matrix cores only so that dequantisation + FMA work does not become the limiter for grouped-query shapes.
//
// Work decomposition: one *wavefront task* = (sequence b, kv head, chunk of `chunk` cached tokens). All H/KVH query
// heads that share the kv head ride in the 16-wide N dimension of v_mfma_f32_16x16x16_f16, so every KV byte is
// loaded once per task. Waves are independent (no LDS, no barriers); a workgroup is just 4 adjacent tasks, ordered
// so that its waves read adjacent kv heads of the same tokens (contiguous bytes in the (MaxT, L, 2, KVH, Dh) slab).
//
// Per 16-token block a lane (m = lane & 15, kq = lane >> 4) does:
//   S^T = K_hat * Q^T   A = K_hat[token m][channels 64*jj + 16*kq + 4*i .. +3]   (two 16 B loads per lane per block)
//                       B = Q^T, held in registers for the whole task
//         -> lane holds scores of head m for tokens 4*kq .. 4*kq+3
//   O^T += V_hat^T * P^T  A = V_hat^T[channel 8*m + i][tokens 4*kq .. +3]         (four 8 B loads per lane per block,
//                       transposed in registers with v_perm), B = P^T straight from the score registers
// int8 -> fp16 is exact: (x ^ 0x80) placed under exponent byte 0x64 reads as 1024 + (x + 128); subtract 1152, then
// multiply by the group's fp16 scale (packed fp16 ops). Softmax runs online in the exp2 domain with fp32 statistics.
//
// Each task writes an un-normalised partial (max, sum, acc[Dh]) per query head into the workspace and
// `decode_merge_kernel` combines the chunks of a sequence with the usual log-sum-exp weights. With a single chunk the
// task normalises and writes fp16 output itself.
#include "common.h"

namespace pplhip {

constexpr int kDh = 128; // head_dim this kernel is specialised for
constexpr int kDecodeWaves = 4;
constexpr int kIterTokens = 64; // tokens per softmax update (4 MFMA sub-blocks of 16)

struct DecodeParams {
    const half_t* q; // [S, H, Dh]
    const int8_t* cache;
    const half_t* scale;
    const int64_t* seqstarts;
    const int64_t* kvstarts;
    const int64_t* cachestarts;
    half_t* out; // [S, H, Dh]
    float* part_acc; // [nd, chunks, H, Dh]
    float* part_ml; // [nd, chunks, H, 2]
    CacheAddr addr;
    int32_t nd; // decode sequences
    int32_t num_heads, kv_heads, rep; // rep = num_heads / kv_heads (<= 16)
    int32_t chunk, num_chunks;
    int64_t total_tasks;
    float score_scale; // log2(e) / sqrt(Dh)
};

__device__ inline half2_t as_half2(uint32_t u) {
    half2_t h;
    __builtin_memcpy(&h, &u, 4);
    return h;
}
__device__ inline uint32_t as_u32(half2_t h) {
    uint32_t u;
    __builtin_memcpy(&u, &h, 4);
    return u;
}

// bytes 0,1 (lo) or 2,3 (hi) of x, each widened to an fp16 bit pattern 0x64bb = 1024 + b
__device__ inline uint32_t widen_lo(uint32_t x) {
    return __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u);
}
__device__ inline uint32_t widen_hi(uint32_t x) {
    return __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);
}
// (1024 + (q + 128)) - 1152 = q exactly; times the group scale, rounded to fp16
__device__ inline half2_t dequant2(uint32_t widened, half2_t s2) {
    const half2_t bias = {(half_t)1152.0f, (half_t)1152.0f};
    return (as_half2(widened) - bias) * s2;
}

__device__ inline float wave_max_over_quads(float v) {
    v = fmaxf(v, __shfl_xor(v, 16));
    v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}
__device__ inline float wave_sum_over_quads(float v) {
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

__global__ __launch_bounds__(kDecodeWaves* kWave, 2) void decode_int8kv_kernel(const DecodeParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t task = (int64_t)blockIdx.x * kDecodeWaves + (threadIdx.x >> 6);
    if (task >= p.total_tasks) return;
    const int kvh = (int)(task % p.kv_heads);
    const int64_t bc = task / p.kv_heads;
    const int c = (int)(bc % p.num_chunks);
    const int b = (int)(bc / p.num_chunks);
    const int64_t kvlen = p.kvstarts[b + 1] - p.kvstarts[b];
    const int64_t t_begin = (int64_t)c * p.chunk;
    if (t_begin >= kvlen) return; // this sequence has fewer chunks; the merge pass never looks here
    const int64_t t_end = (t_begin + p.chunk < kvlen) ? t_begin + p.chunk : kvlen;
    const int64_t tok0 = p.cachestarts[b];
    const int64_t qrow = p.seqstarts[b];

    const int m = lane & 15;
    const int kq = lane >> 4;

    // ---- Q^T as the B operand, kept for the whole task: qB[jj][i] = Q[head m][64*jj + 16*kq + 4*i .. +3]
    half4_t qB[2][4];
    {
        const bool live = m < p.rep;
        const half_t* qp = p.q + ((qrow * p.num_heads) + (int64_t)kvh * p.rep + (live ? m : 0)) * kDh;
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            uint4 lo = *reinterpret_cast<const uint4*>(qp + 64 * jj + 16 * kq);
            uint4 hi = *reinterpret_cast<const uint4*>(qp + 64 * jj + 16 * kq + 8);
            if (!live) lo = hi = make_uint4(0, 0, 0, 0);
            half4_t tmp[4];
            __builtin_memcpy(&tmp[0], &lo, 16);
            __builtin_memcpy(&tmp[2], &hi, 16);
#pragma unroll
            for (int i = 0; i < 4; ++i) qB[jj][i] = tmp[i];
        }
    }

    const int8_t* kbase = p.cache + p.addr.row(tok0, 0, kvh);
    const int8_t* vbase = p.cache + p.addr.row(tok0, 1, kvh);
    const half_t* ksbase = p.scale + p.addr.row(tok0, 0, kvh) / kQuantGroup;
    const half_t* vsbase = p.scale + p.addr.row(tok0, 1, kvh) / kQuantGroup;
    const int64_t stride = p.addr.stride_s;
    const int64_t sstride = p.addr.stride_s / kQuantGroup;

    float4_t oacc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) oacc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY; // running max of head m (same value in the 4 lanes that share m)
    float l_part = 0.f; // this lane's share of the running sum

    const int64_t last_tok = t_end - 1;
    for (int64_t t0 = t_begin; t0 < t_end; t0 += kIterTokens) {
        // ---- issue all loads of this iteration (rows past the chunk end are clamped to its last row and masked)
        uint4 kraw[4][2];
        uint32_t ksc[4][2];
        uint2 vraw[4][4];
        half_t vsc[4][4];
#pragma unroll
        for (int sb = 0; sb < 4; ++sb) {
            int64_t tk = t0 + 16 * sb + m;
            tk = tk < last_tok ? tk : last_tok;
            const int8_t* kr = kbase + tk * stride;
            const half_t* ks = ksbase + tk * sstride;
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                kraw[sb][jj] = *reinterpret_cast<const uint4*>(kr + 64 * jj + 16 * kq);
                ksc[sb][jj] = *reinterpret_cast<const uint32_t*>(ks + 8 * jj + 2 * kq);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                int64_t tv = t0 + 16 * sb + 4 * kq + e;
                tv = tv < last_tok ? tv : last_tok;
                vraw[sb][e] = *reinterpret_cast<const uint2*>(vbase + tv * stride + 8 * m);
                vsc[sb][e] = vsbase[tv * sstride + m];
            }
        }

        // ---- scores: S^T[token, head] for 4 sub-blocks of 16 tokens
        float4_t st[4];
#pragma unroll
        for (int sb = 0; sb < 4; ++sb) {
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const uint32_t w[4] = {kraw[sb][jj].x, kraw[sb][jj].y, kraw[sb][jj].z, kraw[sb][jj].w};
                const half2_t sc = as_half2(ksc[sb][jj]);
                const half2_t s_lo = {sc.x, sc.x};
                const half2_t s_hi = {sc.y, sc.y};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t x = w[i] ^ 0x80808080u;
                    const half2_t s2 = (i < 2) ? s_lo : s_hi;
                    const half2_t a01 = dequant2(widen_lo(x), s2);
                    const half2_t a23 = dequant2(widen_hi(x), s2);
                    const half4_t a = {a01.x, a01.y, a23.x, a23.y};
                    acc = __builtin_amdgcn_mfma_f32_16x16x16f16(a, qB[jj][i], acc, 0, 0, 0);
                }
            }
            // lane now holds head m, tokens t0 + 16*sb + 4*kq + e
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t tk = t0 + 16 * sb + 4 * kq + e;
                acc[e] = (tk < t_end) ? acc[e] * p.score_scale : -INFINITY;
            }
            st[sb] = acc;
        }

        // ---- online softmax update (per head = per lane column m)
        float mx = -INFINITY;
#pragma unroll
        for (int sb = 0; sb < 4; ++sb)
#pragma unroll
            for (int e = 0; e < 4; ++e) mx = fmaxf(mx, st[sb][e]);
        mx = wave_max_over_quads(mx);
        const float m_new = fmaxf(m_run, mx); // finite: the first token of every iteration is inside the chunk
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
        half4_t pB[4];
#pragma unroll
        for (int sb = 0; sb < 4; ++sb) {
            float pe[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                pe[e] = __builtin_amdgcn_exp2f(st[sb][e] - m_new);
                psum += pe[e];
            }
            pB[sb] = half4_t{(half_t)pe[0], (half_t)pe[1], (half_t)pe[2], (half_t)pe[3]};
        }
        l_part = l_part * alpha + psum;
#pragma unroll
        for (int i = 0; i < 8; ++i) oacc[i] *= alpha;

        // ---- O^T[channel, head] += V_hat^T * P^T
#pragma unroll
        for (int sb = 0; sb < 4; ++sb) {
            half2_t d[4][4]; // [token e][channel pair c] dequantised, channels 8*m + 2c, 2c+1
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const half2_t s2 = {vsc[sb][e], vsc[sb][e]};
                const uint32_t x0 = vraw[sb][e].x ^ 0x80808080u;
                const uint32_t x1 = vraw[sb][e].y ^ 0x80808080u;
                d[e][0] = dequant2(widen_lo(x0), s2);
                d[e][1] = dequant2(widen_hi(x0), s2);
                d[e][2] = dequant2(widen_lo(x1), s2);
                d[e][3] = dequant2(widen_hi(x1), s2);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int cpair = i >> 1;
                const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
                const uint32_t t01 = __builtin_amdgcn_perm(as_u32(d[1][cpair]), as_u32(d[0][cpair]), sel);
                const uint32_t t23 = __builtin_amdgcn_perm(as_u32(d[3][cpair]), as_u32(d[2][cpair]), sel);
                const half2_t h01 = as_half2(t01), h23 = as_half2(t23);
                const half4_t a = {h01.x, h01.y, h23.x, h23.y};
                oacc[i] = __builtin_amdgcn_mfma_f32_16x16x16f16(a, pB[sb], oacc[i], 0, 0, 0);
            }
        }
    }

    const float l_tot = wave_sum_over_quads(l_part);
    if (m >= p.rep) return;
    const int head = kvh * p.rep + m;
    // lane (head m, r = kq) holds channels 8*(4*r + e) + i in oacc[i][e]
    if (p.num_chunks == 1) {
        const float inv = 1.0f / l_tot;
        half_t* op = p.out + (qrow * p.num_heads + head) * kDh;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            half_t o[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = (half_t)(oacc[i][e] * inv);
            uint4 packed;
            __builtin_memcpy(&packed, o, 16);
            *reinterpret_cast<uint4*>(op + 8 * (4 * kq + e)) = packed;
        }
    } else {
        const int64_t prow = ((int64_t)b * p.num_chunks + c) * p.num_heads + head;
        float* pa = p.part_acc + prow * kDh;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float4_t lo = {oacc[0][e], oacc[1][e], oacc[2][e], oacc[3][e]};
            const float4_t hi = {oacc[4][e], oacc[5][e], oacc[6][e], oacc[7][e]};
            *reinterpret_cast<float4_t*>(pa + 8 * (4 * kq + e)) = lo;
            *reinterpret_cast<float4_t*>(pa + 8 * (4 * kq + e) + 4) = hi;
        }
        if (kq == 0) {
            p.part_ml[prow * 2 + 0] = m_run;
            p.part_ml[prow * 2 + 1] = l_tot;
        }
    }
}

// One workgroup of 128 lanes per (decode sequence, query head): out[d] = sum_c w_c acc_c[d] / sum_c w_c l_c,
// w_c = exp2(m_c - max_c m_c), over the chunks the sequence really has.
__global__ __launch_bounds__(kDh) void decode_merge_kernel(const DecodeParams p) {
    const int b = blockIdx.y;
    const int head = blockIdx.x;
    const int d = threadIdx.x;
    const int64_t kvlen = p.kvstarts[b + 1] - p.kvstarts[b];
    const int nc = (int)((kvlen + p.chunk - 1) / p.chunk);
    const int64_t base = (int64_t)b * p.num_chunks * p.num_heads + head;
    float mx = -INFINITY;
    for (int c = 0; c < nc; ++c) mx = fmaxf(mx, p.part_ml[(base + (int64_t)c * p.num_heads) * 2]);
    float acc = 0.f, l = 0.f;
    for (int c = 0; c < nc; ++c) {
        const int64_t prow = base + (int64_t)c * p.num_heads;
        const float w = __builtin_amdgcn_exp2f(p.part_ml[prow * 2] - mx);
        l += w * p.part_ml[prow * 2 + 1];
        acc += w * p.part_acc[prow * kDh + d];
    }
    p.out[(p.seqstarts[b] * p.num_heads + head) * kDh + d] = (half_t)(acc / l);
}

pplhip_retcode launch_decode(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* ws, hipStream_t stream) {
    const int nd = (int)a->decoding_batches;
    if (nd == 0) return PPLHIP_RC_SUCCESS;
    DecodeParams p;
    p.q = (const half_t*)a->d_query;
    p.cache = (const int8_t*)a->d_cache;
    p.scale = (const half_t*)a->d_scale;
    p.seqstarts = a->d_seqstarts;
    p.kvstarts = a->d_kvstarts;
    p.cachestarts = a->d_cachestarts;
    p.out = (half_t*)a->d_output;
    p.addr = CacheAddr{a->cache_stride_s, a->cache_stride_l, a->cache_stride_h, a->cache_stride_kv, a->layer_idx};
    p.nd = nd;
    p.num_heads = a->num_heads;
    p.kv_heads = a->num_kv_heads;
    p.rep = a->num_heads / a->num_kv_heads;
    p.chunk = plan->decode_chunk_tokens;
    p.num_chunks = plan->decode_num_chunks;
    p.total_tasks = (int64_t)nd * p.num_chunks * p.kv_heads;
    p.score_scale = 1.4426950408889634f / sqrtf((float)a->head_dim);
    const size_t acc_bytes = (size_t)nd * p.num_chunks * p.num_heads * kDh * sizeof(float);
    p.part_acc = (float*)ws;
    p.part_ml = (float*)((char*)ws + acc_bytes);
    if (p.num_chunks > 1 && ws == nullptr)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "decode: split-k needs the workspace reported by pplhip_mhca_prepare");
    const int64_t blocks = (p.total_tasks + kDecodeWaves - 1) / kDecodeWaves;
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "decode: too many tasks");
    hipLaunchKernelGGL(decode_int8kv_kernel, dim3((unsigned)blocks), dim3(kDecodeWaves * kWave), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("decode_int8kv");
    if (p.num_chunks > 1) {
        hipLaunchKernelGGL(decode_merge_kernel, dim3(p.num_heads, nd), dim3(kDh), 0, stream, p);
        PPLHIP_CHECK_LAUNCH("decode_merge");
    }
    return PPLHIP_RC_SUCCESS;
}

} // namespace pplhip
