// Causal prefill attention over ragged packed sequences (flash-attention style, fp16 MFMA, fp32 online softmax).
//
// Roofline: fp16 MFMA. One workgroup (4 wavefronts) owns 128 query rows of one (sequence, query head); each wave
// owns 32 of them. K/V tiles of 64 tokens are staged in LDS once per workgroup and shared by the 4 waves, with the
// next tile's global loads in flight (held in registers) while the current tile is computed; grouped query heads map
// to their kv head by integer division. Everything is computed transposed so that probabilities never leave registers:
//   S^T = K * Q^T    v_mfma_f32_32x32x16_f16, A = K tile from LDS (16 B per lane per MFMA), B = Q^T held in registers
//                    -> lane (n = lane & 31, hb = lane >> 5) owns query row n and kv tokens {8*(r/4) + 4*hb + r%4}
//   O^T += V^T * P^T A = V^T: a lane reads 8 tokens x 4 channels from LDS (row-major, conflict-free) and transposes
//                    them in registers with v_perm; B = P^T is exactly the layout the score registers already have.
// Softmax statistics are per lane column, so rescaling O^T needs no cross-lane traffic; one shuffle per tile
// combines the two half-waves' maxima. Tiles entirely above the causal diagonal are skipped. Workgroups are numbered
// heaviest query tile first across ALL sequences and heads (longest-processing-time order, which keeps the tail of
// the launch short for causal work), and the query heads of one kv head are spaced 8 apart so that they run on the
// same XCD and share its L2 copy of the K/V rows. The output tile goes through LDS so that global stores are full rows.
//
// K/V source: the fp16 current_key/current_value of the sequence (default), or the int8 slab dequantised on the way
// into LDS (cache-prefill: supports start_pos > 0, i.e. chunked prefill / prompt cache).
#include "common.h"

namespace pplhip {

constexpr int kPDh = 128;
constexpr int kBM = 128; // query rows per workgroup
constexpr int kBN = 64; // kv tokens per tile
constexpr int kLdsRow = kPDh * 2 + 16; // bytes per LDS row: 256 B of fp16 + 16 B pad -> 16-byte reads of 8 consecutive
                                       // rows hit distinct banks

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
    int32_t num_seqs; // prefill sequences
    int32_t num_heads, kv_heads, rep;
    int32_t is_causal;
    float score_scale; // log2(e) / sqrt(Dh)
};

// One thread's share of a 64-token K/V tile on its way from global memory to LDS.
template <bool FROM_CACHE>
struct TileRegs;

template <>
struct TileRegs<false> { // fp16 source: 4 rows x 16 B of K and of V per thread
    uint4 k[4], v[4];
};
template <>
struct TileRegs<true> { // int8 slab: 32 channels (+4 scales) of one row of K and of V per thread
    uint4 q[2][2];
    uint2 s[2];
};

__device__ inline void fetch_tile(TileRegs<false>& t, const PrefillParams& p, int64_t j0, int64_t kvlen, int64_t s0,
                                  int64_t, int kvh) {
    const int tid = threadIdx.x, col = tid & 15;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int64_t j = j0 + (tid >> 4) + 16 * pass;
        t.k[pass] = t.v[pass] = make_uint4(0, 0, 0, 0);
        if (j < kvlen) {
            const int64_t off = ((s0 + j) * p.kv_heads + kvh) * kPDh + col * 8;
            t.k[pass] = *reinterpret_cast<const uint4*>(p.k + off);
            t.v[pass] = *reinterpret_cast<const uint4*>(p.v + off);
        }
    }
}
__device__ inline void store_tile(const TileRegs<false>& t, char* lds_k, char* lds_v) {
    const int tid = threadIdx.x, col = tid & 15;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int row = (tid >> 4) + 16 * pass;
        *reinterpret_cast<uint4*>(lds_k + row * kLdsRow + col * 16) = t.k[pass];
        *reinterpret_cast<uint4*>(lds_v + row * kLdsRow + col * 16) = t.v[pass];
    }
}

__device__ inline void fetch_tile(TileRegs<true>& t, const PrefillParams& p, int64_t j0, int64_t kvlen, int64_t,
                                  int64_t tok0, int kvh) {
    const int tid = threadIdx.x, row = tid >> 2, quarter = tid & 3;
    const int64_t j = j0 + row;
#pragma unroll
    for (int kv = 0; kv < 2; ++kv) {
        t.q[kv][0] = t.q[kv][1] = make_uint4(0, 0, 0, 0);
        t.s[kv] = make_uint2(0, 0);
        if (j < kvlen) {
            const int64_t r = p.addr.row(tok0 + j, kv, kvh);
            t.q[kv][0] = *reinterpret_cast<const uint4*>(p.cache + r + quarter * 32);
            t.q[kv][1] = *reinterpret_cast<const uint4*>(p.cache + r + quarter * 32 + 16);
            t.s[kv] = *reinterpret_cast<const uint2*>(p.scale + r / kQuantGroup + quarter * 4);
        }
    }
}
__device__ inline void store_tile(const TileRegs<true>& t, char* lds_k, char* lds_v) {
    const int tid = threadIdx.x, row = tid >> 2, quarter = tid & 3;
#pragma unroll
    for (int kv = 0; kv < 2; ++kv) {
        char* dst = (kv ? lds_v : lds_k) + row * kLdsRow + quarter * 64;
        const uint32_t w[8] = {t.q[kv][0].x, t.q[kv][0].y, t.q[kv][0].z, t.q[kv][0].w,
                               t.q[kv][1].x, t.q[kv][1].y, t.q[kv][1].z, t.q[kv][1].w};
        half_t sc[4];
        __builtin_memcpy(sc, &t.s[kv], 8);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            half_t o[8];
            const float sf = (float)sc[g];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int qi = (int)(int8_t)((w[2 * g + (i >> 2)] >> (8 * (i & 3))) & 0xff);
                o[i] = (half_t)((float)qi * sf);
            }
            uint4 packed;
            __builtin_memcpy(&packed, o, 16);
            *reinterpret_cast<uint4*>(dst + g * 16) = packed;
        }
    }
}

template <bool FROM_CACHE>
__global__ __launch_bounds__(256, 2) void prefill_attention_kernel(const PrefillParams p) {
    __shared__ __attribute__((aligned(16))) char lds_k[kBN * kLdsRow];
    __shared__ __attribute__((aligned(16))) char lds_v[kBN * kLdsRow];

    // ---- which (query tile, sequence, head): heaviest tiles of every sequence and head first
    const int per_tile = p.num_seqs * p.num_heads;
    const int qt_rev = blockIdx.x / per_tile;
    const int rem = blockIdx.x - qt_rev * per_tile;
    const int b = p.first_seq + rem / p.num_heads;
    const int hl = rem % p.num_heads;
    const int kvh = hl % p.kv_heads;
    const int head = kvh * p.rep + hl / p.kv_heads;
    const int64_t s0 = p.seqstarts[b];
    const int64_t L = p.seqstarts[b + 1] - s0;
    const int64_t sp = FROM_CACHE ? p.start_pos[b] : 0;
    const int64_t kvlen = FROM_CACHE ? (p.kvstarts[b + 1] - p.kvstarts[b]) : L;
    const int64_t tok0 = FROM_CACHE ? p.cachestarts[b] : 0;
    const int ntiles = (int)((L + kBM - 1) / kBM);
    const int ntiles_max = gridDim.x / per_tile;
    const int qt = ntiles_max - 1 - qt_rev; // tile index counted from the start of the sequence
    if (qt >= ntiles) return;
    const int64_t q0 = (int64_t)qt * kBM;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 31;
    const int hb = lane >> 5;
    const int64_t row = q0 + 32 * wave + n; // this lane's query row inside the sequence
    const bool row_ok = row < L;

    // keys visible to the last row of this workgroup's tile
    const int64_t last_row = (q0 + kBM < L ? q0 + kBM : L) - 1;
    int64_t kv_end = p.is_causal ? sp + last_row + 1 : kvlen;
    if (kv_end > kvlen) kv_end = kvlen;

    TileRegs<FROM_CACHE> regs;
    fetch_tile(regs, p, 0, kvlen, s0, tok0, kvh);

    // Q^T as the B operand: qB[kk] = Q[row][16*kk + 8*hb .. +7]
    half8_t qB[8];
    {
        const half_t* qp = p.q + ((s0 + (row_ok ? row : 0)) * p.num_heads + head) * kPDh + 8 * hb;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            uint4 x = *reinterpret_cast<const uint4*>(qp + 16 * kk);
            if (!row_ok) x = make_uint4(0, 0, 0, 0);
            __builtin_memcpy(&qB[kk], &x, 16);
        }
    }

    float16_t oT[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oT[i][r] = 0.f;
    float m_run = -INFINITY, l_part = 0.f; // m_run is the running max of the RAW scores (before the exp2 scaling)

    const int64_t wave_last_vis = p.is_causal ? sp + q0 + 32 * wave + 31 : kvlen; // last key any row of this wave sees
    const int64_t wave_first_vis = p.is_causal ? sp + q0 + 32 * wave : kvlen; // keys <= this are seen by all its rows
    const int64_t vis = p.is_causal ? sp + row : kvlen; // last visible key of this lane's row
    const float c = p.score_scale;

    for (int64_t j0 = 0; j0 < kv_end; j0 += kBN) {
        __syncthreads(); // every wave is done reading the previous tile
        store_tile(regs, lds_k, lds_v);
        __syncthreads();
        if (j0 + kBN < kv_end) fetch_tile(regs, p, j0 + kBN, kvlen, s0, tok0, kvh); // in flight during the compute
        if (j0 > wave_last_vis) continue; // the whole tile is above this wave's diagonal (wave-uniform)

        // ---- S^T tiles: 2 x (32 kv tokens x 32 query rows)
        float16_t sT[2];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            float16_t acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
            const char* kr = lds_k + (32 * blk + n) * kLdsRow + 16 * hb;
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                half8_t a;
                const uint4 x = *reinterpret_cast<const uint4*>(kr + 32 * kk);
                __builtin_memcpy(&a, &x, 16);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qB[kk], acc, 0, 0, 0);
            }
            sT[blk] = acc;
        }
        const bool need_mask = (j0 + kBN - 1 > wave_first_vis) || (j0 + kBN > kvlen);
        if (need_mask) {
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t j = j0 + 32 * blk + 8 * (r >> 2) + 4 * hb + (r & 3);
                    if (j > vis || j >= kvlen) sT[blk][r] = -INFINITY;
                }
        }

        // ---- online softmax for this lane's query row: p = exp2(s*c - m*c), one fma + one exp2 per score
        float mx = -INFINITY;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sT[blk][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        // key 0 is visible to every row, so m_new is finite from the first tile on; rows past the sequence end have
        // all-zero queries and stay finite as well
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c);
        m_run = m_new;
        const float neg_mc = -m_new * c;
        float psum = 0.f;
        half8_t pB[4]; // pB[2*blk + J]: k-slot e8 <-> token 32*blk + 16*J + 8*(e8/4) + 4*hb + e8%4
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int J = 0; J < 2; ++J) {
                float pe[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    pe[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sT[blk][8 * J + e], c, neg_mc));
                    psum += pe[e];
                }
                pB[2 * blk + J] = half8_t{(half_t)pe[0], (half_t)pe[1], (half_t)pe[2], (half_t)pe[3],
                                          (half_t)pe[4], (half_t)pe[5], (half_t)pe[6], (half_t)pe[7]};
            }
        l_part = l_part * alpha + psum;
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int i = 0; i < 4; ++i) oT[i] *= alpha;
        }

        // ---- O^T += V^T * P^T, 16 tokens per MFMA k-block
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            uint2 vr[8]; // vr[e8]: channels 4n .. 4n+3 of token 16*kb + 8*(e8/4) + 4*hb + e8%4
#pragma unroll
            for (int e = 0; e < 8; ++e)
                vr[e] = *reinterpret_cast<const uint2*>(lds_v + (16 * kb + 8 * (e >> 2) + 4 * hb + (e & 3)) * kLdsRow + 8 * n);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
                uint32_t t[4];
#pragma unroll
                for (int pr = 0; pr < 4; ++pr)
                    t[pr] = __builtin_amdgcn_perm((i < 2) ? vr[2 * pr + 1].x : vr[2 * pr + 1].y,
                                                  (i < 2) ? vr[2 * pr].x : vr[2 * pr].y, sel);
                half8_t a;
                __builtin_memcpy(&a, t, 16);
                oT[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pB[kb], oT[i], 0, 0, 0);
            }
        }
    }

    const float l_tot = l_part + __shfl_xor(l_part, 32);
    const float inv = 1.0f / l_tot;
    // ---- output through LDS: each wave parks its 32 x 128 fp16 tile in its own 32 rows, then writes full rows
    __syncthreads(); // all waves are done with the last K/V tile
    char* otile = (wave < 2 ? lds_k : lds_v) + (wave & 1) * 32 * kLdsRow;
    // lane (row n, hb) holds, in oT[i][r], channel 4 * (8*(r/4) + 4*hb + r%4) + i
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int ch = 4 * (8 * (r >> 2) + 4 * hb + (r & 3));
        const half4_t o = {(half_t)(oT[0][r] * inv), (half_t)(oT[1][r] * inv), (half_t)(oT[2][r] * inv),
                           (half_t)(oT[3][r] * inv)};
        uint2 packed;
        __builtin_memcpy(&packed, &o, 8);
        *reinterpret_cast<uint2*>(otile + n * kLdsRow + ch * 2) = packed;
    }
    // (same wave wrote and reads: no workgroup barrier needed, the compiler orders the LDS accesses)
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
        const int rr = 4 * pass + (lane >> 4); // row of the wave's tile
        const int64_t orow = q0 + 32 * wave + rr;
        const uint4 x = *reinterpret_cast<const uint4*>(otile + rr * kLdsRow + (lane & 15) * 16);
        if (orow < L)
            *reinterpret_cast<uint4*>(p.out + ((s0 + orow) * p.num_heads + head) * kPDh + (lane & 15) * 8) = x;
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
    p.num_seqs = npre;
    const int64_t blocks = (int64_t)plan->prefill_num_q_tiles * npre * a->num_heads;
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "prefill: too many query tiles in one call");
    const dim3 grid((unsigned)blocks);
    if (a->enable_cache_prefill)
        hipLaunchKernelGGL(prefill_attention_kernel<true>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(prefill_attention_kernel<false>, grid, dim3(256), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("prefill_attention");
    return PPLHIP_RC_SUCCESS;
}

} // namespace pplhip
