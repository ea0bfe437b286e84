// Causal prefill attention over ragged packed sequences (flash-attention style, fp16 MFMA, fp32 online softmax).
//
// Roofline: fp16 MFMA. One workgroup (4 wavefronts) owns 128 query rows of one (sequence, query head); each wave
// owns 32 of them. K/V tiles of 64 tokens are staged in LDS once per workgroup and shared by the 4 waves; grouped query
// heads map to their kv head by integer division. Everything is computed transposed so that probabilities never leave
// registers:
//   S^T = K * Q^T    v_mfma_f32_32x32x16_f16, A = K tile from LDS (16 B per lane per MFMA), B = Q^T held in registers
//                    -> lane (n = lane & 31, hb = lane >> 5) owns query row n and kv tokens {8*(r/4) + 4*hb + r%4}
//   O^T += V^T * P^T A = V^T from LDS, B = P^T, which is exactly the layout the score registers already have.
// Softmax statistics are per lane column, so rescaling O^T needs no cross-lane traffic. The reference maximum of a row
// is only moved when the running maximum has outgrown it by more than 2^kRescaleLog2 (probabilities then stay below
// that factor, well inside fp16), which removes the accumulator rescale from almost every tile. Tiles entirely above
// the causal diagonal are skipped. Workgroups are numbered heaviest query tile first across ALL sequences and heads
// (longest-processing-time order, which keeps the tail of the launch short for causal work), and the query heads of
// one kv head are spaced 8 apart so that they run on the same XCD and share its L2 copy of the K/V rows. The output
// tile goes through LDS so that global stores are full rows.
//
// Two kernels:
//   prefill_workgroup / prefill_f16_kernel   K/V are fp16 rows (current_key / current_value, MultiHeadAttention's
//       key / value, or the staged rows of a cache-prefill call): tiles travel global -> LDS by DMA, unpadded and
//       swizzled; V stays row-major and its transposed operands come from ds_read_b64_tr_b16; the scores of tile t+1
//       are issued between the exponentials of tile t. Its grid also carries the workgroups that quantise the prompt
//       tokens into the slab.
//   prefill_attention_kernel<true>            K/V are the int8 slab (cache-prefill with small chunks): the next
//       tile's global loads are held in registers while the current tile is computed, and are dequantised -- V also
//       transposed (4 tokens x 8 channels per thread, v_perm) -- on their way into LDS.
#include "common.h"

namespace pplhip {

constexpr int kPDh = 128;
constexpr int kBM = 128; // query rows per workgroup
constexpr int kBN = 64; // kv tokens per tile
constexpr int kLdsRow = kPDh * 2 + 16; // bytes per K row in LDS: 256 B of fp16 + 16 B pad -> 16-byte reads of 16
                                       // consecutive rows hit distinct banks
constexpr int kVtRow = kBN * 2 + 16; // bytes per V^T row (one channel, 64 token positions) + 16 B pad
constexpr int kLdsKBytes = kBN * kLdsRow; // 17408
constexpr int kLdsVBytes = kPDh * kVtRow; // 18432
constexpr int kLdsBufBytes = kLdsKBytes + kLdsVBytes; // one K/V tile
constexpr float kRescaleLog2 = 8.0f;

struct PrefillParams {
    const half_t* q;
    const half_t* k;
    const half_t* v;
    const int8_t* cache;
    const half_t* scale;
    const int64_t* seqstarts;
    const int64_t* kvstarts;
    PageMap pages; // cache source only
    const int64_t* start_pos;
    half_t* out;
    CacheAddr addr;
    int32_t first_seq; // = decoding_batches
    int32_t num_seqs; // prefill sequences
    int32_t num_heads, kv_heads, rep;
    int32_t is_causal;
    float score_scale; // log2(e) / sqrt(Dh)
    // quantize-on-write of the prompt tokens, done by this launch (prefill_f16_kernel only; w_cache null: not)
    int8_t* w_cache;
    half_t* w_scale;
    int64_t w_first_token, w_end_token; // packed new tokens [first, end)
    int32_t w_batch; // all sequences of the call (the sequence of a token is looked up in seqstarts)
    int32_t w_per_tok; // 4-group units per token: 2 * kv_heads * 4
    const int64_t* kv_origin; // null, or the packed kv-token index that row 0 of k / v holds (device scalar)
    int32_t attn_blocks; // workgroups [0, attn_blocks) map to query tiles; the ones behind them only write tokens
    int32_t ntiles_max; // query tiles of the longest sequence allowed (from max_seqlen)
    int32_t compact; // the grid has one workgroup per possible tile instead of per (level, sequence): see the kernel
};

// A thread's share of a 64-token K/V tile: channels 8*col .. 8*col+7 (col = tid & 15) of the four consecutive tokens
// 4*r0 .. 4*r0+3 (r0 = tid >> 4). A wave's load instruction covers four full 256-byte rows.
template <bool FROM_CACHE>
struct TileRegs;

template <>
struct TileRegs<false> { // fp16 source
    uint4 k[4], v[4];
};
template <>
struct TileRegs<true> { // int8 slab: 8 bytes + one fp16 scale per token for K and for V (8 channels = one quant group)
    uint2 kq[4], vq[4];
    uint16_t ks[4], vs[4];
};

// Pins a pointer that is wave-uniform by construction into scalar registers, so that memory instructions take the
// "scalar base + 32-bit lane offset" addressing form. The integer round trip loses the pointer's address space, so the
// result is typed as a global-memory pointer explicitly: loads through a generic pointer become flat_load, which
// counts on the LDS counter as well, and every wait for an LDS read would then also wait for the tile prefetch.
typedef const char __attribute__((address_space(1))) * gptr_t;
__device__ inline gptr_t uniform_ptr(const char* p) {
    const uint64_t u = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return reinterpret_cast<gptr_t>(((uint64_t)hi << 32) | lo);
}
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
__device__ inline uint4 gload16(gptr_t p) {
    const u32x4_t x = *reinterpret_cast<const u32x4_t __attribute__((address_space(1)))*>(p);
    return make_uint4(x[0], x[1], x[2], x[3]);
}
__device__ inline uint2 gload8(gptr_t p) {
    const u32x2_t x = *reinterpret_cast<const u32x2_t __attribute__((address_space(1)))*>(p);
    return make_uint2(x[0], x[1]);
}
__device__ inline uint16_t gload2(gptr_t p) {
    return *reinterpret_cast<const uint16_t __attribute__((address_space(1)))*>(p);
}

// Where a workgroup's K/V rows come from. Token j of the sequence is at (uniform base) + j * row_bytes, and a
// thread's piece of the row it fetches in pass p of tile j0 is at base + (j0 + p) * row_bytes + voff, voff fixed for
// the whole kernel: all per-tile address arithmetic is scalar.
template <bool FROM_CACHE>
struct TileSrc;
template <>
struct TileSrc<false> {
    const char* k; // current_key / current_value row of token 0 of the sequence, this kv head
    const char* v;
    uint32_t row_bytes;
    uint32_t voff; // 4 * r0 rows + 16 * col bytes
};
template <>
struct TileSrc<true> {
    const char* k; // slab rows of slab token 0 (this layer, K / V, this kv head)
    const char* v;
    const char* ks; // their scale rows
    const char* vs;
    const int64_t* page_row; // cache_mode 1: the sequence's row of the page table; cache_mode 0: null
    int64_t tok0; // cache_mode 0: first slab token of the sequence
    int32_t page_shift;
    uint32_t row_bytes, srow_bytes;
    uint32_t voff, svoff;
    // slab token of sequence token j0, the first of a 64-token tile: tiles never straddle a page (pages are powers of
    // two >= 64 tokens and tiles start at multiples of 64)
    __device__ inline int64_t tile_token(int64_t j0) const {
        if (page_shift == 0) return tok0 + j0;
        return page_row[j0 >> page_shift] + (j0 & ((int64_t(1) << page_shift) - 1));
    }
};

__device__ inline void fetch_tile(TileRegs<false>& t, const TileSrc<false>& src, int64_t j0, int64_t kvlen) {
    const int r0 = threadIdx.x >> 4;
    if (j0 + kBN <= kvlen) { // whole tile inside the sequence (wave-uniform)
        const gptr_t kb = uniform_ptr(src.k + j0 * src.row_bytes);
        const gptr_t vb = uniform_ptr(src.v + j0 * src.row_bytes);
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            t.k[pass] = gload16(kb + pass * src.row_bytes + src.voff);
            t.v[pass] = gload16(vb + pass * src.row_bytes + src.voff);
        }
    } else { // last, partial tile: rows past the end read as zero
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int64_t j = j0 + 4 * r0 + pass;
            t.k[pass] = t.v[pass] = make_uint4(0, 0, 0, 0);
            if (j < kvlen) {
                const int64_t off = (j0 + pass) * src.row_bytes + src.voff;
                t.k[pass] = *reinterpret_cast<const uint4*>(src.k + off);
                t.v[pass] = *reinterpret_cast<const uint4*>(src.v + off);
            }
        }
    }
}

__device__ inline void fetch_tile(TileRegs<true>& t, const TileSrc<true>& src, int64_t j0, int64_t kvlen) {
    const int r0 = threadIdx.x >> 4;
    const int64_t tok = src.tile_token(j0);
    const gptr_t kb = uniform_ptr(src.k + tok * src.row_bytes);
    const gptr_t vb = uniform_ptr(src.v + tok * src.row_bytes);
    const gptr_t ksb = uniform_ptr(src.ks + tok * src.srow_bytes);
    const gptr_t vsb = uniform_ptr(src.vs + tok * src.srow_bytes);
    if (j0 + kBN <= kvlen) {
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            t.kq[pass] = gload8(kb + pass * src.row_bytes + src.voff);
            t.vq[pass] = gload8(vb + pass * src.row_bytes + src.voff);
            t.ks[pass] = gload2(ksb + pass * src.srow_bytes + src.svoff);
            t.vs[pass] = gload2(vsb + pass * src.srow_bytes + src.svoff);
        }
    } else {
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int64_t j = j0 + 4 * r0 + pass;
            t.kq[pass] = t.vq[pass] = make_uint2(0, 0);
            t.ks[pass] = t.vs[pass] = 0;
            if (j < kvlen) {
                t.kq[pass] = gload8(kb + pass * src.row_bytes + src.voff);
                t.vq[pass] = gload8(vb + pass * src.row_bytes + src.voff);
                t.ks[pass] = gload2(ksb + pass * src.srow_bytes + src.svoff);
                t.vs[pass] = gload2(vsb + pass * src.srow_bytes + src.svoff);
            }
        }
    }
}

__device__ inline TileSrc<false> make_tile_src_f16(const PrefillParams& p, int64_t s0, int kvh) {
    TileSrc<false> src;
    const int tid = threadIdx.x, col = tid & 15, r0 = tid >> 4;
    src.row_bytes = (uint32_t)p.kv_heads * kPDh * 2;
    const int64_t first = (s0 * p.kv_heads + kvh) * kPDh * 2;
    src.k = reinterpret_cast<const char*>(p.k) + first;
    src.v = reinterpret_cast<const char*>(p.v) + first;
    src.voff = 4 * r0 * src.row_bytes + col * 16;
    return src;
}
__device__ inline TileSrc<true> make_tile_src_cache(const PrefillParams& p, int b, int kvh) {
    TileSrc<true> src;
    const int tid = threadIdx.x, col = tid & 15, r0 = tid >> 4;
    const int64_t rk = p.addr.row(0, 0, kvh), rv = p.addr.row(0, 1, kvh);
    src.row_bytes = (uint32_t)p.addr.stride_s; // int8: one byte per element
    src.srow_bytes = src.row_bytes / kQuantGroup * 2;
    src.k = reinterpret_cast<const char*>(p.cache) + rk;
    src.v = reinterpret_cast<const char*>(p.cache) + rv;
    src.ks = reinterpret_cast<const char*>(p.scale) + rk / kQuantGroup * 2;
    src.vs = reinterpret_cast<const char*>(p.scale) + rv / kQuantGroup * 2;
    src.page_shift = p.pages.page_shift;
    src.page_row = p.pages.page_shift ? p.pages.cachestarts + (int64_t)b * p.pages.stride_b : nullptr;
    src.tok0 = p.pages.page_shift ? 0 : p.pages.cachestarts[b];
    src.voff = 4 * r0 * src.row_bytes + col * 8;
    src.svoff = 4 * r0 * src.srow_bytes + col * 2;
    return src;
}

// 8 int8 values times one fp16 scale -> 8 fp16 values (the product is rounded once, as in the decode kernel's
// dequantisation: |q| <= 128 is exact in fp16 and so is the fp32 product before the final rounding)
__device__ inline uint4 dequant8(uint2 q, uint16_t scale_bits) {
    half_t sc;
    __builtin_memcpy(&sc, &scale_bits, 2);
    const float sf = (float)sc;
    const uint32_t w[2] = {q.x, q.y};
    half_t o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int qi = (int)(int8_t)((w[i >> 2] >> (8 * (i & 3))) & 0xff);
        o[i] = (half_t)((float)qi * sf);
    }
    uint4 packed;
    __builtin_memcpy(&packed, o, 16);
    return packed;
}

// K rows go to LDS as they are; V is transposed: row = channel, and token t of the tile sits at position
// (t with bits 2 and 3 swapped), 16-byte chunks XOR-swizzled by row / 16 so that both these 8-byte writes and the
// 16-byte reads of the PV step spread over all banks.
__device__ inline void store_kv(const uint4 (&kr)[4], const uint4 (&vr)[4], char* lds_k, char* lds_vt) {
    const int tid = threadIdx.x, col = tid & 15, r0 = tid >> 4;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass)
        *reinterpret_cast<uint4*>(lds_k + (4 * r0 + pass) * kLdsRow + col * 16) = kr[pass];
    const int chunk = (2 * (r0 >> 2) + (r0 & 1)) ^ (col >> 1); // (position * 2 / 16) ^ (row / 16), row / 16 = col / 2
    char* dst = lds_vt + (8 * col) * kVtRow + chunk * 16 + 8 * ((r0 >> 1) & 1);
    const uint32_t a[4][4] = {{vr[0].x, vr[0].y, vr[0].z, vr[0].w},
                              {vr[1].x, vr[1].y, vr[1].z, vr[1].w},
                              {vr[2].x, vr[2].y, vr[2].z, vr[2].w},
                              {vr[3].x, vr[3].y, vr[3].z, vr[3].w}};
#pragma unroll
    for (int m = 0; m < 4; ++m) { // dword m of a token = channels 2m, 2m+1
        uint2 lo, hi;
        lo.x = __builtin_amdgcn_perm(a[1][m], a[0][m], 0x05040100u);
        lo.y = __builtin_amdgcn_perm(a[3][m], a[2][m], 0x05040100u);
        hi.x = __builtin_amdgcn_perm(a[1][m], a[0][m], 0x07060302u);
        hi.y = __builtin_amdgcn_perm(a[3][m], a[2][m], 0x07060302u);
        *reinterpret_cast<uint2*>(dst + (2 * m) * kVtRow) = lo;
        *reinterpret_cast<uint2*>(dst + (2 * m + 1) * kVtRow) = hi;
    }
}
__device__ inline void store_tile(const TileRegs<false>& t, char* lds_k, char* lds_vt) {
    store_kv(t.k, t.v, lds_k, lds_vt);
}
__device__ inline void store_tile(const TileRegs<true>& t, char* lds_k, char* lds_vt) {
    uint4 kr[4], vr[4];
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        kr[pass] = dequant8(t.kq[pass], t.ks[pass]);
        vr[pass] = dequant8(t.vq[pass], t.vs[pass]);
    }
    store_kv(kr, vr, lds_k, lds_vt);
}

// the value the lane 32 positions away holds (the two half-waves of a query column exchange partial results)
__device__ inline float other_half(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    // lower lanes: r[1] holds the upper half's value; upper lanes: r[0] holds the lower half's value
    return (threadIdx.x & 32) ? __uint_as_float(r[0]) : __uint_as_float(r[1]);
}

template <bool FROM_CACHE>
__global__ __launch_bounds__(256, 2) void prefill_attention_kernel(const PrefillParams p) {
    // two K/V tile buffers: tile t+1 is written while tile t is read, one workgroup barrier per tile
    __shared__ __attribute__((aligned(16))) char lds[2 * kLdsBufBytes];

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
    // K/V rows of the sequence: slab tokens cachestarts[b] .. +kvlen (cache source), or rows kvstarts[b] .. +kvlen of
    // the packed fp16 key/value tensors. The new tokens are the LAST L of the kvlen keys: query row i sees keys
    // <= sp + i with sp = kvlen - L (= start_pos for the cache source). MultiHeadCacheAttention without cache-prefill
    // passes kvstarts = seqstarts, i.e. kvlen = L and sp = 0.
    const int64_t kv0 = p.kvstarts[b];
    const int64_t kvlen = p.kvstarts[b + 1] - kv0;
    const int64_t sp = FROM_CACHE ? p.start_pos[b] : (kvlen > L ? kvlen - L : 0);
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
    TileSrc<FROM_CACHE> src;
    if constexpr (FROM_CACHE) src = make_tile_src_cache(p, b, kvh);
    else src = make_tile_src_f16(p, kv0, kvh);
    fetch_tile(regs, src, 0, kvlen);

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

    float16_t oT[4]; // O^T accumulators: oT[i][r] = channel 32*i + 8*(r/4) + 4*hb + r%4 of query row n
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oT[i][r] = 0.f;
    // m_ref: reference maximum of the RAW scores (before the exp2 scaling) that the probabilities are taken against
    float m_ref = -INFINITY, l_part = 0.f;

    // last key any row of this wave sees (none when all its rows lie past the end of the sequence)
    const int64_t wave_last_vis = q0 + 32 * wave >= L ? -1 : (p.is_causal ? sp + q0 + 32 * wave + 31 : kvlen);
    const int64_t wave_first_vis = p.is_causal ? sp + q0 + 32 * wave : kvlen; // keys <= this are seen by all its rows
    const int64_t vis = p.is_causal ? sp + row : kvlen; // last visible key of this lane's row
    const int64_t last_key = vis < kvlen - 1 ? vis : kvlen - 1; // last key this lane's row may attend to
    const float c = p.score_scale;

    // per-lane LDS offsets that do not depend on the tile
    const int k_off = n * kLdsRow + 16 * hb;
    int vt_off[4]; // V^T row n of channel block 0 with 16-byte chunk (2*pr + hb) ^ (n >> 4); channel block i adds 32
                   // rows and, through the row / 16 swizzle, flips the pair index pr by i
#pragma unroll
    for (int pr = 0; pr < 4; ++pr) vt_off[pr] = kLdsKBytes + n * kVtRow + (((2 * pr + hb) ^ (n >> 4)) << 4);

    // pipeline: registers hold tile t+1 (in flight from global memory) while tile t is computed out of LDS buffer t & 1;
    // after the compute the registers are parked in the other buffer and the loads of tile t+2 are issued
    store_tile(regs, lds, lds + kLdsKBytes);
    // The query loads were issued behind tile 0: wait for them here, explicitly (s_waitcnt vmcnt(0)). Otherwise the
    // wait lands at the top of the loop, in front of the first MFMA that reads qB, and on every iteration it also
    // waits for the next tile's loads that were issued just before: the prefetch distance would be zero.
    __builtin_amdgcn_s_waitcnt(0x0f70);
    if (kBN < kv_end) fetch_tile(regs, src, kBN, kvlen);
    __syncthreads();
    int buf = 0;
    for (int64_t j0 = 0; j0 < kv_end; j0 += kBN, buf ^= 1) {
        const char* tile = lds + buf * kLdsBufBytes;
        if (j0 <= wave_last_vis) { // else the whole tile is above this wave's diagonal (wave-uniform)
            // ---- S^T tiles: 2 x (32 kv tokens x 32 query rows). The 16 K operands rotate through four registers sets
            // with their LDS reads issued four steps ahead of the MFMA that consumes them (the scheduling barriers pin
            // that order: left alone, the compiler issues each read right before its use and every MFMA waits out a
            // full LDS latency); the first V^T operand group is requested behind the last K reads.
            float16_t sT[2];
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int r = 0; r < 16; ++r) sT[blk][r] = 0.f;
            const char* kr = tile + k_off;
            auto lds_k = [&](int step) { // step = 8 * blk + kk
                half8_t a;
                const uint4 x = *reinterpret_cast<const uint4*>(kr + (step >> 3) * 32 * kLdsRow + 32 * (step & 7));
                __builtin_memcpy(&a, &x, 16);
                return a;
            };
            auto lds_v = [&](int J, int i) {
                half8_t a;
                const uint4 x = *reinterpret_cast<const uint4*>(tile + vt_off[J ^ i] + i * 32 * kVtRow);
                __builtin_memcpy(&a, &x, 16);
                return a;
            };
            half8_t kb[4], va[2][4];
#pragma unroll
            for (int st = 0; st < 4; ++st) kb[st] = lds_k(st);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int st = 0; st < 16; ++st) {
                sT[st >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kb[st & 3], qB[st & 7], sT[st >> 3], 0, 0, 0);
                if (st + 4 < 16) kb[st & 3] = lds_k(st + 4);
                else va[0][st - 12] = lds_v(0, st - 12);
                __builtin_amdgcn_sched_barrier(0);
            }
            const bool need_mask = (j0 + kBN - 1 > wave_first_vis) || (j0 + kBN > kvlen);
            if (need_mask) {
                // last visible token of this row, relative to the tile, clamped to [-1, 63]
                const int64_t lim64 = last_key - j0;
                const int lim = (int)(lim64 < -1 ? -1 : (lim64 > kBN - 1 ? kBN - 1 : lim64));
#pragma unroll
                for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (32 * blk + 8 * (r >> 2) + 4 * hb + (r & 3) > lim) sT[blk][r] = -INFINITY;
            }

            // ---- online softmax for this lane's query row: p = exp2(s*c - m*c), one fma + one exp2 per score
            float mx = -INFINITY;
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sT[blk][r]);
            mx = fmaxf(mx, other_half(mx));
            // key 0 is visible to every row, so the first tile gives every row a finite maximum (m_ref = -inf forces
            // the update); rows past the sequence end have all-zero queries and stay finite as well
            const bool moved = (mx - m_ref) * c > kRescaleLog2;
            if (__any(moved)) { // a row's result depends on its own scores only: rows that did not move keep theirs
                const float m_new = moved ? mx : m_ref;
                const float alpha = __builtin_amdgcn_exp2f((m_ref - m_new) * c);
                m_ref = m_new;
                l_part *= alpha;
#pragma unroll
                for (int i = 0; i < 4; ++i) oT[i] *= alpha;
            }
            const float neg_mc = -m_ref * c;
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
            l_part += psum;

            // ---- O^T += V^T * P^T: channel block i (32 channels), 16 tokens per MFMA k-block; the operands of token
            // group J + 1 are requested before the MFMAs of group J are issued
#pragma unroll
            for (int J = 0; J < 4; ++J) {
                if (J < 3) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) va[(J + 1) & 1][i] = lds_v(J + 1, i);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    oT[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[J & 1][i], pB[J], oT[i], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (j0 + kBN < kv_end) {
            // the other buffer was last read during the previous iteration, which every wave left through the barrier
            char* next = lds + (buf ^ 1) * kLdsBufBytes;
            store_tile(regs, next, next + kLdsKBytes);
            if (j0 + 2 * kBN < kv_end) fetch_tile(regs, src, j0 + 2 * kBN, kvlen);
        }
        __syncthreads();
    }

    const float l_tot = l_part + other_half(l_part);
    const float inv = 1.0f / l_tot;
    // ---- output through LDS (the loop's last barrier freed it): each wave parks its 32 x 128 fp16 tile in its own
    // 32 rows, then writes full rows
    char* otile = lds + wave * 32 * kLdsRow;
    // lane (query row n, hb) holds, in oT[i][r], channel 32*i + 8*(r/4) + 4*hb + r%4
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int ch = 32 * i + 8 * g + 4 * hb;
            const half4_t o = {(half_t)(oT[i][4 * g] * inv), (half_t)(oT[i][4 * g + 1] * inv),
                               (half_t)(oT[i][4 * g + 2] * inv), (half_t)(oT[i][4 * g + 3] * inv)};
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

// ---------------------------------------------------------------------------------------------------------------
// fp16 K/V source: tiles travel global -> LDS by DMA (global_load_lds_dwordx4), no registers and no LDS stores.
//   * K rows land as they are (256 B per token, no padding); the 16-byte chunk q of row r is stored at position
//     q ^ (r & 15), chosen on the GLOBAL side of the transfer (lane i of an instruction fills LDS bytes 16*i .. +15 of
//     four consecutive rows and may fetch any 16 bytes it likes), so the 16-byte operand reads of 16 consecutive rows
//     spread over all banks.
//   * V lands row-major as well (64-byte chunk index ^ (r & 3)); the PV operand is read with ds_read_b64_tr_b16, which
//     hands lane j of a 16-lane block element (j % 4) of the 8 bytes addressed by lanes 4*i + j/4, i = 0..3: with lane
//     4*i + g addressing token t0 + i, channels c0 + 4g .. +3, lane j receives channel c0 + j of tokens t0 .. t0+3,
//     i.e. V^T in MFMA operand layout without any transposition pass.
// The DMA instructions are written as inline assembly: the compiler then does not know that LDS is written behind
// its back and does not make every LDS read wait for the transfers in flight; completion is waited for explicitly
// (s_waitcnt vmcnt(0) by the issuing wave, then the workgroup barrier that ends the iteration).
// Ring: K slots 0/1 at LDS bytes 0 / 16384, V slots 0/1 at 32768 / 49152. Iteration t computes tile t out of slot
// t & 1 while tile t + 1 lands in the other slot (last read in iteration t - 1, which every wave left through the
// barrier).
constexpr int kDmaTile = kBN * kPDh * 2; // 16384 bytes of K (or V) per tile
constexpr int kDmaVBase = 2 * kDmaTile;

__device__ inline void dma16(uint32_t voff, gptr_t base, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(base), "s"(lds_addr)
                 : "memory"); // M0 is written here and nowhere else in this kernel (gfx9 LDS instructions do not read it)
}

__device__ inline void tile_softmax(float16_t (&sT)[2], float16_t (&oT)[4], half8_t (&pB)[4], float& m_ref,
                                    float& l_part, float c) {
    float mx = -INFINITY;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sT[blk][r]);
    mx = fmaxf(mx, other_half(mx));
    const bool moved = (mx - m_ref) * c > kRescaleLog2;
    if (__any(moved)) { // a row's result depends on its own scores only: rows that did not move keep theirs
        const float m_new = moved ? mx : m_ref;
        const float alpha = __builtin_amdgcn_exp2f((m_ref - m_new) * c);
        m_ref = m_new;
        l_part *= alpha;
#pragma unroll
        for (int i = 0; i < 4; ++i) oT[i] *= alpha;
    }
    const float neg_mc = -m_ref * c;
    float psum = 0.f;
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
    l_part += psum;
}

typedef __attribute__((address_space(3))) char* lds_char_t;
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) short4_t* lds_short4_t;

// the compact tile grid pays a search per workgroup: worth it from about 6 us of empty dispatches on
constexpr int64_t kCompactMinEmpty = 8192;
constexpr int kWriteUnits = 2; // units of four quantisation groups per thread of a write-only workgroup
// `block` of `nblocks`: the workgroup's index among the prefill workgroups of the launch; `lds`: 4 * kDmaTile bytes,
// 1024-byte aligned.
__device__ __forceinline__ void prefill_workgroup(const PrefillParams& p, uint32_t block, uint32_t nblocks, char* lds) {
    // Workgroups [0, attn_blocks) map to query tiles. The ones behind them quantise the prompt tokens into the slab
    // and leave: they are dispatched last, into the slots that the launch's tail leaves idle. (Measured against the
    // alternatives on 8 prompts of 64..1024 tokens: the same work as a share of every tile workgroup's prologue 67 us,
    // behind the tiles 62 us; dealt evenly INTO the grid 70 us, because that shifts the tiles' workgroup -> XCD
    // assignment and with it the L2 reuse of K/V among the query heads of a kv head.)
    const uint32_t wblock = block - p.attn_blocks;
    const bool is_wblock = block >= (unsigned)p.attn_blocks;
    const uint32_t ablock = is_wblock ? 0 : block;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int b, hl, qt;
    if (!p.compact || is_wblock) {
        // dense grid: (tile level, sequence, head); a sequence shorter than the longest has no tile at the top levels
        const int per_tile = p.num_seqs * p.num_heads;
        const int qt_rev = ablock / per_tile;
        const int rem = ablock - qt_rev * per_tile;
        b = p.first_seq + rem / p.num_heads;
        hl = rem % p.num_heads;
        qt = p.ntiles_max - 1 - qt_rev;
    } else {
        // Compact grid, for batches whose lengths differ so much that most (level, sequence) pairs are empty (one
        // long prompt among many short ones: every empty workgroup still costs its dispatch, 0.75 us per thousand):
        // the grid only has as many workgroups as there can be tiles, and workgroup -> tile is found here. Same order as
        // the dense grid -- levels from the top, sequences by index within a level -- with the empty pairs left out.
        const int rank = ablock / p.num_heads;
        hl = ablock - rank * p.num_heads;
        constexpr int kRegPasses = 4; // tile counts of the first 256 sequences stay in registers
        int nreg[kRegPasses];
#pragma unroll
        for (int k = 0; k < kRegPasses; ++k) {
            const int i = 64 * k + lane;
            nreg[k] = i < p.num_seqs
                          ? (int)((p.seqstarts[p.first_seq + i + 1] - p.seqstarts[p.first_seq + i] + kBM - 1) / kBM)
                          : 0;
        }
        auto tiles_of = [&](int i) {
            return i < p.num_seqs
                       ? (int)((p.seqstarts[p.first_seq + i + 1] - p.seqstarts[p.first_seq + i] + kBM - 1) / kBM)
                       : 0;
        };
        // sum over the lanes of a small non-negative number, bit by bit with ballots (the scalar unit counts the set
        // bits): a few instructions per bit instead of a cross-lane reduction
        auto wave_sum = [&](int v, int bits) {
            int total = 0;
            for (int bit = 0; bit < bits; ++bit) total += __popcll(__ballot((v >> bit) & 1)) << bit;
            return total;
        };
        const int passes = (p.num_seqs + 63) >> 6;
        const int pbits = 32 - __builtin_clz((unsigned)passes); // a lane adds up one number per pass
        const int nbits = 32 - __builtin_clz((unsigned)p.ntiles_max) + pbits;
        // tiles above level q = sum over the sequences of max(0, tiles - 1 - q)
        auto tiles_above = [&](int q) {
            int v = 0;
#pragma unroll
            for (int k = 0; k < kRegPasses; ++k) v += nreg[k] - 1 - q > 0 ? nreg[k] - 1 - q : 0;
            for (int base = 64 * kRegPasses; base < p.num_seqs; base += 64) {
                const int n = tiles_of(base + lane);
                v += n - 1 - q > 0 ? n - 1 - q : 0;
            }
            return wave_sum(v, nbits);
        };
        // the level of this workgroup's rank: the lowest q with (tiles above q) <= rank
        int lo = 0, hi = p.ntiles_max - 1;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (tiles_above(mid) <= rank)
                hi = mid;
            else
                lo = mid + 1;
        }
        const int q = lo;
        const int cum = tiles_above(q);
        {
            int r = 0; // sequences that have a tile at level q
#pragma unroll
            for (int k = 0; k < kRegPasses; ++k) r += nreg[k] > q;
            for (int base = 64 * kRegPasses; base < p.num_seqs; base += 64) r += tiles_of(base + lane) > q;
            if (rank - cum >= wave_sum(r, pbits)) return; // the grid is an upper bound: no tile left for this workgroup
        }
        int idx = rank - cum; // the idx-th sequence (by index) that reaches level q
        int sel = -1;
        for (int base = 0; base < p.num_seqs && sel < 0; base += 64) {
            int n = 0;
            if (base < 64 * kRegPasses) {
#pragma unroll
                for (int k = 0; k < kRegPasses; ++k)
                    if (base == 64 * k) n = nreg[k];
            } else {
                n = tiles_of(base + lane);
            }
            const uint64_t reach = __ballot(n > q);
            const int pc = __popcll(reach);
            if (idx < pc) {
                const bool mine = (n > q) && __popcll(reach & ((uint64_t(1) << lane) - 1)) == idx;
                sel = base + (int)__builtin_ctzll(__ballot(mine));
            } else {
                idx -= pc;
            }
        }
        b = p.first_seq + __builtin_amdgcn_readfirstlane(sel);
        qt = __builtin_amdgcn_readfirstlane(q);
    }
    const int kvh = hl % p.kv_heads;
    const int head = kvh * p.rep + hl / p.kv_heads;
    const int64_t s0 = p.seqstarts[b];
    const int64_t L = p.seqstarts[b + 1] - s0;
    const int64_t kv_first = p.kvstarts[b];
    const int64_t kvlen = p.kvstarts[b + 1] - kv_first;
    const int64_t kv0 = kv_first - (p.kv_origin ? *p.kv_origin : 0); // row of the sequence's first key in k / v
    const int64_t sp = kvlen > L ? kvlen - L : 0;
    const int ntiles = (int)((L + kBM - 1) / kBM);

    // A write-only workgroup's share of the prompt tokens' quantize-on-write: units of four quantisation groups,
    // kWriteUnits per thread and pass.
    auto write_share = [&]() {
        if (p.w_cache == nullptr) return;
        const int64_t units = (p.w_end_token - p.w_first_token) * p.w_per_tok;
        // kWriteUnits units per thread per pass, their 64-byte loads all issued before the first is used
        for (int64_t u0 = (int64_t)wblock * (256 * kWriteUnits) + threadIdx.x; u0 < units;
             u0 += (int64_t)(nblocks - p.attn_blocks) * (256 * kWriteUnits)) {
            uint4 raw[kWriteUnits][4];
#pragma unroll
            for (int k = 0; k < kWriteUnits; ++k) {
                int64_t u = u0 + 256 * k;
                if (u >= units) u = units - 1; // loaded twice, written once
                const int64_t t = p.w_first_token + u / p.w_per_tok;
                const int r = (int)(u % p.w_per_tok);
                const int hi = r >> 2, grp = (r & 3) * 4; // K heads then V heads; first of the unit's four groups
                const int kv = hi >= p.kv_heads, wh = hi - kv * p.kv_heads;
                const uint4* src =
                    reinterpret_cast<const uint4*>((kv ? p.v : p.k) + ((t * p.kv_heads + wh) * 16 + grp) * 8);
#pragma unroll
                for (int i = 0; i < 4; ++i) raw[k][i] = src[i];
            }
#pragma unroll
            for (int k = 0; k < kWriteUnits; ++k) {
                const int64_t u = u0 + 256 * k;
                if (u >= units) break;
                const int64_t t = p.w_first_token + u / p.w_per_tok;
                const int r = (int)(u % p.w_per_tok);
                const int hi = r >> 2, grp = (r & 3) * 4;
                const int kv = hi >= p.kv_heads, wh = hi - kv * p.kv_heads;
                const int64_t t0 = ((int64_t)__builtin_amdgcn_readfirstlane((int)(t >> 32)) << 32) |
                                   (uint32_t)__builtin_amdgcn_readfirstlane((int)t);
                const int wb = __all(t == t0) ? find_sequence_wave(p.seqstarts, p.w_batch, t0)
                                              : find_sequence(p.seqstarts, p.w_batch, t);
                const int64_t tok = p.pages.token(wb, p.start_pos[wb] + (t - p.seqstarts[wb]));
                uint2 q[4];
                half_t sc[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) quantize_group8(raw[k][i], &q[i], &sc[i]);
                const int64_t row = p.addr.row(tok, kv, wh);
                uint4* dst = reinterpret_cast<uint4*>(p.w_cache + row + grp * 8);
                dst[0] = make_uint4(q[0].x, q[0].y, q[1].x, q[1].y);
                dst[1] = make_uint4(q[2].x, q[2].y, q[3].x, q[3].y);
                uint32_t packed[2];
                __builtin_memcpy(packed, sc, 8);
                uint32_t* sdst = reinterpret_cast<uint32_t*>(p.w_scale + row / kQuantGroup + grp);
                sdst[0] = packed[0];
                sdst[1] = packed[1];
            }
        }
    };
    if (is_wblock) {
        write_share();
        return;
    }
    if (qt >= ntiles) return;
    const int64_t q0 = (int64_t)qt * kBM;

    const int n = lane & 31;
    const int hb = lane >> 5;
    const int64_t row = q0 + 32 * wave + n;
    const bool row_ok = row < L;
    const int64_t last_row = (q0 + kBM < L ? q0 + kBM : L) - 1;
    int64_t kv_end = p.is_causal ? sp + last_row + 1 : kvlen;
    if (kv_end > kvlen) kv_end = kvlen;
    const int nkv = (int)((kv_end + kBN - 1) / kBN);

    // ---- DMA source: instruction i of this wave fills LDS rows 16*wave + 4*i + lane/16, chunk position lane % 16.
    // Per-lane offsets are relative to row 16*wave + 4*i of the tile: K needs one per instruction (its swizzle key
    // depends on i), V a single one.
    const uint32_t row_bytes = (uint32_t)p.kv_heads * kPDh * 2;
    const char* k_seq = reinterpret_cast<const char*>(p.k) + (kv0 * p.kv_heads + kvh) * kPDh * 2;
    const char* v_seq = reinterpret_cast<const char*>(p.v) + (kv0 * p.kv_heads + kvh) * kPDh * 2;
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char_t)lds);
    const int dq = lane & 15, dr = lane >> 4;
    const int dma_row0 = 16 * wave + dr; // LDS row of transfer 0; transfer i: + 4 * i
    const uint32_t k_swz0 = (uint32_t)((dq ^ dr) << 4); // K: chunk dq ^ (row & 15), row & 15 = 4*i + dr -> ^ (i << 6)
    const uint32_t v_swz = (uint32_t)((dq ^ (dr << 2)) << 4); // V: chunk dq ^ ((row & 3) << 2), row & 3 = dr
    // one tile of K or V = 4 transfers per wave; everything that is the same for the 4 is in TileDma
    struct TileDma {
        gptr_t base; // row 0 of the tile
        uint32_t slot; // LDS address of this wave's 16 rows in the ring slot
        int last_row; // rows past the end of the sequence re-read the last one (their scores are masked)
    };
    auto tile_dma = [&](int t, bool is_v) {
        const int64_t j0 = (int64_t)t * kBN;
        TileDma d;
        d.base = uniform_ptr((is_v ? v_seq : k_seq) + j0 * row_bytes);
        d.slot = lds_base + (is_v ? kDmaVBase : 0) + (uint32_t)(t & 1) * kDmaTile + (uint32_t)wave * 4096;
        d.last_row = (int)(kvlen - j0 < kBN ? kvlen - j0 : kBN) - 1;
        return d;
    };
    auto issue_one = [&](const TileDma& d, bool is_v, int i) {
        const int r = dma_row0 + 4 * i;
        const uint32_t rm = (uint32_t)(r < d.last_row ? r : d.last_row);
        dma16(__umul24(rm, row_bytes) + (is_v ? v_swz : (k_swz0 ^ (uint32_t)(i << 6))), d.base,
              d.slot + 1024 * i);
    };
    auto issue = [&](int t, bool is_v) {
        const TileDma d = tile_dma(t, is_v);
#pragma unroll
        for (int i = 0; i < 4; ++i) issue_one(d, is_v, i);
    };
    issue(0, false);
    issue(0, true);
    if (nkv > 1) issue(1, false);

    // Q^T as the B operand: qB[kk] = Q[row][16*kk + 8*hb .. +7]
    half8_t qB[8];
    {
        const half_t* qp = p.q + ((s0 + (row_ok ? row : 0)) * p.num_heads + head) * kPDh + 8 * hb;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const uint4 x = *reinterpret_cast<const uint4*>(qp + 16 * kk); // rows past the end: row 0, zeroed below
            __builtin_memcpy(&qB[kk], &x, 16);
        }
    }
    float16_t oT[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oT[i][r] = 0.f;
    // m_ref: reference maximum of a row in exponent units, always a value fp16 holds exactly; score registers hold
    // (exponent - the m_ref that was current when their MFMAs were issued)
    float m_ref = 0.f, l_part = 0.f;

    const int64_t wave_last_vis = p.is_causal ? sp + q0 + 32 * wave + 31 : kvlen;
    const int64_t wave_first_vis = p.is_causal ? sp + q0 + 32 * wave : kvlen;
    const int64_t vis = p.is_causal ? sp + row : kvlen;
    const int64_t last_key = vis < kvlen - 1 ? vis : kvlen - 1;
    // tiles this wave computes: those with a key some row of the wave sees (a prefix of the workgroup's tiles)
    int n_act = (int)(wave_last_vis / kBN) + 1;
    if (n_act > nkv) n_act = nkv;
    // a wave whose 32 rows all lie past the end of the sequence (the last query tile of a sequence is rarely full)
    // computes nothing: it only takes part in the transfers and the barriers, and leaves the matrix cores to the
    // workgroup it shares the CU with
    if (q0 + 32 * wave >= L) n_act = 0;

    // ---- per-lane LDS read offsets (relative to the slot)
    // K operand of step (blk, kk): row 32*blk + n, chunk 2*kk + hb, stored at position chunk ^ (n & 15), which is
    // (position of chunk hb) ^ 2*kk: one register, one XOR per read
    const int k_off0 = n * 256 + ((hb ^ (n & 15)) << 4);
    // V operand of (channel block i, token group): this lane addresses token 4*hb + (lane % 16) / 4 of the group's
    // 8-token half, channels 32*i + 16*((lane / 16) & 1) + 4*(lane % 4) .. +3; 64-byte chunk i sits at i ^ (token & 3)
    const int v_off0 = kDmaVBase + (4 * hb + ((lane & 15) >> 2)) * 256 + (((lane & 15) >> 2) << 6) +
                       32 * ((lane >> 4) & 1) + 8 * (lane & 3);
    const lds_char_t lds3 = (lds_char_t)lds;
    auto lds_k = [&](int t, int step) { // step = 8 * blk + kk
        half8_t a;
        const u32x4_t x = *reinterpret_cast<const __attribute__((address_space(3))) u32x4_t*>(
            lds3 + (t & 1) * kDmaTile + (k_off0 ^ ((step & 7) << 5)) + (step >> 3) * 32 * 256);
        __builtin_memcpy(&a, &x, 16);
        return a;
    };
    // tokens 16*G + 8*q + 4*hb + e, e = 0..3, for q = 0 (low half of the operand) and q = 1
    auto lds_v = [&](int t, int G, int i) {
        const lds_char_t at = lds3 + (t & 1) * kDmaTile + (v_off0 ^ (i << 6));
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_t)(at + (16 * G) * 256));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_t)(at + (16 * G + 8) * 256));
        const short8_t x = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        half8_t a;
        __builtin_memcpy(&a, &x, 16);
        return a;
    };

    // tile 0 and the queries have to be there before the first MFMA (see prefill_attention_kernel for why the wait
    // is explicit)
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    // the queries are scaled once by log2(e) / sqrt(Dh), so that the MFMA result is the exponent of exp2 directly and
    // no per-score multiply is left in the loop. Packed fp16 multiplies: the factor is rounded to fp16, i.e. the
    // softmax runs at a temperature that is off by at most 2^-12 relative, far inside the output tolerance.
    {
        // (rows past the end of the sequence loaded a real row to stay inside memory: factor 0 makes them zero
        // queries, whose scores are finite and whose output rows are never stored)
        const half_t c16 = row_ok ? (half_t)p.score_scale : (half_t)0.f;
        const half8_t cv = {c16, c16, c16, c16, c16, c16, c16, c16};
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) qB[kk] = qB[kk] * cv;
    }


    // Software pipeline over the tiles: iteration t exponentiates the scores of tile t (vector ALU) while the MFMAs
    // of tile t + 1's scores are issued from the same instruction stream, then accumulates P(t) * V(t). Ring use in
    // iteration t: reads K(t+1) and V(t), transfers K(t+2) -> K slot t & 1 and V(t+1) -> V slot (t+1) & 1, both last
    // read in iteration t - 1.
    float16_t sA[2], sB[2]; // raw scores of the current and the next tile, alternating
    {
        half8_t kb[4];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int r = 0; r < 16; ++r) sA[blk][r] = 0.f;
#pragma unroll
        for (int st = 0; st < 4; ++st) kb[st] = lds_k(0, st);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int st = 0; st < 16; ++st) {
            sA[st >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kb[st & 3], qB[st & 7], sA[st >> 3], 0, 0, 0);
            if (st + 4 < 16) kb[st & 3] = lds_k(0, st + 4);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // running maximum of the raw scores of the tile about to be exponentiated (per lane: half of a query row's keys)
    float mx_raw = -INFINITY;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx_raw = fmaxf(mx_raw, sA[blk][r]);
    __syncthreads(); // every wave is done with K(0) before K(2) is sent into its slot

    auto step = [&](int t, float16_t (&sC)[2], float16_t (&sN)[2]) __attribute__((always_inline)) {
        const int64_t j0 = (int64_t)t * kBN;
        // transfers of this iteration: K(t+2) and V(t+1)
        if (t + 2 < nkv) issue(t + 2, false);
        if (t + 1 < nkv) issue(t + 1, true);
        if (t < n_act) {
            // ---- stage 1 (vector ALU only): mask, row maxima, move the reference maximum if it has to
            const bool need_mask = (j0 + kBN - 1 > wave_first_vis) || (j0 + kBN > kvlen);
            if (need_mask) {
                const int64_t lim64 = last_key - j0;
                const int lim = (int)(lim64 < -1 ? -1 : (lim64 > kBN - 1 ? kBN - 1 : lim64));
#pragma unroll
                for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (32 * blk + 8 * (r >> 2) + 4 * hb + (r & 3) > lim) sC[blk][r] = -INFINITY;
            }
            float mx = mx_raw; // taken over the unmasked scores while the previous tile's PV MFMAs ran
            if (need_mask) {
                mx = -INFINITY;
#pragma unroll
                for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sC[blk][r]);
            }
            mx = fmaxf(mx, other_half(mx));
            // mx is relative to m_ref. The reference only moves when the row's maximum has outgrown it by more than
            // 2^kRescaleLog2 (always on the first tile, where it becomes the tile's maximum: key 0 is visible to every
            // row, so that maximum is finite)
            const bool moved = mx > kRescaleLog2 || t == 0;
            if (__any(moved)) { // a row's result depends on its own scores only: rows that did not move keep theirs
                const float m_new = (float)(half_t)(m_ref + mx);
                const float delta = moved ? m_new - m_ref : 0.f; // exact: both are fp16 values
                // (nothing is accumulated yet on the first tile, and 0 * 2^(large) must not be formed)
                const float alpha = t == 0 ? 1.0f : __builtin_amdgcn_exp2f(-delta);
                m_ref += delta;
                l_part *= alpha;
#pragma unroll
                for (int i = 0; i < 4; ++i) oT[i] *= alpha;
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) sC[blk] -= delta;
            }
            half8_t pB[4]; // pB[G]: k-slot e8 <-> token 16*G + 8*(e8/4) + 4*hb + e8%4
            half8_t va[4]; // V^T operands, requested four MFMAs ahead
            float psum = 0.f;
            // scores 2*j and 2*j + 1 of the lane's 32 (j = 0..15): two exp2; one step later (so that nothing waits for
            // the exponentials' latency) one packed conversion and one dot2 that adds the two ROUNDED probabilities to
            // the row sum (the sum then matches what the PV MFMAs multiply)
            float e0 = 0.f, e1 = 0.f;
            auto pack_pair = [&](int j) {
                const int G = j >> 2, e = 2 * (j & 3);
                const half2_t pk = {(half_t)e0, (half_t)e1};
                psum = __builtin_amdgcn_fdot2(pk, half2_t{(half_t)1.0f, (half_t)1.0f}, psum, false);
                pB[G][e] = pk[0];
                pB[G][e + 1] = pk[1];
            };
            auto exp_pair = [&](int j, float x0, float x1) {
                if (j > 0) pack_pair(j - 1);
                e0 = __builtin_amdgcn_exp2f(x0);
                e1 = __builtin_amdgcn_exp2f(x1);
                if (j == 15) pack_pair(15);
            };
            // ---- stage 2: scores of tile t + 1 (MFMA) interleaved with the exponentials of tile t (vector ALU): the
            // source order below is the instruction order (the scheduling barriers keep the compiler from regrouping
            // it). The two sides of the branch must not look alike, or the exponentials are hoisted above it as common
            // code, out of the block that holds the MFMAs.
            __builtin_amdgcn_sched_barrier(0);
            if (t + 1 < n_act) {
                half8_t kb[4];
#pragma unroll
                for (int st = 0; st < 4; ++st) kb[st] = lds_k(t + 1, st);
                // -m_ref enters the scores through one MFMA per block: A = ones, B = -m_ref in a single k-slot
                half8_t mB;
#pragma unroll
                for (int e = 0; e < 8; ++e) mB[e] = (half_t)0.f;
                mB[0] = hb == 0 ? (half_t)(-m_ref) : (half_t)0.f;
                half8_t ones;
#pragma unroll
                for (int e = 0; e < 8; ++e) ones[e] = (half_t)1.0f;
                float16_t zero;
#pragma unroll
                for (int r = 0; r < 16; ++r) zero[r] = 0.f;
                __builtin_amdgcn_sched_barrier(0);
                sN[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ones, mB, zero, 0, 0, 0);
                sN[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ones, mB, zero, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int st = 0; st < 16; ++st) {
                    sN[st >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kb[st & 3], qB[st & 7], sN[st >> 3], 0, 0, 0);
                    if (st + 4 < 16) kb[st & 3] = lds_k(t + 1, st + 4);
                    else va[st - 12] = lds_v(t, 0, st - 12);
                    exp_pair(st, sC[st >> 3][2 * (st & 7)], sC[st >> 3][2 * (st & 7) + 1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) va[i] = lds_v(t, 0, i);
                float bias = 0.f; // (opaque zero: keeps this copy of the exponentials from being merged with the other)
                asm volatile("" : "+v"(bias));
#pragma unroll
                for (int j = 0; j < 16; ++j) exp_pair(j, sC[j >> 3][2 * (j & 7)] + bias, sC[j >> 3][2 * (j & 7) + 1] + bias);
                __builtin_amdgcn_sched_barrier(0);
            }
            l_part += psum;
            // ---- stage 3: O^T += V^T * P^T, step 4*G + i = token group G, channel block i
            float mxa = -INFINITY, mxb = -INFINITY;
#pragma unroll
            for (int st = 0; st < 16; ++st) {
                oT[st & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[st & 3], pB[st >> 2], oT[st & 3], 0, 0, 0);
                if (st + 4 < 16) va[st & 3] = lds_v(t, (st + 4) >> 2, st & 3);
                // the next tile's row maximum rides along (two chains of max3; unused after the wave's last tile)
                if (st & 1) mxb = fmaxf(fmaxf(mxb, sN[st >> 3][2 * (st & 7)]), sN[st >> 3][2 * (st & 7) + 1]);
                else mxa = fmaxf(fmaxf(mxa, sN[st >> 3][2 * (st & 7)]), sN[st >> 3][2 * (st & 7) + 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
            mx_raw = fmaxf(mxa, mxb);
        }
        // this wave's transfers have landed; the barrier publishes everybody's and frees the slots read above
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
    };
    for (int t = 0; t < nkv; t += 2) { // the two score register sets swap roles from tile to tile
        step(t, sA, sB);
        if (t + 1 < nkv) step(t + 1, sB, sA);
    }

    const float l_tot = l_part + other_half(l_part);
    const float inv = 1.0f / l_tot;
    char* otile = lds + wave * 32 * kLdsRow;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int ch = 32 * i + 8 * g + 4 * hb;
            const half4_t o = {(half_t)(oT[i][4 * g] * inv), (half_t)(oT[i][4 * g + 1] * inv),
                               (half_t)(oT[i][4 * g + 2] * inv), (half_t)(oT[i][4 * g + 3] * inv)};
            uint2 packed;
            __builtin_memcpy(&packed, &o, 8);
            *reinterpret_cast<uint2*>(otile + n * kLdsRow + ch * 2) = packed;
        }
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
        const int rr = 4 * pass + (lane >> 4);
        const int64_t orow = q0 + 32 * wave + rr;
        const uint4 x = *reinterpret_cast<const uint4*>(otile + rr * kLdsRow + (lane & 15) * 16);
        if (orow < L)
            *reinterpret_cast<uint4*>(p.out + ((s0 + orow) * p.num_heads + head) * kPDh + (lane & 15) * 8) = x;
    }
}

__global__ __launch_bounds__(256, 2) void prefill_f16_kernel(const PrefillParams p) {
    __shared__ __attribute__((aligned(1024))) char lds[4 * kDmaTile];
    prefill_workgroup(p, blockIdx.x, gridDim.x, lds);
}

// Whether the prefill launch quantises the prompt tokens into the slab itself (instead of a separate launch before
// it): whenever it reads K/V from the fp16 inputs, i.e. does not depend on the slab holding them.
bool prefill_writes_new_tokens(const pplhip_mhca_args* a) {
    return !a->enable_cache_prefill && a->batch > a->decoding_batches;
}

// Fills the launch parameters of the prompts' attention (and enqueues the staging pass where the plan has one).
// *blocks: workgroups of the launch; *from_slab: the kernel that dequantises the int8 slab itself has to run it.
// with_decode_tokens: the write-only workgroups also quantise the decode sequences' new tokens (the first
// decoding_batches packed tokens); *out has w_first_token == 0 then.
static pplhip_retcode prefill_setup(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* ws, hipStream_t stream,
                                    bool with_decode_tokens, PrefillParams* out, int64_t* out_blocks, bool* from_slab) {
    const int npre = (int)(a->batch - a->decoding_batches);
    PrefillParams p;
    p.kv_origin = nullptr;
    p.q = (const half_t*)a->d_query;
    p.k = (const half_t*)a->d_current_key;
    p.v = (const half_t*)a->d_current_value;
    p.cache = (const int8_t*)a->d_cache;
    p.scale = (const half_t*)a->d_scale;
    p.seqstarts = a->d_seqstarts;
    // fp16 source: the keys of a prefill sequence are its own new tokens, packed like the queries
    p.kvstarts = a->enable_cache_prefill ? a->d_kvstarts : a->d_seqstarts;
    p.pages = PageMap{a->d_cachestarts, a->cachestart_stride_b, page_shift_of(a->cache_mode, a->page_size)};
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
    // cache-prefill over staged fp16 rows: the slab rows of the prompts (the new tokens are in there by now) are
    // dequantised in one streaming pass, and attention reads those like it reads current_key / current_value
    const bool staged = a->enable_cache_prefill && plan->prefill_staging;
    if (staged) {
        const int64_t tokens = prefill_staging_tokens(a);
        if (tokens == 0 || ws == nullptr)
            PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "prefill: plan was not produced by pplhip_mhca_prepare for these arguments");
        half_t* k_stage = (half_t*)((char*)ws + (uint64_t)plan->prefill_staging_offset_256 * 256);
        half_t* v_stage = k_stage + tokens * a->num_kv_heads * a->head_dim;
        pplhip_retcode rc = launch_kv_stage_prefill(a, k_stage, v_stage, tokens, stream);
        if (rc != PPLHIP_RC_SUCCESS) return rc;
        p.k = k_stage;
        p.v = v_stage;
        p.kv_origin = a->d_kvstarts + a->decoding_batches; // staging row 0 = the first prompt's first cached token
    }
    p.w_cache = nullptr;
    if (prefill_writes_new_tokens(a)) {
        p.w_cache = (int8_t*)a->d_cache;
        p.w_scale = (half_t*)a->d_scale;
        // one new token per decode sequence, then the prompts
        p.w_first_token = with_decode_tokens ? 0 : a->decoding_batches;
        p.w_end_token = a->total_new_tokens;
        p.w_batch = (int32_t)a->batch;
        p.w_per_tok = 2 * a->num_kv_heads * 4;
    }
    int64_t blocks = (int64_t)plan->prefill_num_q_tiles * npre * a->num_heads;
    p.ntiles_max = plan->prefill_num_q_tiles;
    p.compact = 0;
    if (!a->enable_cache_prefill || staged) {
        // the prompts hold total_new_tokens - decoding_batches tokens: at most that many / kBM + one per sequence tiles
        const int64_t prompt_tokens = a->total_new_tokens - a->decoding_batches;
        const int64_t tile_bound = (prompt_tokens / kBM + npre) * a->num_heads;
        if (blocks - tile_bound >= kCompactMinEmpty) {
            blocks = tile_bound;
            p.compact = 1;
        }
    }
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "prefill: too many query tiles in one call");
    p.attn_blocks = (int32_t)blocks;
    if (p.w_cache != nullptr) {
        const int64_t units = (p.w_end_token - p.w_first_token) * p.w_per_tok;
        blocks += (units + 256 * kWriteUnits - 1) / (256 * kWriteUnits);
        if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "prefill: too many tokens in one call");
    }
    *out = p;
    *out_blocks = blocks;
    *from_slab = a->enable_cache_prefill && !staged;
    return PPLHIP_RC_SUCCESS;
}

pplhip_retcode launch_prefill(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* ws, hipStream_t stream) {
    if (a->batch <= a->decoding_batches || plan->prefill_num_q_tiles <= 0) return PPLHIP_RC_SUCCESS;
    PrefillParams p;
    int64_t blocks;
    bool from_slab;
    const pplhip_retcode rc = prefill_setup(a, plan, ws, stream, false, &p, &blocks, &from_slab);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    const dim3 grid((unsigned)blocks);
    if (from_slab)
        hipLaunchKernelGGL(prefill_attention_kernel<true>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(prefill_f16_kernel, grid, dim3(256), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("prefill_attention");
    return PPLHIP_RC_SUCCESS;
}

// opmx.dynamic_batching::MultiHeadAttention: the same kernel over explicit packed fp16 key/value tensors; every
// sequence (decode ones included) is a set of query tiles.
pplhip_retcode launch_mha(const pplhip_mha_args* a, hipStream_t stream) {
    if (a->batch <= 0 || a->max_seqlen <= 0) return PPLHIP_RC_SUCCESS;
    PrefillParams p;
    p.q = (const half_t*)a->d_query;
    p.k = (const half_t*)a->d_key;
    p.v = (const half_t*)a->d_value;
    p.cache = nullptr;
    p.scale = nullptr;
    p.seqstarts = a->d_seqstarts;
    p.kvstarts = a->d_kvstarts;
    p.pages = PageMap{nullptr, 0, 0};
    p.start_pos = nullptr;
    p.out = (half_t*)a->d_output;
    p.addr = CacheAddr{0, 0, 0, 0, 0};
    p.first_seq = 0;
    p.num_heads = a->num_heads;
    p.kv_heads = a->num_kv_heads;
    p.rep = a->num_heads / a->num_kv_heads;
    p.is_causal = a->is_causal;
    p.score_scale = 1.4426950408889634f / sqrtf((float)a->head_dim);
    p.num_seqs = (int32_t)a->batch;
    p.kv_origin = nullptr;
    p.w_cache = nullptr; // MultiHeadAttention has no cache to write
    p.w_scale = nullptr;
    const int64_t q_tiles = (a->max_seqlen + kBM - 1) / kBM;
    const int64_t blocks = q_tiles * a->batch * a->num_heads;
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "attention: too many query tiles in one call");
    p.attn_blocks = (int32_t)blocks;
    p.ntiles_max = (int32_t)q_tiles;
    p.compact = 0; // (the token total that bounds the number of tiles is not among this op's arguments)
    hipLaunchKernelGGL(prefill_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("multi_head_attention");
    return PPLHIP_RC_SUCCESS;
}

} // namespace pplhip
