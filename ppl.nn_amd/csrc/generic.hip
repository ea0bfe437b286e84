// The attention kernels for everything the specialised kernels (decode.hip, prefill.hip: head_dim 128, at most 16 query
// heads per kv head, no mask) do not take: any head_dim that is a multiple of 16 up to 256, any number of query heads
// per kv head, and an additive attn_mask; for MultiHeadCacheAttention and MultiHeadAttention.
// The kernels are compiled for head dims that are multiples of 32 (DH). Another head_dim (80, 112, ...) runs the next
// larger DH with the channels past head_dim held as zeros where rows enter LDS or registers (zero query and key
// channels add nothing to a score, zero value channels give output channels that are not stored); rows in memory keep
// their real length. Such calls go through the tile kernel only.
//
// generic_attention_kernel (the tile kernel: prompts, MultiHeadAttention, decode tokens with more than 16 query heads
// per kv head). Rows of a workgroup are (query token, query head of the kv head) pairs of ONE (sequence, kv head): row
// r of the sequence is token r / rep, head kvh * rep + r % rep, so the K/V tile a workgroup stages in LDS is shared by
// all query heads of its kv head, and a decode sequence (one token) fills rep rows of a tile instead of one. 64 rows
// per workgroup, 16 per wave. Per K/V tile: S^T = K Q^T and O^T += V^T P^T with v_mfma_f32_16x16x32_f16, a query row
// living in the 16 lanes' same column throughout (row maxima are per lane, reduced only over the four 16-lane groups;
// row sums come out of the matrix cores); P never leaves registers (the result layout of the first product is the B
// operand layout of the second); V^T operands come from row-major V through ds_read_b64_tr_b16. K/V come from the
// int8 slab (dequantised on the way into LDS, value = fp16(float(q) * float(scale)) as everywhere) or from packed fp16
// rows. The next K/V tile is requested from memory before the current one is computed.
//
// generic_decode_kernel (decode sequences with at most 16 query heads per kv head): a wave per (sequence, one or two
// kv heads, piece of the keys), K straight from the slab into the matrix-core operands; generic_merge_kernel combines
// the pieces of a sequence. Described where they are defined.
#include "common.h"

#include <type_traits>

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
    int32_t head_dim; // channels of a row in q / k16 / v16 / out and of a head in the slab (<= the kernel's DH)
    int32_t first_fp16_seq; // sequences [0, first_fp16_seq) read the slab, the others the fp16 rows
    int32_t k16_holds_new_tokens; // the fp16 rows are the sequences' NEW tokens only (MultiHeadCacheAttention's
                                  // current_key / current_value), packed by seqstarts: such a sequence has seqlen keys
    int32_t is_causal;
    int32_t tiles_max; // row tiles of the longest sequence
    float scale_log2; // log2(e) / sqrt(DH)
    // Decode sequences (the first `split_seqs`) are cut into pieces of `piece_tokens` keys (whole tiles; at most
    // `nsplit` of them for the longest sequence), one workgroup each, whose un-normalised results (accumulator,
    // maximum, sum) go to the workspace and are combined by generic_merge_kernel: one workgroup per (sequence, kv
    // head) would walk a 4 096-token sequence's 64 tiles one after the other while the short sequences' workgroups are
    // long gone. A piece that starts past its sequence's end has no workgroup work and no partial result. nsplit 1: no
    // pieces, no workspace.
    int32_t nsplit, split_seqs, piece_tokens;
    // generic_attention_kernel covers sequences [first_seq, batch): the decode sequences before them are
    // generic_decode_kernel's when it can take them (see there)
    int32_t first_seq;
    float* part_o; // [split_seqs * num_heads, nsplit, DH]
    float* part_ml; // [split_seqs * num_heads, nsplit, 2]
};

constexpr int kGenRows = 64;
// head dims at which a wave takes two blocks of 16 rows (tiles of 128 rows): measured on four 2 048-token prompts,
// one block against two: head_dim 32 135 / 142 us, 64 176 / 194 us, 96 301 / 268 us, 128 (with a mask) 405 / 398 us;
// above 128 two blocks' accumulators do not fit the registers
constexpr bool gen_two_row_blocks(int head_dim) { return head_dim >= 96 && head_dim <= 128; }
constexpr float kLog2e = 1.4426950408889634f;

// RB: blocks of 16 rows per wave (the workgroup's tile has 64 * RB rows). The staging of a K/V tile, its barriers and
// a tile's bookkeeping cost every wave the same whatever its rows, and every K and V operand read from LDS feeds RB
// matrix-core instructions; two blocks' state costs a wave per SIMD (see gen_two_row_blocks).
template <int DH, int RB>
__global__ __launch_bounds__(256, (RB == 2 ? 2 : DH <= 32 ? 5 : DH <= 64 ? 4 : DH <= 96 ? 3 : 2))
void generic_attention_kernel(const GenericParams p) {
    constexpr int GR = kGenRows * RB; // rows of the workgroup's tile
    constexpr int BN = DH <= 128 ? 64 : 32; // kv tokens per tile
    constexpr int LDK = DH + 8; // halves per LDS row (padding spreads the rows over the banks)
    constexpr int KC = DH / 16;
    constexpr int TB = BN / 16;
    __shared__ __attribute__((aligned(16))) half_t lds[2 * BN * LDK];
    half_t* const Ks = lds;
    half_t* const Vs = lds + BN * LDK;

    // Workgroups go to the chip's 8 XCDs in turn (workgroup i to XCD i % 8). The kv heads of one (sequence, row tile,
    // piece) sit next to each other in the slab (a token's row of head_dim 64 is half a cache line), so they run on
    // the same XCD, one after the other in its share of the grid; the (sequence, tile, piece) groups themselves go
    // round the XCDs in the order: every sequence's row tiles, then the second pieces of the decode sequences, the
    // third, ... so that each XCD gets its share of every piece index (pieces with a high index exist for long
    // sequences only).
    const int64_t wi = blockIdx.x >> 3;
    const int kvh = (int)(wi % p.kv_heads);
    const int64_t group = (wi / p.kv_heads) * 8 + (blockIdx.x & 7);
    const int64_t whole = (int64_t)(p.batch - p.first_seq) * p.tiles_max;
    int split = 0, b, tile;
    if (group < whole) {
        b = (int)(group / p.tiles_max);
        tile = (int)(group - (int64_t)b * p.tiles_max);
        b += p.first_seq;
    } else {
        const int64_t extra = group - whole;
        if (extra >= (int64_t)p.split_seqs * (p.nsplit - 1)) return; // (the grid is rounded up to 8 groups)
        split = 1 + (int)(extra / p.split_seqs);
        b = (int)(extra - (int64_t)(split - 1) * p.split_seqs);
        tile = 0;
    }
    // this sequence's keys are shared out among up to nsplit workgroups (a decode sequence: packed token b, its only
    // one, whose rep <= 64 rows are one tile)
    const bool pieces = b < p.split_seqs;
    const int64_t s0 = p.seqstarts[b];
    const int64_t L = p.seqstarts[b + 1] - s0;
    const int64_t kv_first = p.kvstarts[b];
    const bool from_slab = b < p.first_fp16_seq;
    // The prompts of a MultiHeadCacheAttention call without cache-prefill attend over the fp16 rows they bring:
    // current_key / current_value hold exactly L rows for the sequence, whatever kvstarts says (a start_pos > 0 is
    // history that such a call does not look at), so its keys are those L rows. kvstarts still places the sequence's
    // columns in an attn_mask.
    const int64_t kvlen = (!from_slab && p.k16_holds_new_tokens) ? L : p.kvstarts[b + 1] - kv_first;
    const int64_t rows = L * p.rep;
    const int64_t row0 = (int64_t)tile * GR;
    if (row0 >= rows || kvlen <= 0) return;
    const int64_t sp = kvlen > L ? kvlen - L : 0;
    const int64_t k16_row0 = from_slab ? 0 : p.k16_starts[b];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r_lane = lane & 15, g = lane >> 4;
    const int hd = p.head_dim; // <= DH; rows in memory are hd channels long
    // the lane's rows: one in each of the wave's RB blocks of 16
    bool valid[RB];
    int64_t tok[RB], row_limit[RB];
    int head[RB];
    const int64_t all = kvlen - 1;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const int64_t my_row_raw = row0 + (wave * RB + rb) * 16 + r_lane;
        valid[rb] = my_row_raw < rows;
        const int64_t my_row = valid[rb] ? my_row_raw : rows - 1;
        tok[rb] = my_row / p.rep;
        head[rb] = kvh * p.rep + (int)(my_row - tok[rb] * p.rep);
        // keys 0 .. row_limit are visible to this lane's row
        row_limit[rb] = !valid[rb] ? -1 : (p.is_causal ? (sp + tok[rb] < all ? sp + tok[rb] : all) : all);
    }
    const int64_t last_row = (row0 + GR - 1 < rows - 1) ? row0 + GR - 1 : rows - 1;
    int64_t kv_end = p.is_causal ? ((sp + last_row / p.rep + 1 < kvlen) ? sp + last_row / p.rep + 1 : kvlen) : kvlen;
    int64_t kv_begin = 0;
    if (pieces) { // (a decode sequence: one token, which sees every key)
        kv_begin = (int64_t)split * p.piece_tokens;
        if (kv_begin >= kvlen) return; // the merge knows from kvlen that this piece does not exist
        kv_end = kv_begin + p.piece_tokens < kvlen ? kv_begin + p.piece_tokens : kvlen;
    }

    // Q^T as the B operand of the score product (v_mfma_f32_16x16x32_f16: 32 channels a step, 8 of them per lane):
    // channels 32 * kc + 8 * g .. + 7 of the lane's row
    constexpr int KC2 = DH / 32;
    half8_t qf[RB][KC2];
    const half_t* mrow[RB];
    const bool masked = p.mask != nullptr;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const half_t* qp = p.q + ((s0 + tok[rb]) * p.num_heads + head[rb]) * hd + 8 * g;
#pragma unroll
        for (int kc = 0; kc < KC2; ++kc) {
            if (32 * kc + 8 * g < hd) {
                qf[rb][kc] = *reinterpret_cast<const half8_t*>(qp + 32 * kc);
            } else { // a padding channel group
#pragma unroll
                for (int e = 0; e < 8; ++e) qf[rb][kc][e] = (half_t)0.f;
            }
        }
        mrow[rb] = masked ? p.mask + (int64_t)head[rb] * p.mask_stride_h + (s0 + tok[rb]) * p.mask_stride_q + kv_first
                          : nullptr;
    }

    // The running maximum is kept in the domain the scores are held in: raw products (times `cs` = scale_log2 inside
    // the exponentials) without a mask, exp2-domain values (cs = 1) with one. The row's sum of probabilities comes out
    // of the matrix cores (a row of ones as the A operand against P^T: every component of l_acc holds it), which also
    // adds up the four lane groups' shares.
    const float cs = masked ? 1.0f : p.scale_log2;
    float m_run[RB];
    float4_t l_acc[RB];
    float4_t o[RB][KC];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        m_run[rb] = -INFINITY;
        l_acc[rb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < KC; ++i) o[rb][i] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

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
    // Where the thread's chunks of the current tile start: halves into k16 / v16, or bytes into the slab (K row; the V
    // row is stride_kv further). Tiles are fetched in order, so the offsets move on by one tile's worth per fetch; only
    // a paged slab looks every token up.
    const bool paged = from_slab && p.pages.page_shift != 0;
    const int64_t seq_tok0 = from_slab && !paged ? p.pages.cachestarts[b] : 0;
    const int64_t tile_stride = from_slab ? (int64_t)BN * p.addr.stride_s : (int64_t)BN * p.kv_heads * hd;
    int64_t koff[NCH];
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
        const int c = tid + 256 * n;
        const int r = c / CH, ch = c - r * CH;
        koff[n] = from_slab ? p.addr.row(seq_tok0 + kv_begin + r, 0, kvh) + ch * 8
                            : ((k16_row0 + kv_begin + r) * p.kv_heads + kvh) * hd + ch * 8;
    }
    auto fetch = [&](int64_t kv0) {
        const int64_t left64 = kvlen - kv0;
        const int left = left64 > BN ? BN : (int)left64; // tokens of the tile that exist
#pragma unroll
        for (int n = 0; n < NCH; ++n) {
            const int c = tid + 256 * n;
            const int r = c / CH, ch = c - r * CH;
            if (c < BN * CH && r < left && ch * 8 < hd) { // (chunks past head_dim are padding: zeros)
                if (from_slab) {
                    int64_t rk = koff[n];
                    if (paged) rk = p.addr.row(p.pages.token(b, kv0 + r), 0, kvh) + ch * 8;
                    const int64_t rv = rk + p.addr.stride_kv;
                    const uint2 qk = *reinterpret_cast<const uint2*>(p.cache + rk);
                    const uint2 qv = *reinterpret_cast<const uint2*>(p.cache + rv);
                    uint16_t sk, sv; // (rk = row + 8 * ch: the group's scale is element rk / 8)
                    __builtin_memcpy(&sk, &p.scale[rk / kQuantGroup], 2);
                    __builtin_memcpy(&sv, &p.scale[rv / kQuantGroup], 2);
                    raw[n].k = make_uint4(qk.x, qk.y, sk, 0);
                    raw[n].v = make_uint4(qv.x, qv.y, sv, 0);
                } else {
                    raw[n].k = *reinterpret_cast<const uint4*>(p.k16 + koff[n]);
                    raw[n].v = *reinterpret_cast<const uint4*>(p.v16 + koff[n]);
                }
            } else {
                raw[n].k = raw[n].v = make_uint4(0, 0, 0, 0);
            }
            koff[n] += tile_stride;
        }
    };
    auto dequant = [&](const uint4& x) { // slab chunk -> 8 halves, fp16(float(q) * float(scale)) as everywhere
        half_t sc;
        const uint16_t bits = (uint16_t)x.z;
        __builtin_memcpy(&sc, &bits, 2);
        return dequant8(x.x, x.y, sc);
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
    const bool wave_has_rows = row0 + wave * 16 * RB < rows;
    // one K/V tile for the lane's rows
    auto tile_step = [&](const int64_t kv0) {
        // keys kv0 .. kv0 + lim of the tile are visible to the lane's row; a tile all of whose keys are visible to all of
        // the wave's rows (every tile but a causal sequence's last ones, and a ragged tile's) skips the comparisons
        int lim4[RB];
        bool vis = true;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int64_t rel = row_limit[rb] - kv0;
            lim4[rb] = (int)(rel < -1 ? -1 : rel > BN ? BN : rel) - 4 * g;
            vis = vis && lim4[rb] + 4 * g >= BN - 1;
        }
        const bool all_visible = __all(vis);
        // the tile's mask entries of the lane's rows, requested before the score products and without a branch per
        // element: an index past the row's last key is pulled back onto it (that entry exists; its score is masked
        // out by the comparison below)
        float mk[RB][TB][4];
        if (masked) {
            const int64_t last = kvlen - 1;
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
                for (int tb = 0; tb < TB; ++tb) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int64_t j = kv0 + 16 * tb + 4 * g + i;
                        mk[rb][tb][i] = (float)mrow[rb][j < last ? j : last] * kLog2e;
                    }
                }
            }
        }
        // ---- scores of the lane's rows against tokens kv0 + 16 * tb + 4 * g + i
        float s[RB][TB][4];
        float mx[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) mx[rb] = -INFINITY;
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            float4_t acc[RB];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) acc[rb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kc = 0; kc < KC2; ++kc) {
                const half8_t a = *reinterpret_cast<const half8_t*>(&Ks[(16 * tb + r_lane) * LDK + 32 * kc + 8 * g]);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
                    acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qf[rb][kc], acc[rb], 0, 0, 0);
            }
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                if (masked) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[rb][i] = 16 * tb + i <= lim4[rb] ? __builtin_fmaf(acc[rb][i], p.scale_log2, mk[rb][tb][i])
                                                             : -INFINITY;
                } else if (!all_visible) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[rb][i] = 16 * tb + i <= lim4[rb] ? acc[rb][i] : -INFINITY;
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[rb][tb][i] = acc[rb][i];
                    mx[rb] = fmaxf(mx[rb], acc[rb][i]);
                }
            }
        }
        // The second product takes 32 tokens a step: the lane's k-indices 8 * g + e are tokens 16 * tb + 4 * g + e
        // (e < 4) and 16 * (tb + 1) + 4 * g + e - 4 of a pair of 16-token blocks, in the P^T operand (straight from
        // the score registers) and in the V^T operand alike.
        static_assert(TB % 2 == 0, "pairs of 16-token blocks");
        const half8_t ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f,
                              (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
        half8_t pp[RB][TB / 2];
        bool still = true;
        float alpha[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            float m = mx[rb];
            m = fmaxf(m, __shfl_xor(m, 16));
            m = fmaxf(m, __shfl_xor(m, 32));
            const float m_new = fmaxf(m_run[rb], m);
            // a row that has seen nothing but masked keys so far keeps max -inf: against 0 in the exponents its
            // probabilities are exp2(-inf) = 0, not NaN
            const float m_safe = m_new == -INFINITY ? 0.f : m_new;
            alpha[rb] = __builtin_amdgcn_exp2f((m_run[rb] - m_safe) * cs);
            const float shift = -m_safe * cs;
            half4_t pf[TB];
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    pf[tb][i] = (half_t)__builtin_amdgcn_exp2f(__builtin_fmaf(s[rb][tb][i], cs, shift));
            }
            m_run[rb] = m_new;
            still = still && alpha[rb] == 1.0f;
#pragma unroll
            for (int t2 = 0; t2 < TB / 2; ++t2)
                pp[rb][t2] = half8_t{pf[2 * t2][0], pf[2 * t2][1], pf[2 * t2][2], pf[2 * t2][3],
                                     pf[2 * t2 + 1][0], pf[2 * t2 + 1][1], pf[2 * t2 + 1][2], pf[2 * t2 + 1][3]};
        }
        if (!__all(still)) { // (the maximum has moved for some row of the wave)
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                l_acc[rb] *= alpha[rb];
#pragma unroll
                for (int db = 0; db < KC; ++db) o[rb][db] *= alpha[rb];
            }
        }
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int t2 = 0; t2 < TB / 2; ++t2)
                l_acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pp[rb][t2], l_acc[rb], 0, 0, 0);
#pragma unroll
        for (int db = 0; db < KC; ++db) {
#pragma unroll
            for (int t2 = 0; t2 < TB / 2; ++t2) {
                // V^T operand: lane (block g, j) receives channel 16 * db + j of tokens 16 * tb + 4 * g .. + 3 when
                // lane 4 * i + c of the block addresses token 16 * tb + 4 * g + i, channels 16 * db + 4 * c .. + 3
                const half_t* src = &Vs[(32 * t2 + 4 * g + (r_lane >> 2)) * LDK + 16 * db + 4 * (r_lane & 3)];
                const short4_t lo =
                    __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)src);
                const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) short4_t*)(src + 16 * LDK));
                half8_t a;
                __builtin_memcpy(&a, &lo, 8);
                __builtin_memcpy(reinterpret_cast<char*>(&a) + 8, &hi, 8);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
                    o[rb][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pp[rb][t2], o[rb][db], 0, 0, 0);
            }
        }
    };
    fetch(kv_begin);
    for (int64_t kv0 = kv_begin; kv0 < kv_end; kv0 += BN) {
        __syncthreads(); // everybody has finished reading the previous tile
        stash();
        if (kv0 + BN < kv_end) fetch(kv0 + BN);
        __syncthreads();
        if (!wave_has_rows) continue;
        tile_step(kv0);
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const float l = l_acc[rb][0];
        if (!valid[rb]) continue;
        if (pieces) {
            const int64_t prow = ((int64_t)b * p.num_heads + head[rb]) * p.nsplit + split;
            float* dst = p.part_o + prow * DH + 4 * g;
#pragma unroll
            for (int db = 0; db < KC; ++db) *reinterpret_cast<float4_t*>(dst + 16 * db) = o[rb][db];
            if (g == 0) {
                p.part_ml[prow * 2] = m_run[rb] * cs; // -inf for a piece without (unmasked) keys: weight 0 in the merge
                p.part_ml[prow * 2 + 1] = l;
            }
            continue;
        }
        // a row whose keys were all masked out has no distribution: zeros
        const float inv_l = l > 0.f ? 1.0f / l : 0.f;
        half_t* dst = p.out + ((s0 + tok[rb]) * p.num_heads + head[rb]) * hd + 4 * g;
#pragma unroll
        for (int db = 0; db < KC; ++db) {
            const half4_t r = {(half_t)(o[rb][db][0] * inv_l), (half_t)(o[rb][db][1] * inv_l),
                               (half_t)(o[rb][db][2] * inv_l), (half_t)(o[rb][db][3] * inv_l)};
            if (16 * db + 4 * g < hd) *reinterpret_cast<half4_t*>(dst + 16 * db) = r;
        }
    }
}

// ---- decode sequences with no more than 16 query heads per kv head: a wave per (sequence, kv head, piece of keys)
//
// The tile kernel above would give such a sequence one wave of arithmetic and three that only stage tiles and wait at
// its two barriers per tile. Here every wave works alone, with no barrier at all: it walks its piece 16 tokens at a
// time, the int8 rows and scales of the next kBlocksAhead blocks already requested (straight into registers, in program
// order, so that waiting for the oldest block leaves the younger ones in flight).
//   S^T = K Q^T   A = K[token m][channels]: lane (m = lane & 15, g = lane >> 4) loads the g-th quarter of the token's
//                 row and takes 4 of its int8 per 16-channel step of the product; which channels a step multiplies
//                 does not matter as long as the query operand is loaded in the same order, so K never passes through
//                 LDS;
//   O^T += V^T P^T  needs 4 tokens of one channel per lane: the wave's own LDS region takes the dequantised block
//                 [16 tokens][DH] and gives it back transposed (ds_read_b64_tr_b16), as in the tile kernel.
// Whole sequences (nsplit 1) are normalised and written; pieces leave (accumulator, maximum, sum) for the merge.
// Paged slabs: a block of 16 tokens lies within one page (pages are powers of two of at least 64 tokens, checked at
// the entry points), so the page's start is one wave-uniform look-up through the constant address space: a scalar
// load, which does not queue behind the vector loads in flight.
typedef const int64_t __attribute__((address_space(4)))* gen_const_tab_t;

// HP: kv heads per wave. At head_dim 32 and 64 a head's row is a quarter or half of a 128-byte line and its scales an
// eighth of one, and a wave asking for its head's part alone makes the memory system move every line as often as there
// are heads in it (measured on the bare loads of 120 sequences: 150 us a head per wave, 103 us two heads per wave at
// head_dim 64; 123 and 66 us at head_dim 32). With HP = 2 (kv heads next to each other in the slab, their number even)
// the wave loads both heads' rows as one row of 2 * DH bytes, lane g its quarter: lanes g = 0, 1 hold the halves of
// the first head, g = 2, 3 those of the second. Each head's score product runs over all four lanes' K operands with
// that head's query operand set to zero in the other head's lanes.
template <int DH, int HP>
struct GenDecodeShape {
    static constexpr int kRowBytes = DH * HP;
    static constexpr int kBlocksAhead = kRowBytes <= 64 ? 4 : kRowBytes <= 128 ? 3 : 2;
    // waves per SIMD the register allocator is to leave room for (one fewer with a mask, whose values travel with
    // the blocks; two with two heads' state)
    static constexpr int kMinWaves = DH <= 64 ? 4 : DH <= 128 ? 3 : 2;
};

template <int DH, bool MASK, int HP>
__global__ __launch_bounds__(256, (HP > 1 ? 2 : (GenDecodeShape<DH, HP>::kMinWaves) -
                                                     (MASK && (GenDecodeShape<DH, HP>::kMinWaves) > 2 ? 1 : 0)))
void generic_decode_kernel(const GenericParams p) {
    constexpr int KC = DH / 16; // 16-channel blocks of a head's output
    // A token's row (of the wave's HP heads) goes to its four lanes by quarters: lane g holds bytes g * CPL .. + CPL - 1,
    // as NCK chunks of 8 int8 (one quantisation group, one 8-byte load each). The first of these loads touches every
    // cache line of the block's rows; handing the chunks round the four lanes instead (each load covering consecutive
    // bytes of a row, the lines of a block requested over several loads) measured up to twice slower, and 16-byte
    // chunks no faster.
    constexpr int CB = 8;
    constexpr int CPL = DH * HP / 4; // channels per lane
    constexpr int NCK = CPL / CB; // chunks per lane
    constexpr int KS = CPL / 4; // 4-channel steps of a score product per lane
    constexpr int LPH = 4 / HP; // lanes (of the four) per head
    typedef uint2 chunk_t;
    constexpr int LDV = DH * HP + 8; // halves per LDS row
    constexpr int NB = GenDecodeShape<DH, HP>::kBlocksAhead;
    static_assert(HP == 1 || (HP == 2 && DH <= 96), "two heads per wave: their state has to fit the registers");
    __shared__ __attribute__((aligned(16))) half_t lds[4 * 16 * LDV];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r_lane = lane & 15, g = lane >> 4;
    half_t* const Vs = lds + wave * 16 * LDV;

    // unit -> (piece, sequence, kv heads): the kv heads of a (sequence, piece) are neighbours in the slab and in the
    // grid (waves of one workgroup); first pieces first, so that the pieces only long sequences have come last
    const int64_t unit = (int64_t)blockIdx.x * 4 + wave;
    const int head_groups = p.kv_heads / HP;
    const int kvh = (int)(unit % head_groups) * HP; // the wave's first kv head
    const int64_t item = unit / head_groups;
    const int piece = (int)(item / p.split_seqs);
    const int b = (int)(item - (int64_t)piece * p.split_seqs);
    if (piece >= p.nsplit) return; // (the grid is rounded up to whole workgroups)
    const gen_const_tab_t seqstarts = (gen_const_tab_t)p.seqstarts, kvstarts = (gen_const_tab_t)p.kvstarts,
                          cachestarts = (gen_const_tab_t)p.pages.cachestarts;
    const int64_t s0 = seqstarts[b]; // the sequence's one new token
    const int64_t kv_first = kvstarts[b];
    const int64_t kvlen = kvstarts[b + 1] - kv_first;
    const int64_t kv_begin = (int64_t)piece * p.piece_tokens;
    if (kv_begin >= kvlen) return; // the merge knows from kvlen that this piece does not exist
    const int64_t kv_end = kv_begin + p.piece_tokens < kvlen ? kv_begin + p.piece_tokens : kvlen;

    const bool valid = r_lane < p.rep;
    int head[HP]; // the lane's query head (row r_lane) of each kv head
    half4_t qf[HP][KS];
    const half_t* mrow[HP];
#pragma unroll
    for (int h = 0; h < HP; ++h) {
        head[h] = (kvh + h) * p.rep + (valid ? r_lane : p.rep - 1);
        // step kc of head h's score product: the lane's channels 4 * kc .. + 3, which are head g / LPH's channels
        // (g % LPH) * CPL + 4 * kc .. + 3; zero where the lane holds the other head
        const half_t* qp = p.q + (s0 * p.num_heads + head[h]) * DH + (g % LPH) * CPL;
        const bool mine = g / LPH == h;
#pragma unroll
        for (int kc = 0; kc < KS; ++kc) {
            const half4_t x = *reinterpret_cast<const half4_t*>(qp + 4 * kc);
            qf[h][kc] = mine ? x : half4_t{(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
        }
        mrow[h] = MASK ? p.mask + (int64_t)head[h] * p.mask_stride_h + s0 * p.mask_stride_q + kv_first : nullptr;
    }

    // a block of 16 tokens as it comes from memory: the lane's quarter of token (block start + r_lane)'s K and V row
    struct RawBlock {
        chunk_t k[NCK], v[NCK];
        uint32_t ks[NCK], vs[NCK]; // the chunks' scales: fp16 bits
        uint32_t m[HP][4]; // MASK: the mask values (fp16 bits) of the lane's rows for tokens block start + 4 * g .. + 3
    };
    RawBlock raw[NB];
    const int64_t seq_tok0 = p.pages.page_shift == 0 ? cachestarts[b] : 0;
    const gen_const_tab_t page_row = cachestarts + (int64_t)b * p.pages.stride_b;
    const int64_t head_off = p.addr.row(0, 0, kvh) + g * CPL; // + token * stride_s (+ stride_kv for V)
    auto fetch = [&](RawBlock& r, int64_t kv0) {
        // past the piece's end: its last token again (finite values under a probability of zero)
        if (kv0 > kv_end - 1) kv0 = (kv_end - 1) & ~int64_t(15);
        int64_t j = kv0 + r_lane;
        if (j > kv_end - 1) j = kv_end - 1;
        int64_t t_slab;
        if (p.pages.page_shift == 0) {
            t_slab = seq_tok0 + j;
        } else {
            const int64_t page0 = page_row[kv0 >> p.pages.page_shift]; // (kv0: wave-uniform)
            t_slab = page0 + (j & ((int64_t(1) << p.pages.page_shift) - 1));
        }
        const int64_t rk = t_slab * p.addr.stride_s + head_off, rv = rk + p.addr.stride_kv;
        const uint16_t* sk = reinterpret_cast<const uint16_t*>(p.scale) + rk / kQuantGroup;
        const uint16_t* sv = reinterpret_cast<const uint16_t*>(p.scale) + rv / kQuantGroup;
#pragma unroll
        for (int i = 0; i < NCK; ++i) {
            r.k[i] = *reinterpret_cast<const chunk_t*>(p.cache + rk + CB * i);
            r.v[i] = *reinterpret_cast<const chunk_t*>(p.cache + rv + CB * i);
            r.ks[i] = sk[i];
            r.vs[i] = sv[i];
        }
        if (MASK) {
            const int64_t last = kvlen - 1, j0 = kv0 + 4 * g;
#pragma unroll
            for (int h = 0; h < HP; ++h) {
                const uint16_t* mp = reinterpret_cast<const uint16_t*>(mrow[h]);
#pragma unroll
                for (int i = 0; i < 4; ++i) r.m[h][i] = mp[j0 + i < last ? j0 + i : last];
            }
        }
    };
    auto as_half = [](uint32_t bits16) {
        const uint16_t bits = (uint16_t)bits16;
        half_t h;
        __builtin_memcpy(&h, &bits, 2);
        return h;
    };

    constexpr float kOne = 1.0f;
    const float cs = MASK ? kOne : p.scale_log2; // what the exponentials multiply the held scores by
    float m_run[HP], l_part[HP];
    float4_t o[HP][KC];
#pragma unroll
    for (int h = 0; h < HP; ++h) {
        m_run[h] = -INFINITY, l_part[h] = 0.f;
#pragma unroll
        for (int i = 0; i < KC; ++i) o[h][i] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    // A block is taken out of its registers first (V into the wave's LDS rows as fp16, K through the score products:
    // nothing of it is needed afterwards but the 4 scores a head and the mask values), so that the same registers can
    // be sent for a later block before the rest of the arithmetic.
    float4_t acc[HP];
    float mask4[HP][4];
    auto unpack = [&](const RawBlock& r) {
#pragma unroll
        for (int h = 0; h < HP; ++h) acc[h] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NCK; ++i) {
            *reinterpret_cast<half8_t*>(&Vs[r_lane * LDV + g * CPL + CB * i]) =
                dequant8(r.v[i].x, r.v[i].y, as_half(r.vs[i]));
            const half8_t k8 = dequant8(r.k[i].x, r.k[i].y, as_half(r.ks[i]));
            const half4_t lo = {k8[0], k8[1], k8[2], k8[3]}, hi = {k8[4], k8[5], k8[6], k8[7]};
#pragma unroll
            for (int h = 0; h < HP; ++h) {
                acc[h] = __builtin_amdgcn_mfma_f32_16x16x16f16(lo, qf[h][2 * i], acc[h], 0, 0, 0);
                acc[h] = __builtin_amdgcn_mfma_f32_16x16x16f16(hi, qf[h][2 * i + 1], acc[h], 0, 0, 0);
            }
        }
        if (MASK) {
#pragma unroll
            for (int h = 0; h < HP; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i) mask4[h][i] = (float)as_half(r.m[h][i]) * kLog2e;
        }
    };
    auto block_step = [&](const int64_t kv0) {
        half4_t pf[HP];
        float alpha[HP];
        // tokens kv0 + 4 * g + i of the block exist for i < left (only the piece's last block is ragged)
        const int left = (int)(kv_end - kv0 < 16 ? kv_end - kv0 : 16) - 4 * g;
#pragma unroll
        for (int h = 0; h < HP; ++h) {
            // ---- scores of the lane's row against tokens kv0 + 4 * g + i: raw products without a mask (the scale goes
            // into the exponentials' multiply-add), exp2-domain values with one
            float sc[4];
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = MASK ? __builtin_fmaf(acc[h][i], p.scale_log2, mask4[h][i]) : acc[h][i];
                if (kv0 + 16 > kv_end) v = i < left ? v : -INFINITY; // (wave-uniform condition)
                sc[i] = v;
                mx = fmaxf(mx, v);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run[h], mx);
            // a row that has seen nothing but masked keys so far keeps max -inf: against 0 in the exponents its
            // probabilities are exp2(-inf) = 0, not NaN
            const float m_safe = m_new == -INFINITY ? 0.f : m_new;
            alpha[h] = __builtin_amdgcn_exp2f((m_run[h] - m_safe) * cs);
            const float shift = -m_safe * cs;
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const half_t x = (half_t)__builtin_amdgcn_exp2f(__builtin_fmaf(sc[i], cs, shift));
                pf[h][i] = x;
                psum += (float)x; // the sum of what the second product multiplies
            }
            l_part[h] = l_part[h] * alpha[h] + psum;
            m_run[h] = m_new;
        }
        // the block's V rows, written by the wave's other lanes: LDS operations of one wave complete in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int h = 0; h < HP; ++h) {
#pragma unroll
            for (int db = 0; db < KC; ++db) {
                o[h][db] *= alpha[h];
                // V^T operand: lane (block g, j) receives channel 16 * db + j of tokens 4 * g .. + 3 when lane
                // 4 * i + c of the block addresses token 4 * g + i, channels 16 * db + 4 * c .. + 3
                const half_t* src = &Vs[(4 * g + (r_lane >> 2)) * LDV + h * DH + 16 * db + 4 * (r_lane & 3)];
                const short4_t t =
                    __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)src);
                half4_t a;
                __builtin_memcpy(&a, &t, 8);
                o[h][db] = __builtin_amdgcn_mfma_f32_16x16x16f16(a, pf[h], o[h][db], 0, 0, 0);
            }
        }
        // (the next block's V rows are written after these reads: same wave, in order)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

#pragma unroll
    for (int u = 0; u < NB; ++u) fetch(raw[u], kv_begin + 16 * u);
    for (int64_t kv0 = kv_begin; kv0 < kv_end; kv0 += 16 * NB) {
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int64_t kvu = kv0 + 16 * u;
            if (kvu >= kv_end) break; // wave-uniform
            unpack(raw[u]);
            fetch(raw[u], kvu + 16 * NB);
            block_step(kvu);
        }
    }

#pragma unroll
    for (int h = 0; h < HP; ++h) {
        float l = l_part[h];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        if (!valid) continue;
        if (p.nsplit > 1) {
            const int64_t prow = ((int64_t)b * p.num_heads + head[h]) * p.nsplit + piece;
            float* dst = p.part_o + prow * DH + 4 * g;
#pragma unroll
            for (int db = 0; db < KC; ++db) *reinterpret_cast<float4_t*>(dst + 16 * db) = o[h][db];
            if (g == 0) {
                p.part_ml[prow * 2] = m_run[h] * cs; // (the merge works in the exp2 domain)
                p.part_ml[prow * 2 + 1] = l;
            }
            continue;
        }
        const float inv_l = l > 0.f ? 1.0f / l : 0.f; // a row whose keys were all masked out: zeros
        half_t* dst = p.out + (s0 * p.num_heads + head[h]) * DH + 4 * g;
#pragma unroll
        for (int db = 0; db < KC; ++db) {
            const half4_t r = {(half_t)(o[h][db][0] * inv_l), (half_t)(o[h][db][1] * inv_l),
                               (half_t)(o[h][db][2] * inv_l), (half_t)(o[h][db][3] * inv_l)};
            *reinterpret_cast<half4_t*>(dst + 16 * db) = r;
        }
    }
}

// Combines the pieces of a decode sequence's row: out = sum_s w_s o_s / sum_s w_s l_s, w_s = exp2(m_s - max m). A
// thread per four channels of a row (query head of a decode token), kGenMergeRows<DH> rows to a workgroup.
template <int DH>
constexpr int kGenMergeRows = 256 / (DH / 4);
template <int DH>
__global__ __launch_bounds__(256) void generic_merge_kernel(const GenericParams p) {
    const int r_in_block = threadIdx.x / (DH / 4);
    const int64_t row = (int64_t)blockIdx.x * kGenMergeRows<DH> + r_in_block; // token * num_heads + head over the decode tokens
    const int d4 = (threadIdx.x - r_in_block * (DH / 4)) * 4;
    if (r_in_block >= kGenMergeRows<DH> || row >= (int64_t)p.split_seqs * p.num_heads) return;
    const int64_t b = row / p.num_heads;
    const int64_t kvlen = p.kvstarts[b + 1] - p.kvstarts[b];
    int n = (int)((kvlen + p.piece_tokens - 1) / p.piece_tokens); // the pieces that exist
    if (n > p.nsplit) n = p.nsplit;
    // four pieces' loads go out together; the pieces are folded into a running (maximum, sum, accumulator)
    float M = -INFINITY, L = 0.f;
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < n; s0 += 4) {
        float2 ml[4];
        float4_t o4[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t pr = row * p.nsplit + (s0 + k < n ? s0 + k : n - 1);
            ml[k] = *reinterpret_cast<const float2*>(p.part_ml + pr * 2);
            o4[k] = *reinterpret_cast<const float4_t*>(p.part_o + pr * DH + d4);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float m_new = fmaxf(M, ml[k].x);
            // (a piece without unmasked keys has maximum -inf and weight 0; while nothing else was seen, nothing moves)
            if (s0 + k < n && m_new != -INFINITY) {
                const float wa = __builtin_amdgcn_exp2f(M - m_new), wb = __builtin_amdgcn_exp2f(ml[k].x - m_new);
                acc = acc * wa + o4[k] * wb;
                L = L * wa + ml[k].y * wb;
                M = m_new;
            }
        }
    }
    const float inv = L > 0.f ? 1.0f / L : 0.f; // (no piece with unmasked keys: zeros)
    const half4_t r = {(half_t)(acc[0] * inv), (half_t)(acc[1] * inv), (half_t)(acc[2] * inv), (half_t)(acc[3] * inv)};
    if (d4 < p.head_dim) *reinterpret_cast<half4_t*>(p.out + row * p.head_dim + d4) = r;
}

// two kv heads per wave of the decode kernel: head_dim up to 96 (registers), heads next to each other in the slab
static int generic_decode_heads_per_wave(const GenericParams& p, int head_dim) {
    return head_dim <= 96 && p.kv_heads % 2 == 0 && p.addr.stride_h == head_dim ? 2 : 1;
}

template <int DH>
static void launch_one(const GenericParams& p, int64_t blocks, int64_t decode_blocks, int row_blocks, hipStream_t stream) {
    if (decode_blocks > 0) { // the decode sequences, a wave per (sequence, kv head or pair of them, piece)
        const dim3 grid((unsigned)decode_blocks), block(256);
        if constexpr (DH <= 96) {
            if (generic_decode_heads_per_wave(p, DH) == 2) {
                if (p.mask)
                    hipLaunchKernelGGL((generic_decode_kernel<DH, true, 2>), grid, block, 0, stream, p);
                else
                    hipLaunchKernelGGL((generic_decode_kernel<DH, false, 2>), grid, block, 0, stream, p);
                goto decode_launched;
            }
        }
        if (p.mask)
            hipLaunchKernelGGL((generic_decode_kernel<DH, true, 1>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((generic_decode_kernel<DH, false, 1>), grid, block, 0, stream, p);
    }
decode_launched:
    if (blocks > 0) {
        GenericParams t = p;
        if (decode_blocks > 0) t.first_seq = p.split_seqs, t.split_seqs = 0, t.nsplit = 1;
        if constexpr (gen_two_row_blocks(DH)) {
            if (row_blocks == 2) {
                hipLaunchKernelGGL((generic_attention_kernel<DH, 2>), dim3((unsigned)blocks), dim3(256), 0, stream, t);
                goto tiles_launched;
            }
        }
        hipLaunchKernelGGL((generic_attention_kernel<DH, 1>), dim3((unsigned)blocks), dim3(256), 0, stream, t);
    }
tiles_launched:
    if (p.nsplit > 1 && p.split_seqs > 0)
        hipLaunchKernelGGL(generic_merge_kernel<DH>,
                           dim3((unsigned)(((int64_t)p.split_seqs * p.num_heads + kGenMergeRows<DH> - 1) / kGenMergeRows<DH>)),
                           dim3(256), 0, stream, p);
}

bool generic_head_dim_supported(int head_dim) {
    return head_dim >= 16 && head_dim <= 256 && head_dim % 16 == 0;
}
// the head_dim the kernels are compiled for: the next multiple of 32
static int generic_kernel_head_dim(int head_dim) { return (head_dim + 31) / 32 * 32; }

// skip_first: the tile kernel leaves out the first `skip_first` sequences (decode sequences that another kernel serves)
static pplhip_retcode launch_generic(GenericParams& p, int head_dim, int64_t max_seqlen, hipStream_t stream,
                                     int skip_first = 0) {
    if (!generic_head_dim_supported(head_dim))
        PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "head_dim %d: must be a multiple of 16 between 16 and 256", head_dim);
    p.scale_log2 = kLog2e / sqrtf((float)head_dim);
    p.head_dim = head_dim;
    const int dh = generic_kernel_head_dim(head_dim);
    const bool padded = dh != head_dim;
    // tiles of 128 rows (two blocks of 16 per wave) where a sequence has more than 64 rows
    const int row_blocks = gen_two_row_blocks(dh) && max_seqlen * p.rep > kGenRows ? 2 : 1;
    const int64_t tiles = (max_seqlen * p.rep + kGenRows * row_blocks - 1) / (kGenRows * row_blocks);
    if (tiles <= 0 || p.batch <= 0) return PPLHIP_RC_SUCCESS;
    // p.split_seqs: the decode sequences (the first of the batch, one new token each, all of whose keys are in the slab)
    if (p.nsplit < 1) p.nsplit = 1;
    p.first_seq = 0;
    int64_t blocks, decode_blocks = 0;
    if (skip_first > 0) {
        p.nsplit = 1, p.split_seqs = 0;
        p.first_seq = skip_first;
        const int64_t groups = tiles * (int64_t)(p.batch - skip_first);
        blocks = (groups + 7) / 8 * 8 * p.kv_heads;
    } else if (p.split_seqs > 0 && p.rep <= 16 && !padded && (p.pages.page_shift == 0 || p.pages.page_shift >= 4)) {
        // generic_decode_kernel takes them; the tile kernel the rest of the batch
        if (p.nsplit == 1) p.piece_tokens = 0x7fffffc0; // the whole sequence
        decode_blocks = ((int64_t)p.split_seqs * p.nsplit * (p.kv_heads / generic_decode_heads_per_wave(p, head_dim)) + 3) / 4;
        const int64_t groups = tiles * (int64_t)(p.batch - p.split_seqs);
        blocks = (groups + 7) / 8 * 8 * p.kv_heads;
    } else {
        // the tile kernel takes everything: pieces for decode tokens of one row tile, else whole sequences
        if (p.nsplit == 1 || p.rep > kGenRows) p.nsplit = 1, p.split_seqs = 0;
        const int64_t groups = tiles * (int64_t)p.batch + (int64_t)p.split_seqs * (p.nsplit - 1);
        blocks = (groups + 7) / 8 * 8 * p.kv_heads;
    }
    if (tiles > 0x7fffffffLL || blocks > 0x7fffffffLL || decode_blocks > 0x7fffffffLL)
        PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "attention: too many row tiles");
    p.tiles_max = (int32_t)tiles;
    switch (dh) {
        case 32: launch_one<32>(p, blocks, decode_blocks, row_blocks, stream); break;
        case 64: launch_one<64>(p, blocks, decode_blocks, row_blocks, stream); break;
        case 96: launch_one<96>(p, blocks, decode_blocks, row_blocks, stream); break;
        case 128: launch_one<128>(p, blocks, decode_blocks, row_blocks, stream); break;
        case 160: launch_one<160>(p, blocks, decode_blocks, row_blocks, stream); break;
        case 192: launch_one<192>(p, blocks, decode_blocks, row_blocks, stream); break;
        case 224: launch_one<224>(p, blocks, decode_blocks, row_blocks, stream); break;
        default: launch_one<256>(p, blocks, decode_blocks, row_blocks, stream); break;
    }
    PPLHIP_CHECK_LAUNCH("generic_attention");
    return PPLHIP_RC_SUCCESS;
}

// How many pieces the longest decode sequence of a call is cut into (1: no pieces). A piece is one to sixteen tiles of
// keys: sixteen when even whole sequences would fill the chip many times over (fewer partial results and starts),
// fewer when the batch is small; more than 64 pieces are not made (the pieces of a very long sequence grow instead). Host-only, a
// function of the argument block and the CU count.
constexpr int kGenMaxPieces = 64;
int generic_decode_splits(const pplhip_mhca_args* a, int cu_count) {
    // (more than 64 query heads per kv head: a decode token has more than one row tile; left whole)
    if (a->decoding_batches <= 0 || a->max_kvlen < 2 * 64 || a->num_heads / a->num_kv_heads > kGenRows) return 1;
    const int64_t tiles = (a->max_kvlen + 63) / 64; // of the longest sequence
    const int64_t wgs = a->decoding_batches * a->num_kv_heads;
    int64_t per = wgs * tiles / ((int64_t)cu_count * 32); // tiles a piece: about 32 pieces per CU at the least
    per = per < 1 ? 1 : per > 16 ? 16 : per;
    if (per * kGenMaxPieces < tiles) per = (tiles + kGenMaxPieces - 1) / kGenMaxPieces;
    const int64_t n = (tiles + per - 1) / per;
    return n < 2 ? 1 : (int)n;
}
// keys per piece when the longest sequence (max_kvlen keys) is cut into nsplit pieces: whole tiles
static int generic_piece_tokens(int64_t max_kvlen, int nsplit) {
    return (int)(((max_kvlen + nsplit - 1) / nsplit + 63) / 64 * 64);
}
uint64_t generic_workspace_bytes(const pplhip_mhca_args* a, int nsplit) {
    if (nsplit <= 1) return 0;
    return (uint64_t)a->decoding_batches * a->num_heads * nsplit * (generic_kernel_head_dim(a->head_dim) + 2) * sizeof(float);
}

// MultiHeadCacheAttention through the general kernel; the new tokens are already in the slab.
pplhip_retcode launch_generic_mhca(const pplhip_mhca_args* a, int nsplit, void* ws, hipStream_t stream,
                                   bool prompts_only) {
    GenericParams p;
    p.nsplit = nsplit < 1 ? 1 : nsplit;
    p.split_seqs = (int32_t)a->decoding_batches;
    p.piece_tokens = generic_piece_tokens(a->max_kvlen, p.nsplit);
    p.part_o = (float*)ws;
    p.part_ml = p.nsplit > 1 ? (float*)ws + (size_t)a->decoding_batches * a->num_heads * p.nsplit *
                                                generic_kernel_head_dim(a->head_dim)
                             : nullptr;
    if (p.nsplit > 1 && ws == nullptr)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "attention: needs the workspace reported by pplhip_mhca_prepare");
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
    p.k16_holds_new_tokens = 1;
    p.is_causal = a->is_causal;
    const int64_t max_rows_tokens = a->batch > a->decoding_batches ? a->max_seqlen : 1;
    return launch_generic(p, a->head_dim, max_rows_tokens, stream, prompts_only ? (int)a->decoding_batches : 0);
}

pplhip_retcode launch_generic_mha(const pplhip_mha_args* a, hipStream_t stream) {
    GenericParams p;
    p.nsplit = 1;
    p.split_seqs = 0;
    p.piece_tokens = 0;
    p.part_o = p.part_ml = nullptr;
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
    p.k16_holds_new_tokens = 0; // key / value hold every key of a sequence, packed by kvstarts
    p.is_causal = a->is_causal;
    return launch_generic(p, a->head_dim, a->max_seqlen, stream);
}

} // namespace pplhip
