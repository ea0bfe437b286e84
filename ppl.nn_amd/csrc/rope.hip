// opmx.dynamic_batching::RotaryPositionEmbedding and ::PositionIndex over ragged packed batches: the step that
// precedes attention and uses the same seqstarts / start_pos tables.
//
// Both are streaming kernels (HBM roofline): RotaryPositionEmbedding reads and writes every query and key element
// once, 16 bytes per lane; the angle of a (position, channel pair) is formed in float64 (position * theta^(-2i/d),
// reduced mod 2*pi before it is narrowed), because a float32 product loses the low bits of a 100k-token position;
// once per token (workgroup), shared through LDS.
// Pair i rotates by position * theta^(-2i / rotary_dim); its two channels are (2i, 2i + 1) or (i, i + rotary_dim / 2),
// the caller's pair_layout; channels >= rotary_dim pass through.
//
// The same kernel can quantise the new tokens into the KV slab on the way (rope_kernel<true>): the 8 channels a lane
// rotates are exactly one quantisation group, so the rotated key group is quantised from the registers it is written
// to rotated_key from (the fp16-rounded values, i.e. the bytes are those of quantising rotated_key afterwards), and the
// value rows ride along as rows that are only quantised. One launch then replaces the rotary launch and the
// quantize-on-write launch, and the key and value rows are read once instead of twice.
#include "common.h"

namespace pplhip {

struct RopeParams {
    const half_t* q;
    const half_t* k;
    half_t* q_out;
    half_t* k_out;
    const int64_t* seqstarts;
    const int64_t* start_pos;
    int32_t batch;
    int32_t num_heads, num_key_heads;
    int32_t head_dim, rotary_dim;
    int32_t bypass_key;
    int32_t half_split; // pairs are (i, i + rotary_dim / 2) instead of (2i, 2i + 1)
    int32_t scaling_type;
    int32_t max_position_embeddings;
    double log2_theta;
    double scaling_factor;
    // rope_kernel<true> only: where the new tokens' K (rotated) and V go in the slab
    const half_t* v; // current_value [S, num_key_heads, head_dim]
    int8_t* cache;
    half_t* scale;
    PageMap pages;
    CacheAddr addr;
};

constexpr double kTwoPi = 6.283185307179586476925286766559;
constexpr int kMaxRotaryPairs = 1024; // rotary_dim <= head_dim <= 2048 (checked at the entry point)

template <bool WRITE_KV>
__global__ __launch_bounds__(256) void rope_kernel(const RopeParams p) {
    // cosine and sine of the token's rotary_dim / 2 angles: each is formed once per workgroup (a float64 exp2, a
    // reduction mod 2 pi, cosf and sinf: several hundred instructions, which every lane used to repeat for its own pairs
    // and which then took longer than the kernel's memory traffic) and handed to the lanes through LDS
    __shared__ float cos_tab[kMaxRotaryPairs], sin_tab[kMaxRotaryPairs];
    const int64_t t = blockIdx.x; // packed token
    const int cpr = p.head_dim / 8; // 16-byte chunks per head row
    const int rows_per_pass = 256 / cpr;
    const int slot = threadIdx.x / cpr;
    const int chunk = threadIdx.x - slot * cpr;

    // (every lane of the workgroup looks for the same token: one table read per lane and a count, one memory round
    // trip instead of a binary search's chain of them)
    const int b = find_sequence_wave(p.seqstarts, p.batch, t);
    const int64_t s0 = p.seqstarts[b];
    const int64_t sp = p.start_pos[b];
    double pos = (double)(sp + (t - s0));
    double log2_theta = p.log2_theta;
    if (p.scaling_type == PPLHIP_ROPE_SCALING_LINEAR) {
        pos /= p.scaling_factor;
    } else if (p.scaling_type == PPLHIP_ROPE_SCALING_DYNAMIC) {
        const double total = (double)(sp + (p.seqstarts[b + 1] - s0));
        if (total > (double)p.max_position_embeddings) {
            const double grow = p.scaling_factor * total / (double)p.max_position_embeddings - (p.scaling_factor - 1.0);
            log2_theta += log2(grow) * ((double)p.rotary_dim / (double)(p.rotary_dim - 2));
        }
    }
    // The lane owns the 8 channels 8*chunk .. +7 of every head row it visits. Interleaved layout: they are the 4 whole
    // pairs 4*chunk .. +3. Half-split layout: they are one half of the 8 pairs (8*chunk mod rotary_dim/2) .. +7, whose
    // other halves sit rotary_dim/2 channels away (the lane reads them as well; the row is in cache).
    const bool rotate = 8 * chunk < p.rotary_dim; // rotary_dim is a multiple of 8: a chunk is rotated whole or not at all
    const int half = p.rotary_dim / 2;
    const bool upper = p.half_split && 8 * chunk >= half;
    const int npairs = p.half_split ? 8 : 4;
    const int pair0 = p.half_split ? 8 * chunk - (upper ? half : 0) : 4 * chunk;
    for (int i = threadIdx.x; i < half; i += 256) {
        const double inv_freq = exp2(-(2.0 * i / (double)p.rotary_dim) * log2_theta);
        double a = pos * inv_freq;
        a -= kTwoPi * rint(a / kTwoPi);
        cos_tab[i] = cosf((float)a);
        sin_tab[i] = sinf((float)a);
    }
    __syncthreads();
    const bool lane_has_rows = slot < rows_per_pass; // 256 need not be a multiple of the chunks per row
    float cs[8], sn[8];
    if (rotate && lane_has_rows) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (j < npairs) {
                cs[j] = cos_tab[pair0 + j];
                sn[j] = sin_tab[pair0 + j];
            }
        }
    }
    // rows of a token: query heads, key heads and, when the launch also fills the slab, value heads
    const int rows = p.num_heads + p.num_key_heads * (WRITE_KV ? 2 : 1);
    const int64_t slab_tok = WRITE_KV ? p.pages.token(b, sp + (t - s0)) : 0;
    // Half-split pairs rotated in place (outputs aliasing inputs): a lane reads its partner's chunk, which the partner
    // overwrites. Within a wavefront every lane's loads are issued before any lane's store. When the chunks per row do
    // not divide 64 (head_dim 80, 96, 160, ...) a row's lanes can sit in two wavefronts, so a pass then loads, meets
    // at a workgroup barrier, and stores: every thread walks the same number of passes.
    const bool sync_pass = p.half_split && (kWave % cpr) != 0;
    for (int r0 = 0; r0 < rows; r0 += rows_per_pass) {
        const int r = r0 + slot;
        const bool active = lane_has_rows && r < rows;
        const bool is_value = WRITE_KV && r >= p.num_heads + p.num_key_heads;
        const bool is_key = r >= p.num_heads && !is_value;
        const int head = is_value ? r - p.num_heads - p.num_key_heads : (is_key ? r - p.num_heads : r);
        const int64_t off = ((t * (is_key || is_value ? p.num_key_heads : p.num_heads) + head) * (int64_t)p.head_dim) + 8 * chunk;
        const half_t* src = is_value ? p.v : (is_key ? p.k : p.q);
        const bool rotated = active && rotate && !is_value && !(is_key && p.bypass_key);
        uint4 raw = make_uint4(0, 0, 0, 0), other = make_uint4(0, 0, 0, 0);
        if (active) raw = *reinterpret_cast<const uint4*>(src + off);
        // the other halves of this lane's pairs
        if (rotated && p.half_split) other = *reinterpret_cast<const uint4*>(src + off + (upper ? -half : half));
        if (sync_pass) __syncthreads();
        if (!active) continue;
        uint4 res = raw;
        if (rotated) {
            half_t x[8], y[8];
            __builtin_memcpy(x, &raw, 16);
            if (p.half_split) {
                half_t o[8];
                __builtin_memcpy(o, &other, 16);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float mine = (float)x[j], part = (float)o[j];
                    // lower half: y = x cos - partner sin; upper half: y = x cos + partner sin
                    y[j] = (half_t)(upper ? mine * cs[j] + part * sn[j] : mine * cs[j] - part * sn[j]);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float x0 = (float)x[2 * j], x1 = (float)x[2 * j + 1];
                    y[2 * j] = (half_t)(x0 * cs[j] - x1 * sn[j]);
                    y[2 * j + 1] = (half_t)(x1 * cs[j] + x0 * sn[j]);
                }
            }
            __builtin_memcpy(&res, y, 16);
        }
        if (!is_value) *reinterpret_cast<uint4*>((is_key ? p.k_out : p.q_out) + off) = res;
        if (WRITE_KV && (is_key || is_value)) {
            uint2 q;
            half_t sc;
            quantize_group8(res, &q, &sc);
            const int64_t row = p.addr.row(slab_tok, is_value ? 1 : 0, head);
            *reinterpret_cast<uint2*>(p.cache + row + 8 * chunk) = q;
            p.scale[row / kQuantGroup + chunk] = sc;
        }
    }
}

__global__ __launch_bounds__(256) void position_index_kernel(const int64_t* __restrict__ seqstarts,
                                                             const int64_t* __restrict__ start_pos, int batch,
                                                             int64_t total, int64_t* __restrict__ out) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    const int b = find_sequence(seqstarts, batch, t);
    out[t] = start_pos[b] + (t - seqstarts[b]);
}

// w: null, or where the launch also quantises the new tokens to (same tables, key heads and head_dim as `a`: checked
// by the entry point)
pplhip_retcode launch_rope(const pplhip_rope_args* a, const pplhip_kv_write_args* w, hipStream_t stream) {
    if (a->total_tokens == 0 || a->batch == 0) return PPLHIP_RC_SUCCESS;
    RopeParams p;
    p.q = (const half_t*)a->d_query;
    p.k = (const half_t*)a->d_key;
    p.q_out = (half_t*)a->d_rotated_query;
    p.k_out = (half_t*)a->d_rotated_key;
    p.seqstarts = a->d_seqstarts;
    p.start_pos = a->d_start_pos;
    p.batch = (int32_t)a->batch;
    p.num_heads = a->num_heads;
    p.num_key_heads = a->num_key_heads;
    p.head_dim = a->head_dim;
    p.rotary_dim = a->rotary_dim == 0 ? a->head_dim : a->rotary_dim;
    p.bypass_key = a->bypass_key;
    p.half_split = a->pair_layout == PPLHIP_ROPE_PAIRS_HALF_SPLIT;
    p.scaling_type = a->scaling_type;
    p.max_position_embeddings = a->max_position_embeddings;
    p.log2_theta = log2((double)a->theta);
    p.scaling_factor = (double)a->scaling_factor;
    if (a->total_tokens > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "rotary embedding: too many tokens");
    p.v = nullptr;
    p.cache = nullptr;
    p.scale = nullptr;
    p.pages = PageMap{nullptr, 0, 0};
    p.addr = CacheAddr{0, 0, 0, 0, 0};
    if (w) {
        p.v = (const half_t*)w->d_current_value;
        p.cache = (int8_t*)w->d_cache;
        p.scale = (half_t*)w->d_scale;
        p.pages = PageMap{w->d_cachestarts, w->cachestart_stride_b, page_shift_of(w->cache_mode, w->page_size)};
        p.addr = CacheAddr{w->cache_stride_s, w->cache_stride_l, w->cache_stride_h, w->cache_stride_kv, w->layer_idx};
        hipLaunchKernelGGL(rope_kernel<true>, dim3((unsigned)a->total_tokens), dim3(256), 0, stream, p);
    } else {
        hipLaunchKernelGGL(rope_kernel<false>, dim3((unsigned)a->total_tokens), dim3(256), 0, stream, p);
    }
    PPLHIP_CHECK_LAUNCH("rotary_position_embedding");
    return PPLHIP_RC_SUCCESS;
}

pplhip_retcode launch_position_index(const int64_t* d_seqstarts, const int64_t* d_start_pos, int64_t batch,
                                     int64_t total_tokens, int64_t* d_out, hipStream_t stream) {
    if (total_tokens == 0 || batch == 0) return PPLHIP_RC_SUCCESS;
    const int64_t blocks = (total_tokens + 255) / 256;
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "position index: too many tokens");
    hipLaunchKernelGGL(position_index_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, d_seqstarts, d_start_pos,
                       (int)batch, total_tokens, d_out);
    PPLHIP_CHECK_LAUNCH("position_index");
    return PPLHIP_RC_SUCCESS;
}

} // namespace pplhip
