// Quantize-on-write of new K/V tokens into the int8 group-8 KV slab, and the KeyValueCache op's
// gather + dequantise. Both are pure streaming kernels over groups of 8 channels (16 B fp16 <-> 8 B int8 + 2 B
// scale); the write kernel gives a lane four consecutive groups, the gather one.
//
// Rounding rule (bit-exact contract with the CPU oracle):
//   a = max|x_i| ; s = max(fp16_rne(float(a) / 127.0f), fp16_rne(1e-5f)) ; q_i = int8(rint(fp16_rne(float(x_i) / float(s))))
// The fp32 divisions are IEEE correctly rounded (HIP's default), conversions are round-to-nearest-even.
#include "common.h"

namespace pplhip {

struct QuantWriteParams {
    const half_t* key;
    const half_t* value;
    const int64_t* seqstarts;
    PageMap pages;
    const int64_t* start_pos;
    int8_t* cache;
    half_t* scale;
    CacheAddr addr;
    int32_t batch;
    int32_t kv_heads;
    int32_t per_tok; // 4-group units per token: 2 * kv_heads * units_per_head
    int32_t units_per_head; // ceil(head_dim / 32): the last unit of a head holds two groups when head_dim % 32 == 16
    int32_t groups_per_head; // head_dim / 8 (even)
    uint32_t inv_units_per_head; // ceil(65536 / units_per_head): r / units_per_head == (r * inv) >> 16 for r < 8192
    int32_t blocks_per_tok, tok_per_block; // one of the two is 1
    uint32_t inv_per_tok; // ceil(65536 / per_tok)
    int64_t first_token, end_token; // packed tokens [first_token, end_token) are written
};

// One thread owns four consecutive groups (64 B of fp16 in, 32 B of int8 + 8 B of scales out) so that enough bytes
// are in flight per CU to cover the memory latency. Thread -> (token, K or V, head, quarter of the head) without
// integer division: a token has per_tok = 2 * kv_heads * ceil(head_dim / 32) such units; a block covers 256 / per_tok
// whole tokens, one token, or a 256-unit slice of one. head_dim is a multiple of 16: a head's last unit holds four
// groups or two.
__global__ __launch_bounds__(256) void kv_quantize_write_kernel(const QuantWriteParams p) {
    int64_t t; // packed new-token index
    int r; // unit index inside the token
    if (p.tok_per_block == 1) {
        const uint32_t tb = blockIdx.x / p.blocks_per_tok; // block-uniform
        t = p.first_token + tb;
        r = (int)(blockIdx.x - tb * p.blocks_per_tok) * 256 + (int)threadIdx.x;
        if (r >= p.per_tok) return;
    } else {
        const int lt = (int)((threadIdx.x * p.inv_per_tok) >> 16); // threadIdx.x / per_tok, exact below 256
        if (lt >= p.tok_per_block) return;
        t = p.first_token + (int64_t)blockIdx.x * p.tok_per_block + lt;
        r = (int)threadIdx.x - lt * p.per_tok;
    }
    if (t >= p.end_token) return;
    const int hi = (int)(((uint32_t)r * p.inv_units_per_head) >> 16); // 0 .. 2 * kv_heads - 1: K heads, then V heads
    const int grp = (r - hi * p.units_per_head) * 4; // first of the unit's four groups
    const int kv = hi >= p.kv_heads;
    const int head = hi - kv * p.kv_heads;
    // the values do not depend on which sequence the token belongs to: their loads go out before the look-up
    const bool four = grp + 4 <= p.groups_per_head; // (else two: the rest of the unit lies past the head's row)
    const uint4* src = reinterpret_cast<const uint4*>((kv ? p.value : p.key) +
                                                      ((t * p.kv_heads + head) * p.groups_per_head + grp) * 8);
    uint4 raw[4];
    raw[0] = src[0];
    raw[1] = src[1];
    raw[2] = four ? src[2] : make_uint4(0, 0, 0, 0);
    raw[3] = four ? src[3] : make_uint4(0, 0, 0, 0);
    // decode sequences come first and hold one token each, so for them the packed token index IS the sequence index:
    // two independent loads settle it; only prompt tokens pay for a search of the table
    int b;
    if (t < p.batch && p.seqstarts[t] == t && p.seqstarts[t + 1] == t + 1) {
        b = (int)t;
    } else {
        // a wave normally sits inside one token: then the table is searched by the whole wave at once
        const int64_t t0 = ((int64_t)__builtin_amdgcn_readfirstlane((int)(t >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)t);
        if (__all(t == t0))
            b = find_sequence_wave(p.seqstarts, p.batch, t0);
        else
            b = find_sequence(p.seqstarts, p.batch, t);
    }
    const int64_t tok = p.pages.token(b, p.start_pos[b] + (t - p.seqstarts[b]));
    uint2 q[4];
    half_t sc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) quantize_group8(raw[i], &q[i], &sc[i]);
    const int64_t row = p.addr.row(tok, kv, head);
    uint4* dst = reinterpret_cast<uint4*>(p.cache + row + grp * 8); // rows and grp * 8 are multiples of 16
    dst[0] = make_uint4(q[0].x, q[0].y, q[1].x, q[1].y);
    if (four) dst[1] = make_uint4(q[2].x, q[2].y, q[3].x, q[3].y);
    uint32_t packed[2];
    __builtin_memcpy(packed, sc, 8);
    uint32_t* sdst = reinterpret_cast<uint32_t*>(p.scale + row / kQuantGroup + grp); // row / 8 and grp are even
    sdst[0] = packed[0];
    if (four) sdst[1] = packed[1];
}

pplhip_retcode launch_kv_quantize_write(const pplhip_kv_write_args* a, hipStream_t stream, int64_t first_token,
                                        int64_t end_token) {
    if (end_token < 0) end_token = a->total_new_tokens;
    const int64_t num_tokens = end_token - first_token;
    if (num_tokens <= 0 || a->batch == 0) return PPLHIP_RC_SUCCESS;
    QuantWriteParams p;
    p.key = (const half_t*)a->d_current_key;
    p.value = (const half_t*)a->d_current_value;
    p.seqstarts = a->d_seqstarts;
    p.pages = PageMap{a->d_cachestarts, a->cachestart_stride_b, page_shift_of(a->cache_mode, a->page_size)};
    p.start_pos = a->d_start_pos;
    p.cache = (int8_t*)a->d_cache;
    p.scale = (half_t*)a->d_scale;
    p.addr = CacheAddr{a->cache_stride_s, a->cache_stride_l, a->cache_stride_h, a->cache_stride_kv, a->layer_idx};
    p.batch = (int32_t)a->batch;
    p.kv_heads = a->num_kv_heads;
    if (a->head_dim <= 0 || a->head_dim % (2 * kQuantGroup) || a->head_dim > 256)
        PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "kv_quantize_write: head_dim must be a multiple of 16, at most 256");
    p.groups_per_head = a->head_dim / kQuantGroup;
    p.units_per_head = (p.groups_per_head + 3) / 4;
    p.inv_units_per_head = (65536u + (uint32_t)p.units_per_head - 1) / (uint32_t)p.units_per_head;
    p.per_tok = 2 * a->num_kv_heads * p.units_per_head;
    if (p.per_tok >= 8192) PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "kv_quantize_write: too many kv heads (%d)", a->num_kv_heads);
    p.blocks_per_tok = p.per_tok >= 256 ? (p.per_tok + 255) / 256 : 1;
    p.tok_per_block = p.per_tok >= 256 ? 1 : 256 / p.per_tok;
    p.inv_per_tok = (65536u + (uint32_t)p.per_tok - 1) / (uint32_t)p.per_tok;
    p.first_token = first_token;
    p.end_token = end_token;
    const int64_t blocks = p.tok_per_block == 1 ? num_tokens * p.blocks_per_tok
                                                : (num_tokens + p.tok_per_block - 1) / p.tok_per_block;
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "kv_quantize_write: too many groups");
    hipLaunchKernelGGL(kv_quantize_write_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("kv_quantize_write");
    return PPLHIP_RC_SUCCESS;
}

// ---- cache-prefill staging: the cached K/V of the prompts (history and the just written new tokens) as packed fp16
// rows, so that attention can run in the fp16 kernel. One thread = four groups (32 int8 + 4 scales in, 64 bytes out).
struct StageParams {
    const int64_t* kvstarts;
    PageMap pages;
    const int8_t* cache;
    const half_t* scale;
    half_t* key_out;
    half_t* value_out;
    CacheAddr addr;
    int32_t first_seq, batch; // sequences [first_seq, batch)
    int32_t kv_heads;
    int32_t per_tok; // 4-group units per token: 2 * kv_heads * 4
    int64_t max_units;
};

__global__ __launch_bounds__(256) void kv_stage_prefill_kernel(const StageParams p) {
    const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (u >= p.max_units) return;
    const int64_t jr = u / p.per_tok; // row of the staging buffers
    const int r = (int)(u - jr * p.per_tok);
    const int64_t j = p.kvstarts[p.first_seq] + jr; // packed kv-token index
    if (j >= p.kvstarts[p.batch]) return; // the grid covers the worst case (every prompt max_kvlen long)
    const int hi = r >> 2, grp = (r & 3) * 4; // K heads then V heads; first of the unit's four groups
    const int kv = hi >= p.kv_heads, head = hi - kv * p.kv_heads;
    int b;
    {
        const int64_t j0 = ((int64_t)__builtin_amdgcn_readfirstlane((int)(j >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)j);
        const int64_t* starts = p.kvstarts + p.first_seq;
        const int n = p.batch - p.first_seq;
        b = p.first_seq + (__all(j == j0) ? find_sequence_wave(starts, n, j0) : find_sequence(starts, n, j));
    }
    const int64_t tok = p.pages.token(b, j - p.kvstarts[b]);
    const int64_t row = p.addr.row(tok, kv, head);
    const uint4* src = reinterpret_cast<const uint4*>(p.cache + row + grp * 8); // rows and grp * 8: multiples of 16
    const uint4 q0 = src[0], q1 = src[1];
    const uint32_t* ssrc = reinterpret_cast<const uint32_t*>(p.scale + row / kQuantGroup + grp);
    const uint32_t s01 = ssrc[0], s23 = ssrc[1];
    const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    const uint32_t sw[2] = {s01, s23};
    uint4* dst = reinterpret_cast<uint4*>((kv ? p.value_out : p.key_out) + ((jr * p.kv_heads + head) * 16 + grp) * 8);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        half_t sc;
        const uint16_t sbits = (uint16_t)(sw[g >> 1] >> (16 * (g & 1)));
        __builtin_memcpy(&sc, &sbits, 2);
        const half8_t o = dequant8(qw[2 * g], qw[2 * g + 1], sc); // = fp16(float(q) * float(scale)), one rounding
        uint4 packed;
        __builtin_memcpy(&packed, &o, 16);
        dst[g] = packed;
    }
}

// The staging pass moves 5.25 bytes per cached channel (1.25 read, 2 written, 2 read back) and lets the prompts run in
// the fp16 kernel (about 1.0 against 0.6 PFLOP/s for the kernel that dequantises the slab itself on 8 k-token
// contexts): it pays from chunks of roughly 1024 / (query heads per kv head) new tokens per prompt on. Staging rows
// exist for the worst case the host can bound -- every prompt max_kvlen long -- and are capped at 1 GiB.
int64_t prefill_staging_tokens(const pplhip_mhca_args* a) {
    const int64_t npre = a->batch - a->decoding_batches;
    if (!a->enable_cache_prefill || npre <= 0 || a->head_dim != 128) return 0;
    const int64_t prompt_tokens = a->total_new_tokens - a->decoding_batches;
    const int64_t rep = a->num_heads / a->num_kv_heads;
    if (prompt_tokens * rep < 1024 * npre) return 0;
    const int64_t tokens = npre * a->max_kvlen;
    if (tokens * 2 * a->num_kv_heads * a->head_dim * (int64_t)sizeof(half_t) > (int64_t(1) << 30)) return 0;
    return tokens;
}

pplhip_retcode launch_kv_stage_prefill(const pplhip_mhca_args* a, half_t* key_out, half_t* value_out, int64_t max_tokens,
                                       hipStream_t stream) {
    StageParams p;
    p.kvstarts = a->d_kvstarts;
    p.pages = PageMap{a->d_cachestarts, a->cachestart_stride_b, page_shift_of(a->cache_mode, a->page_size)};
    p.cache = (const int8_t*)a->d_cache;
    p.scale = (const half_t*)a->d_scale;
    p.key_out = key_out;
    p.value_out = value_out;
    p.addr = CacheAddr{a->cache_stride_s, a->cache_stride_l, a->cache_stride_h, a->cache_stride_kv, a->layer_idx};
    p.first_seq = (int32_t)a->decoding_batches;
    p.batch = (int32_t)a->batch;
    p.kv_heads = a->num_kv_heads;
    p.per_tok = 2 * a->num_kv_heads * 4;
    p.max_units = max_tokens * p.per_tok;
    const int64_t blocks = (p.max_units + 255) / 256;
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "kv_stage_prefill: too many groups");
    hipLaunchKernelGGL(kv_stage_prefill_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("kv_stage_prefill");
    return PPLHIP_RC_SUCCESS;
}

struct GatherParams {
    const int64_t* kvstarts;
    const int64_t* cachestarts;
    const int8_t* cache;
    const half_t* scale;
    half_t* key_out;
    half_t* value_out;
    CacheAddr addr;
    int32_t batch;
    int32_t kv_heads;
    int32_t groups_per_head;
    int64_t total_units; // total_kv_tokens * 2 * kv_heads * ceil(groups_per_head / 4)
};

// A thread takes four groups (32 channels) of one (token, K or V, head): 32 bytes of int8 and four scales in, 64 bytes
// of fp16 out; the index arithmetic (three divisions) is spent once per 32 channels.
__global__ __launch_bounds__(256) void kv_gather_dequant_kernel(const GatherParams p) {
    const int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; // unit of four groups
    if (u >= p.total_units) return;
    const int uph = (p.groups_per_head + 3) / 4; // units per head (the last holds two groups when head_dim % 32 == 16)
    const int per_kv = p.kv_heads * uph;
    const int per_tok = 2 * per_kv;
    // packed kv-token index (a 32-bit division where the numbers allow it)
    const int64_t j = (uint64_t)u >> 32 ? u / per_tok : (int64_t)((uint32_t)u / (uint32_t)per_tok);
    const int r = (int)(u - j * per_tok);
    const int kv = r / per_kv;
    const int r2 = r - kv * per_kv;
    const int head = r2 / uph;
    const int grp = (r2 - head * uph) * 4; // first of the unit's four groups
    int b;
    {
        const int64_t j0 = ((int64_t)__builtin_amdgcn_readfirstlane((int)(j >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)j);
        if (__all(j == j0))
            b = find_sequence_wave(p.kvstarts, p.batch, j0);
        else
            b = find_sequence(p.kvstarts, p.batch, j);
    }
    const int64_t tok = p.cachestarts[b] + (j - p.kvstarts[b]);
    const int64_t row = p.addr.row(tok, kv, head);
    const uint4* src = reinterpret_cast<const uint4*>(p.cache + row + grp * 8); // rows and grp * 8: multiples of 16
    const bool four = grp + 4 <= p.groups_per_head;
    const uint4 q0 = src[0], q1 = four ? src[1] : make_uint4(0, 0, 0, 0);
    const uint32_t* ssrc = reinterpret_cast<const uint32_t*>(p.scale + row / kQuantGroup + grp);
    const uint32_t sw[2] = {ssrc[0], four ? ssrc[1] : 0u};
    const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    uint4* dst = reinterpret_cast<uint4*>((kv ? p.value_out : p.key_out) +
                                          ((j * p.kv_heads + head) * p.groups_per_head + grp) * 8);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        half_t sc;
        const uint16_t sbits = (uint16_t)(sw[g >> 1] >> (16 * (g & 1)));
        __builtin_memcpy(&sc, &sbits, 2);
        const half8_t o = dequant8(qw[2 * g], qw[2 * g + 1], sc); // = fp16(float(q) * float(scale)), one rounding
        uint4 packed;
        __builtin_memcpy(&packed, &o, 16);
        if (g < 2 || four) dst[g] = packed;
    }
}

pplhip_retcode launch_kv_gather_dequant(const pplhip_kv_cache_args* a, hipStream_t stream) {
    if (a->total_kv_tokens == 0 || a->write.batch == 0) return PPLHIP_RC_SUCCESS;
    const pplhip_kv_write_args* w = &a->write;
    GatherParams p;
    p.kvstarts = a->d_kvstarts;
    p.cachestarts = w->d_cachestarts;
    p.cache = (const int8_t*)w->d_cache;
    p.scale = (const half_t*)w->d_scale;
    p.key_out = (half_t*)a->d_key_out;
    p.value_out = (half_t*)a->d_value_out;
    p.addr = CacheAddr{w->cache_stride_s, w->cache_stride_l, w->cache_stride_h, w->cache_stride_kv, w->layer_idx};
    p.batch = (int32_t)w->batch;
    p.kv_heads = w->num_kv_heads;
    p.groups_per_head = w->head_dim / kQuantGroup;
    p.total_units = a->total_kv_tokens * 2 * (int64_t)w->num_kv_heads * ((p.groups_per_head + 3) / 4);
    const int64_t blocks = (p.total_units + 255) / 256;
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "kv_gather_dequant: too many groups");
    hipLaunchKernelGGL(kv_gather_dequant_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("kv_gather_dequant");
    return PPLHIP_RC_SUCCESS;
}

} // namespace pplhip
