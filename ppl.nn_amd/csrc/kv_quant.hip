// Quantize-on-write of new K/V tokens into the int8 group-8 KV slab, and the KeyValueCache op's
// gather + dequantise. Both are pure streaming kernels: one lane owns one group of 8 channels
// (16 B fp16 in, 8 B int8 + 2 B scale out), so a wavefront moves 1 KiB / 512 B + 128 B per instruction.
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
    int32_t groups_per_head; // head_dim / 8
    int64_t total_groups; // S * 2 * kv_heads * groups_per_head
};

__device__ inline void quantize_group8(const uint4 raw, uint2* q_out, half_t* s_out) {
    half_t x[8];
    __builtin_memcpy(x, &raw, 16);
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf((float)x[i]));
    half_t s = (half_t)(amax / 127.0f);
    const half_t eps = (half_t)1e-5f;
    if ((float)s < (float)eps) s = eps;
    const float sf = (float)s;
    uint32_t w[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float ratio = (float)(half_t)((float)x[i] / sf);
        float r = rintf(ratio);
        r = fminf(fmaxf(r, -128.f), 127.f);
        const int qi = (int)r;
        w[i >> 2] |= (uint32_t)(qi & 0xff) << (8 * (i & 3));
    }
    *q_out = make_uint2(w[0], w[1]);
    *s_out = s;
}

__global__ __launch_bounds__(256) void kv_quantize_write_kernel(const QuantWriteParams p) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= p.total_groups) return;
    const int gph = p.groups_per_head;
    const int per_kv = p.kv_heads * gph;
    const int per_tok = 2 * per_kv;
    const int64_t t = g / per_tok; // packed new-token index
    const int r = (int)(g - t * per_tok);
    const int kv = r / per_kv;
    const int r2 = r - kv * per_kv;
    const int head = r2 / gph;
    const int grp = r2 - head * gph;
    // decode sequences come first and hold one token each, so for them the packed token index IS the sequence index:
    // two independent loads settle it; only prompt tokens pay for the binary search (a chain of dependent loads)
    int b;
    if (t < p.batch && p.seqstarts[t] == t && p.seqstarts[t + 1] == t + 1)
        b = (int)t;
    else
        b = find_sequence(p.seqstarts, p.batch, t);
    const int64_t tok = p.pages.token(b, p.start_pos[b] + (t - p.seqstarts[b]));
    const half_t* src = (kv ? p.value : p.key) + ((t * p.kv_heads + head) * gph + grp) * 8;
    const uint4 raw = *reinterpret_cast<const uint4*>(src);
    uint2 q;
    half_t s;
    quantize_group8(raw, &q, &s);
    const int64_t row = p.addr.row(tok, kv, head);
    *reinterpret_cast<uint2*>(p.cache + row + grp * 8) = q;
    p.scale[row / kQuantGroup + grp] = s;
}

pplhip_retcode launch_kv_quantize_write(const pplhip_kv_write_args* a, hipStream_t stream) {
    if (a->total_new_tokens == 0 || a->batch == 0) return PPLHIP_RC_SUCCESS;
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
    p.groups_per_head = a->head_dim / kQuantGroup;
    p.total_groups = a->total_new_tokens * 2 * (int64_t)a->num_kv_heads * p.groups_per_head;
    const int64_t blocks = (p.total_groups + 255) / 256;
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "kv_quantize_write: too many groups");
    hipLaunchKernelGGL(kv_quantize_write_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("kv_quantize_write");
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
    int64_t total_groups; // total_kv_tokens * 2 * kv_heads * groups_per_head
};

__global__ __launch_bounds__(256) void kv_gather_dequant_kernel(const GatherParams p) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= p.total_groups) return;
    const int gph = p.groups_per_head;
    const int per_kv = p.kv_heads * gph;
    const int per_tok = 2 * per_kv;
    const int64_t j = g / per_tok; // packed kv-token index
    const int r = (int)(g - j * per_tok);
    const int kv = r / per_kv;
    const int r2 = r - kv * per_kv;
    const int head = r2 / gph;
    const int grp = r2 - head * gph;
    const int b = find_sequence(p.kvstarts, p.batch, j);
    const int64_t tok = p.cachestarts[b] + (j - p.kvstarts[b]);
    const int64_t row = p.addr.row(tok, kv, head);
    const uint2 q = *reinterpret_cast<const uint2*>(p.cache + row + grp * 8);
    const float s = (float)p.scale[row / kQuantGroup + grp];
    half_t o[8];
    const uint32_t w[2] = {q.x, q.y};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int qi = (int)(int8_t)((w[i >> 2] >> (8 * (i & 3))) & 0xff);
        o[i] = (half_t)((float)qi * s); // the fp32 product is exact; one rounding to fp16
    }
    uint4 packed;
    __builtin_memcpy(&packed, o, 16);
    half_t* dst = (kv ? p.value_out : p.key_out) + ((j * p.kv_heads + head) * gph + grp) * 8;
    *reinterpret_cast<uint4*>(dst) = packed;
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
    p.total_groups = a->total_kv_tokens * 2 * (int64_t)w->num_kv_heads * p.groups_per_head;
    const int64_t blocks = (p.total_groups + 255) / 256;
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "kv_gather_dequant: too many groups");
    hipLaunchKernelGGL(kv_gather_dequant_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("kv_gather_dequant");
    return PPLHIP_RC_SUCCESS;
}

} // namespace pplhip
