// Shared host/device helpers of the gfx950 kernel library (internal; the public surface is the C ABI header).
#ifndef PPLHIP_CSRC_COMMON_H_
#define PPLHIP_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/ppl_llm_kernel_hip.h"

namespace pplhip {

// thread-local text behind pplhip_last_error()
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

#define PPLHIP_FAIL(rc, ...)              \
    do {                                  \
        ::pplhip::set_error(__VA_ARGS__); \
        return (rc);                      \
    } while (0)

#define PPLHIP_CHECK_LAUNCH(what)                                                                 \
    do {                                                                                          \
        hipError_t e_ = hipGetLastError();                                                        \
        if (e_ != hipSuccess)                                                                     \
            PPLHIP_FAIL(PPLHIP_RC_DEVICE_RUNTIME_ERROR, "%s: %s", (what), hipGetErrorString(e_)); \
    } while (0)

constexpr int kQuantGroup = 8;
constexpr int kWave = 64;

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// Where one KV head's row of `head_dim` int8 channels starts, and the matching row of head_dim/8 fp16 scales.
struct CacheAddr {
    int64_t stride_s, stride_l, stride_h, stride_kv;
    int32_t layer;
    __host__ __device__ inline int64_t row(int64_t tok, int kv, int head) const {
        return tok * stride_s + (int64_t)layer * stride_l + (int64_t)kv * stride_kv + (int64_t)head * stride_h;
    }
};

// Where token j of sequence b lives in the slab: a contiguous region per sequence (cache_mode 0, page_shift == 0) or
// pages of 2^page_shift tokens listed per sequence in a [batch, stride_b] table (cache_mode 1).
struct PageMap {
    const int64_t* cachestarts;
    int64_t stride_b;
    int32_t page_shift;
    __device__ inline int64_t token(int64_t b, int64_t j) const {
        if (page_shift == 0) return cachestarts[b] + j;
        return cachestarts[b * stride_b + (j >> page_shift)] + (j & ((int64_t(1) << page_shift) - 1));
    }
};
inline int page_shift_of(int cache_mode, int page_size) { // host: 0 for the contiguous mode
    if (cache_mode == 0) return 0;
    int s = 0;
    while ((1 << s) < page_size) ++s;
    return s;
}

// One quantisation group: 8 fp16 values -> 8 int8 + one fp16 scale. THE rounding rule of the KV cache (bit-exact
// contract with the CPU oracle): s = max(fp16(absmax / 127), fp16(1e-5)), q = int8(rint(fp16(x / s))).
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
    // x / s as x * (1 / s): one correctly rounded division per group instead of eight. The fp32 products differ from
    // the fp32 quotients in the last bits, the int8 results do not: for every fp16 x (all 65 536 patterns) and every
    // scale the rule can produce (all fp16 from eps to +inf) both ways give the same q, checked by enumerating the
    // pairs on the device with this file's compiler flags (no contraction, IEEE division).
    const float rs = 1.0f / sf;
    uint32_t w[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float ratio = (float)(half_t)((float)x[i] * rs);
        float r = rintf(ratio);
        r = fminf(fmaxf(r, -128.f), 127.f);
        const int qi = (int)r;
        w[i >> 2] |= (uint32_t)(qi & 0xff) << (8 * (i & 3));
    }
    *q_out = make_uint2(w[0], w[1]);
    *s_out = s;
}

// ---- the way back: int8 -> fp16 without a trip through fp32
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
// 8 int8 channels (one quantisation group) -> 8 fp16 values times the group scale
__device__ inline half8_t dequant8(uint32_t w0, uint32_t w1, half_t scale) {
    const half2_t s2 = {scale, scale};
    const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
    const half2_t a = dequant2(widen_lo(x0), s2), b = dequant2(widen_hi(x0), s2);
    const half2_t c = dequant2(widen_lo(x1), s2), d = dequant2(widen_hi(x1), s2);
    return half8_t{a.x, a.y, b.x, b.y, c.x, c.y, d.x, d.y};
}

// first index b in [0, n) with starts[b+1] > x  (starts is a non-decreasing prefix-sum table with n+1 entries)
__device__ inline int find_sequence(const int64_t* __restrict__ starts, int n, int64_t x) {
    int lo = 0, hi = n;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (starts[mid + 1] > x)
            hi = mid;
        else
            lo = mid + 1;
    }
    return lo;
}

// The same index for an x that every ACTIVE lane of the wave shares (inactive lanes are allowed): the table is read
// one entry per active lane at a time and the entries <= x are counted, so the look-up costs one memory latency per
// 64 sequences instead of a chain of log2(n) dependent loads.
__device__ inline int find_sequence_wave(const int64_t* __restrict__ starts, int n, int64_t x) {
    const uint64_t active = __ballot(1);
    const int lane = threadIdx.x & 63;
    const int rank = __popcll(active & ((uint64_t(1) << lane) - 1));
    const int width = __popcll(active);
    int count = 0;
    for (int base = 1; base <= n; base += width) {
        const int i = base + rank;
        const bool le = i <= n && starts[i] <= x;
        count += __popcll(__ballot(le));
    }
    return count;
}

inline int ceil_div(int64_t a, int64_t b) {
    return (int)((a + b - 1) / b);
}

// launchers implemented in the .hip files
// first_token: packed new tokens before it are skipped (the decode kernel writes the decode tokens itself)
pplhip_retcode launch_kv_quantize_write(const pplhip_kv_write_args* a, hipStream_t stream, int64_t first_token = 0,
                                        int64_t end_token = -1);
pplhip_retcode launch_kv_gather_dequant(const pplhip_kv_cache_args* a, hipStream_t stream);
// cache-prefill: dequantises the cached K/V of sequences [decoding_batches, batch) into packed fp16 rows
// [kv token - kvstarts[decoding_batches], kv head, head_dim] at `key_out` / `value_out`; `max_tokens` bounds the rows
pplhip_retcode launch_kv_stage_prefill(const pplhip_mhca_args* a, half_t* key_out, half_t* value_out, int64_t max_tokens,
                                       hipStream_t stream);
// whether (and where in the workspace) a cache-prefill call stages its K/V as fp16: see pplhip_mhca_plan
int64_t prefill_staging_tokens(const pplhip_mhca_args* a);
int decode_heads_per_block(int kv_heads);
// head dims 64 / 32 whose decode sequences run the head_dim-128 decode kernel over groups of 2 / 4 neighbouring kv
// heads: the number of such groups, or 0 when the call does not qualify
int decode_virtual_heads(const pplhip_mhca_args* a);
bool prefill_writes_new_tokens(const pplhip_mhca_args* a);
int decode_blocks_per_cu();
int decode_waves_per_block();
// new_tokens_in_slab: the decode sequences' new tokens were quantised into the slab by an earlier launch
pplhip_retcode launch_decode(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* ws, hipStream_t stream,
                             bool new_tokens_in_slab = false);
pplhip_retcode launch_prefill(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* ws, hipStream_t stream);
// both, in one launch where the call has decode sequences and prompts
pplhip_retcode launch_decode_and_prefill(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* ws,
                                         hipStream_t stream);
pplhip_retcode launch_mha(const pplhip_mha_args* a, hipStream_t stream);
// the general attention kernel: any head_dim that is a multiple of 16 up to 256, any number of query heads per kv
// head, optional attn_mask. The MHCA form reads the slab, which must already hold the call's new tokens.
bool generic_head_dim_supported(int head_dim);
// nsplit pieces per decode sequence (generic_decode_splits), their partial results in `ws` (generic_workspace_bytes)
int generic_decode_splits(const pplhip_mhca_args* a, int cu_count);
uint64_t generic_workspace_bytes(const pplhip_mhca_args* a, int nsplit);
// prompts_only: the decode sequences of the call are somebody else's (the decode kernel's)
pplhip_retcode launch_generic_mhca(const pplhip_mhca_args* a, int nsplit, void* ws, hipStream_t stream,
                                   bool prompts_only = false);
pplhip_retcode launch_generic_mha(const pplhip_mha_args* a, hipStream_t stream);
// w != null: the launch also quantises the rotated keys and the values of the new tokens into the slab
pplhip_retcode launch_rope(const pplhip_rope_args* a, const pplhip_kv_write_args* w, hipStream_t stream);
pplhip_retcode launch_position_index(const int64_t* d_seqstarts, const int64_t* d_start_pos, int64_t batch,
                                     int64_t total_tokens, int64_t* d_out, hipStream_t stream);
pplhip_retcode launch_pack_tables(const pplhip_pack_args* a, hipStream_t stream);
pplhip_retcode launch_advance_slots(int64_t* kvlen, const int64_t* newlen, int n, hipStream_t stream);
pplhip_retcode launch_check_tables(const pplhip_mhca_args* a, int64_t max_slab_tokens, int32_t* d_flag, hipStream_t stream);
void check_tables_host(const pplhip_mhca_args* a, int64_t max_slab_tokens, int32_t* flag);

} // namespace pplhip

#endif
