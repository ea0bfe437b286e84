// C ABI entry points: argument validation (same outcomes as the reference wrapper's checks), the split-k
// heuristic, and the launch sequence write -> decode(+merge) -> prefill on the caller's stream.
#include <stdarg.h>
#include <atomic>
#include <stdlib.h>
#include <string.h>

#include "common.h"

namespace pplhip {

static thread_local char g_last_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
}

// Scratch of the entry point that allocates nothing (pplhip_mhca_forward_noalloc): split-k partial results and the
// per-range first-sequence table of one call. Every GPU the library runs on holds its own copy of the array until the
// process ends. The name below is a host-side stand-in, not a device address: host code only ever uses the per-device
// address that hipGetSymbolAddress returned.
constexpr uint64_t kNoAllocScratchBytes = 16ull << 20;
static __device__ __align__(256) unsigned char g_noalloc_scratch[kNoAllocScratchBytes];
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_noalloc_scratch_ptr[kMaxDevices];

// the current device's copy of the scratch array (looked up once per device, with that device current)
static pplhip_retcode noalloc_scratch_of_current_device(void** out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        PPLHIP_FAIL(PPLHIP_RC_DEVICE_RUNTIME_ERROR, "no current HIP device (or more than %d devices)", kMaxDevices);
    void* ptr = g_noalloc_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_noalloc_scratch));
        if (e != hipSuccess || !ptr)
            PPLHIP_FAIL(PPLHIP_RC_DEVICE_RUNTIME_ERROR, "cannot locate the scratch array on device %d: %s", dev,
                        hipGetErrorString(e));
        g_noalloc_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return PPLHIP_RC_SUCCESS;
}

// Compute units the decode plan is sized for: MI355X's 256 until pplhip_init() has read the current device's count.
static std::atomic<int> g_cu_count{256};
static int device_cu_count() {
    return g_cu_count.load(std::memory_order_relaxed);
}

static pplhip_retcode validate_common(int num_kv_heads, int head_dim, int num_layer, int layer_idx,
                                      int64_t stride_s, int64_t stride_l, int64_t stride_h, int64_t stride_kv,
                                      const void* cache, const void* scale) {
    if (num_kv_heads <= 0 || num_layer <= 0 || layer_idx < 0 || layer_idx >= num_layer)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "bad num_kv_heads/num_layer/layer_idx (%d/%d/%d)", num_kv_heads,
                    num_layer, layer_idx);
    if (!generic_head_dim_supported(head_dim))
        PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "head_dim %d: must be a multiple of 16 between 16 and 256", head_dim);
    if (!cache) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "cache pointer is null");
    if (!scale)
        PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "currently only support quantized cache but scale not found");
    if (stride_s <= 0 || stride_s % 16 || stride_l % 16 || stride_h % 16 || stride_kv % 16)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "cache strides must be positive multiples of 16 elements");
    // the kernels keep the offsets inside a stage of 32 (decode) or a tile of 64 (prefill) tokens in 32 bits
    if (stride_s >= (int64_t(1) << 25))
        PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "cache_stride_s %lld: at most 2^25 - 16 elements between tokens",
                    (long long)stride_s);
    if (((uintptr_t)cache & 15) || ((uintptr_t)scale & 15))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "cache and scale must be 16-byte aligned");
    return PPLHIP_RC_SUCCESS;
}

// The tuned kernels take head_dim 128 with at most 16 query heads per kv head and no mask; everything else runs the
// general kernel.
static bool needs_general_kernel(int head_dim, int num_heads, int num_kv_heads, const void* mask) {
    return head_dim != 128 || num_heads / num_kv_heads > 16 || mask != nullptr;
}

// Workspace of the tuned decode path for `ranges` ranges: partial accumulators and (max, sum) pairs per (slot, head),
// slots = ranges + decode sequences, then one int per range (its first sequence).
static uint64_t decode_workspace_bytes(const pplhip_mhca_args* a, int64_t ranges) {
    if (a->decoding_batches <= 0 || ranges <= 0) return 0;
    const uint64_t rows = ((uint64_t)ranges + (uint64_t)a->decoding_batches) * a->num_heads;
    // (rows of 128 channels also for the head dims that run this kernel over groups of kv heads)
    return rows * (128 + 2) * sizeof(float) + (uint64_t)ranges * sizeof(int32_t);
}

static pplhip_retcode validate_mask(const void* mask, int64_t stride_h, int64_t stride_q) {
    if (!mask) return PPLHIP_RC_SUCCESS;
    if ((uintptr_t)mask & 1) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "attn_mask must be 2-byte aligned");
    if (stride_q <= 0 || stride_h < 0)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "attn_mask strides: stride_q %lld must be positive, stride_h %lld not negative",
                    (long long)stride_q, (long long)stride_h);
    return PPLHIP_RC_SUCCESS;
}

static void write_args_from_mhca(const pplhip_mhca_args* a, pplhip_kv_write_args* w) {
    memset(w, 0, sizeof(*w));
    w->d_current_key = a->d_current_key;
    w->d_current_value = a->d_current_value;
    w->d_seqstarts = a->d_seqstarts;
    w->d_cachestarts = a->d_cachestarts;
    w->d_start_pos = a->d_start_pos;
    w->batch = a->batch;
    w->total_new_tokens = a->total_new_tokens;
    w->layer_idx = a->layer_idx;
    w->num_layer = a->num_layer;
    w->num_kv_heads = a->num_kv_heads;
    w->head_dim = a->head_dim;
    w->cache_stride_s = a->cache_stride_s;
    w->cache_stride_l = a->cache_stride_l;
    w->cache_stride_h = a->cache_stride_h;
    w->cache_stride_kv = a->cache_stride_kv;
    w->d_cache = a->d_cache;
    w->d_scale = a->d_scale;
    w->cache_mode = a->cache_mode;
    w->page_size = a->page_size;
    w->cachestart_stride_b = a->cachestart_stride_b;
}

// cache_mode 0 (one contiguous slab region per sequence) or 1 (paged; multi_head_cache_attention_kernel.cc:161-168
// requires the 2-D page table, whose second extent arrives here as cachestart_stride_b)
static pplhip_retcode validate_cache_mode(int cache_mode, int page_size, int64_t cachestart_stride_b) {
    if (cache_mode != 0 && cache_mode != 1) PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "unknown cache_mode %d", cache_mode);
    if (cache_mode == 1) {
        if (cachestart_stride_b <= 0)
            PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "cachestarts must be a 2d tensor in cache_mode 1");
        if (page_size < 64 || (page_size & (page_size - 1)))
            PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "page_size %d: must be a power of two, at least 64", page_size);
    }
    return PPLHIP_RC_SUCCESS;
}

static pplhip_retcode validate_write(const pplhip_kv_write_args* a) {
    if (!a) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block");
    if (a->batch < 0 || a->total_new_tokens < 0) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "negative batch or token count");
    pplhip_retcode rc = validate_common(a->num_kv_heads, a->head_dim, a->num_layer, a->layer_idx, a->cache_stride_s,
                                        a->cache_stride_l, a->cache_stride_h, a->cache_stride_kv, a->d_cache, a->d_scale);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    rc = validate_cache_mode(a->cache_mode, a->page_size, a->cachestart_stride_b);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    if (a->batch > 0 && a->total_new_tokens > 0) {
        if (!a->d_current_key || !a->d_current_value || !a->d_seqstarts || !a->d_cachestarts || !a->d_start_pos)
            PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null tensor pointer");
        if (((uintptr_t)a->d_current_key & 15) || ((uintptr_t)a->d_current_value & 15))
            PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "current_key/current_value must be 16-byte aligned");
    }
    return PPLHIP_RC_SUCCESS;
}

} // namespace pplhip

using namespace pplhip;

extern "C" {

const char* pplhip_last_error(void) {
    return g_last_error;
}

int32_t pplhip_version(void) {
    return 300; // 0.3.0
}

pplhip_retcode pplhip_init(void) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
        PPLHIP_FAIL(PPLHIP_RC_DEVICE_RUNTIME_ERROR, "init: no current HIP device");
    if (prop.multiProcessorCount > 0) g_cu_count.store(prop.multiProcessorCount, std::memory_order_relaxed);
    void* scratch = nullptr; // this device's copy of the no-allocation entry point's scratch array
    return noalloc_scratch_of_current_device(&scratch);
}

// The decode decomposition: the kernel cuts the decode sequences' cached tokens, laid end to end, into S equal ranges
// on the device; the host only picks S from the chip size. One workgroup (4 waves) per range and group of <= 4 kv heads
// (`kv_heads` of them as the kernel sees them), two resident workgroups per CU. Sets decode_num_ranges,
// decode_heads_per_block and workspace_bytes.
static pplhip_retcode plan_decode_ranges(const pplhip_mhca_args* a, int kv_heads, pplhip_mhca_plan* plan) {
    const int64_t nd = a->decoding_batches;
    const int hpb = decode_heads_per_block(kv_heads);
    const int64_t groups = kv_heads / hpb;
    const int64_t slots = (int64_t)device_cu_count() * decode_blocks_per_cu();
    // halves of a slot: every workgroup streams the same number of bytes, so one workgroup per slot (a single,
    // perfectly filled round) measures best; the knob moves it to half or twice that
    const int64_t half_slots = a->specify_decoding_attn_split_k == 0 ? 1 : a->specify_decoding_attn_split_k == 1 ? 2 : 4;
    // ranges x groups workgroups must not spill over the slots (a second, nearly empty round doubles the time:
    // 40 kv heads = 10 groups took 56 ranges = 560 workgroups on 512 slots), so the quotient rounds DOWN
    int64_t ranges = slots * half_slots / 2 / groups;
    // never more ranges than 128-token pieces of the worst case (every sequence max_kvlen long)
    const int64_t cap = (nd * a->max_kvlen + 127) / 128;
    if (ranges > cap) ranges = cap;
    if (ranges < 8) ranges = 8;
    if (ranges > 0x3fffffff) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "decode: too many ranges");
    plan->decode_num_ranges = (int32_t)ranges;
    plan->decode_heads_per_block = hpb;
    plan->workspace_bytes = decode_workspace_bytes(a, ranges);
    return PPLHIP_RC_SUCCESS;
}

pplhip_retcode pplhip_mhca_prepare(const pplhip_mhca_args* a, pplhip_mhca_plan* plan) {
    if (!a || !plan) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block");
    memset(plan, 0, sizeof(*plan));
    if (a->d_alibi_slopes) PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "currently only support is_alibi == false");
    {
        pplhip_retcode rcm = validate_cache_mode(a->cache_mode, a->page_size, a->cachestart_stride_b);
        if (rcm != PPLHIP_RC_SUCCESS) return rcm;
        rcm = validate_mask(a->d_attn_mask, a->attn_mask_stride_h, a->attn_mask_stride_q);
        if (rcm != PPLHIP_RC_SUCCESS) return rcm;
    }
    if (a->num_heads <= 0 || a->num_kv_heads <= 0 || a->num_heads % a->num_kv_heads)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "num_heads %d is not a multiple of num_kv_heads %d", a->num_heads,
                    a->num_kv_heads);
    pplhip_retcode rc = validate_common(a->num_kv_heads, a->head_dim, a->num_layer, a->layer_idx, a->cache_stride_s,
                                        a->cache_stride_l, a->cache_stride_h, a->cache_stride_kv, a->d_cache, a->d_scale);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    if (a->batch < 0 || a->decoding_batches < 0 || a->decoding_batches > a->batch || a->total_new_tokens < a->batch ||
        a->max_seqlen < 0 || a->max_kvlen < a->max_seqlen)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE,
                    "inconsistent batch sizes: batch %lld decoding_batches %lld tokens %lld max_seqlen %lld max_kvlen %lld",
                    (long long)a->batch, (long long)a->decoding_batches, (long long)a->total_new_tokens,
                    (long long)a->max_seqlen, (long long)a->max_kvlen);
    if (a->batch > 0) {
        if (!a->d_query || !a->d_current_key || !a->d_current_value || !a->d_seqstarts || !a->d_kvstarts ||
            !a->d_cachestarts || !a->d_start_pos || !a->d_output)
            PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null tensor pointer");
        if (((uintptr_t)a->d_query & 15) || ((uintptr_t)a->d_current_key & 15) || ((uintptr_t)a->d_current_value & 15) ||
            ((uintptr_t)a->d_output & 15))
            PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "query/current_key/current_value/output must be 16-byte aligned");
    }
    if (a->specify_decoding_attn_split_k < 0 || a->specify_decoding_attn_split_k > 2)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "specify_decoding_attn_split_k must be 0, 1 or 2");
    if (a->specify_decoding_attn_tpb != 0 && a->specify_decoding_attn_tpb != 256 && a->specify_decoding_attn_tpb != 512)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "specify_decoding_attn_tpb must be 0, 256 or 512");

    if (needs_general_kernel(a->head_dim, a->num_heads, a->num_kv_heads, a->d_attn_mask)) {
        // write kernel + one launch of the general attention kernel (+ the merge of the decode sequences' pieces)
        plan->general_kernel = 1;
        const int vheads = a->decoding_batches > 0 ? decode_virtual_heads(a) : 0;
        if (vheads > 0) {
            // head_dim 64 / 32: the decode sequences run the head_dim-128 decode kernel over groups of 2 / 4 kv heads
            // (decode_num_ranges > 0 says so); the general kernel takes the prompts
            plan->decode_waves_per_block = decode_waves_per_block();
            const pplhip_retcode rc = plan_decode_ranges(a, vheads, plan);
            if (rc != PPLHIP_RC_SUCCESS) return rc;
            plan->general_decode_splits = 1;
            plan->workspace_bytes = (plan->workspace_bytes + 255) / 256 * 256;
            return PPLHIP_RC_SUCCESS;
        }
        plan->general_decode_splits = generic_decode_splits(a, device_cu_count());
        plan->workspace_bytes = (generic_workspace_bytes(a, plan->general_decode_splits) + 255) / 256 * 256;
        return PPLHIP_RC_SUCCESS;
    }

    // ---- decode: the kernel cuts the decode sequences' cached tokens, laid end to end, into S equal ranges on the
    // device; the host only picks S from the chip size. One workgroup (4 waves) per range and group of <= 4 kv heads,
    // two resident workgroups per CU.
    plan->decode_waves_per_block = decode_waves_per_block();
    if (a->decoding_batches > 0) {
        const pplhip_retcode rc = plan_decode_ranges(a, a->num_kv_heads, plan);
        if (rc != PPLHIP_RC_SUCCESS) return rc;
    }
    // ---- prefill
    plan->prefill_q_tile = 128;
    if (a->batch > a->decoding_batches)
        plan->prefill_num_q_tiles = (int32_t)((a->max_seqlen + plan->prefill_q_tile - 1) / plan->prefill_q_tile);
    plan->workspace_bytes = (plan->workspace_bytes + 255) / 256 * 256;
    if (const int64_t staged = prefill_staging_tokens(a)) {
        plan->prefill_staging = 1;
        plan->prefill_staging_offset_256 = (int32_t)(plan->workspace_bytes / 256);
        plan->workspace_bytes += (uint64_t)staged * 2 * a->num_kv_heads * a->head_dim * sizeof(uint16_t);
        plan->workspace_bytes = (plan->workspace_bytes + 255) / 256 * 256;
    }
    return PPLHIP_RC_SUCCESS;
}

pplhip_retcode pplhip_mhca_forward(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* d_workspace,
                                   void* stream) {
    if (!a || !plan) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block");
    if (a->batch == 0) return PPLHIP_RC_SUCCESS;
    if (plan->workspace_bytes > 0 && (!d_workspace || ((uintptr_t)d_workspace & 255)))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "workspace of %llu bytes (256-byte aligned) required",
                    (unsigned long long)plan->workspace_bytes);
    const bool general = needs_general_kernel(a->head_dim, a->num_heads, a->num_kv_heads, a->d_attn_mask);
    // (head_dim 64 / 32: the decode sequences may run the head_dim-128 decode kernel over groups of kv heads)
    const bool grouped_decode = general && a->decoding_batches > 0 && plan->decode_num_ranges > 0;
    if ((plan->general_kernel != 0) != general || (!general && a->decoding_batches > 0 && plan->decode_num_ranges <= 0) ||
        (grouped_decode && decode_virtual_heads(a) <= 0))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "plan was not produced by pplhip_mhca_prepare for these arguments");
    // the plan is checked against the arguments before anything is enqueued: a rejected call leaves the slab untouched,
    // and the kernels never write past the workspace the plan declares
    if (grouped_decode) {
        if (decode_workspace_bytes(a, plan->decode_num_ranges) > plan->workspace_bytes)
            PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "plan was not produced by pplhip_mhca_prepare for these arguments");
    } else if (general) {
        if (plan->general_decode_splits < 0 || plan->general_decode_splits > 64 ||
            generic_workspace_bytes(a, plan->general_decode_splits) > plan->workspace_bytes)
            PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "plan was not produced by pplhip_mhca_prepare for these arguments");
    } else {
        const uint64_t decode_bytes = decode_workspace_bytes(a, plan->decode_num_ranges);
        bool ok = plan->decode_num_ranges >= 0 && decode_bytes <= plan->workspace_bytes;
        if (ok && plan->prefill_staging) { // fp16 staging rows of a cache-prefill call, behind the decode partials
            const uint64_t first = (uint64_t)(uint32_t)plan->prefill_staging_offset_256 * 256;
            const uint64_t rows = (uint64_t)prefill_staging_tokens(a) * 2 * a->num_kv_heads * a->head_dim * sizeof(uint16_t);
            ok = plan->prefill_staging_offset_256 >= 0 && first >= decode_bytes && first + rows <= plan->workspace_bytes;
        }
        if (!ok) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "plan was not produced by pplhip_mhca_prepare for these arguments");
    }
    hipStream_t s = (hipStream_t)stream;
    pplhip_kv_write_args w;
    write_args_from_mhca(a, &w);
    if (general) {
        // every new token goes into the slab first; decode sequences (and, in a cache-prefill call, the prompts) then
        // attend over the slab
        pplhip_retcode rcw = launch_kv_quantize_write(&w, s);
        if (rcw != PPLHIP_RC_SUCCESS) return rcw;
        if (grouped_decode) {
            // the decode sequences through the decode kernel (their new tokens are in the slab already), the prompts
            // through the general kernel
            rcw = launch_decode(a, plan, d_workspace, s, true);
            if (rcw != PPLHIP_RC_SUCCESS) return rcw;
            return a->batch > a->decoding_batches ? launch_generic_mhca(a, 1, nullptr, s, true) : PPLHIP_RC_SUCCESS;
        }
        return launch_generic_mhca(a, plan->general_decode_splits, d_workspace, s);
    }
    // the decode kernel quantises the decode sequences' new tokens (the first decoding_batches packed tokens) into the
    // slab itself, and the prompt tokens are left to the prefill launch unless it reads them back from the slab
    // (cache-prefill): on the default path this launches nothing
    pplhip_retcode rc = launch_kv_quantize_write(&w, s, a->decoding_batches,
                                                 prefill_writes_new_tokens(a) ? a->decoding_batches : -1);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    return launch_decode_and_prefill(a, plan, d_workspace, s);
}

pplhip_retcode pplhip_mhca_forward_noalloc(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* stream) {
    if (!a || !plan) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block");
    if (plan->workspace_bytes > kNoAllocScratchBytes)
        PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE,
                    "this call needs %llu bytes of scratch, the built-in array holds %llu: use pplhip_mhca_forward with "
                    "a caller-owned workspace", (unsigned long long)plan->workspace_bytes,
                    (unsigned long long)kNoAllocScratchBytes);
    if (plan->prefill_staging)
        PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "cache-prefill with fp16 staging rows needs a caller-owned workspace (clear "
                                           "plan.prefill_staging, or use pplhip_mhca_forward)");
    void* scratch = nullptr;
    const pplhip_retcode rc = noalloc_scratch_of_current_device(&scratch);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    // nothing in the scratch has to start at zero: every partial result and table entry a call reads was written by
    // that call's own decode workgroups
    return pplhip_mhca_forward(a, plan, scratch, stream);
}

pplhip_retcode pplhip_mha_forward(const pplhip_mha_args* a, void* stream) {
    if (!a) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block");
    if (a->is_alibi) PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "currently only support is_alibi == false");
    if (!generic_head_dim_supported(a->head_dim))
        PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "head_dim %d: must be a multiple of 16 between 16 and 256", a->head_dim);
    {
        const pplhip_retcode rcm = validate_mask(a->d_attn_mask, a->attn_mask_stride_h, a->attn_mask_stride_q);
        if (rcm != PPLHIP_RC_SUCCESS) return rcm;
    }
    if (a->num_heads <= 0 || a->num_kv_heads <= 0 || a->num_heads % a->num_kv_heads != 0)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "num_heads %d must be a positive multiple of num_kv_heads %d",
                    a->num_heads, a->num_kv_heads);
    if (a->batch < 0 || a->max_seqlen < 0 || a->max_kvlen < a->max_seqlen)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "inconsistent batch %lld / max_seqlen %lld / max_kvlen %lld",
                    (long long)a->batch, (long long)a->max_seqlen, (long long)a->max_kvlen);
    if (a->batch == 0) return PPLHIP_RC_SUCCESS;
    if (!a->d_query || !a->d_key || !a->d_value || !a->d_seqstarts || !a->d_kvstarts || !a->d_output)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null tensor pointer");
    if (((uintptr_t)a->d_query & 15) || ((uintptr_t)a->d_key & 15) || ((uintptr_t)a->d_value & 15) ||
        ((uintptr_t)a->d_output & 15))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "query/key/value/output must be 16-byte aligned");
    if (needs_general_kernel(a->head_dim, a->num_heads, a->num_kv_heads, a->d_attn_mask))
        return launch_generic_mha(a, (hipStream_t)stream);
    return launch_mha(a, (hipStream_t)stream);
}

// *empty: nothing to do (no sequences or no tokens)
static pplhip_retcode validate_rope(const pplhip_rope_args* a, bool* empty) {
    *empty = false;
    if (!a) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block");
    if (a->scaling_type != PPLHIP_ROPE_SCALING_NONE && a->scaling_type != PPLHIP_ROPE_SCALING_LINEAR &&
        a->scaling_type != PPLHIP_ROPE_SCALING_DYNAMIC)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "invalid scaling type: %d", a->scaling_type);
    const int rotary_dim = a->rotary_dim == 0 ? a->head_dim : a->rotary_dim;
    if (a->pair_layout != PPLHIP_ROPE_PAIRS_INTERLEAVED && a->pair_layout != PPLHIP_ROPE_PAIRS_HALF_SPLIT)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "invalid pair layout: %d", a->pair_layout);
    if (a->head_dim <= 0 || a->head_dim % 8 || a->head_dim > 2048)
        PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "head_dim %d: must be a multiple of 8, at most 2048", a->head_dim);
    if (rotary_dim < 0 || rotary_dim % 8 || rotary_dim > a->head_dim)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "rotary_dim %d: must be a multiple of 8 within head_dim %d", rotary_dim,
                    a->head_dim);
    if (a->pair_layout == PPLHIP_ROPE_PAIRS_HALF_SPLIT && rotary_dim % 16)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "rotary_dim %d: must be a multiple of 16 for the half-split pair layout",
                    rotary_dim);
    if (a->num_heads <= 0 || a->num_key_heads <= 0)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "num_heads %d / num_key_heads %d", a->num_heads, a->num_key_heads);
    if (!(a->theta > 0.f)) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "theta must be positive");
    if (a->scaling_type != PPLHIP_ROPE_SCALING_NONE && !(a->scaling_factor > 0.f))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "scaling_factor must be positive");
    if (a->scaling_type == PPLHIP_ROPE_SCALING_DYNAMIC && (a->max_position_embeddings <= 0 || rotary_dim <= 2))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "dynamic scaling needs max_position_embeddings > 0 and rotary_dim > 2");
    if (a->batch < 0 || a->total_tokens < 0) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "negative batch or token count");
    if (a->batch == 0 || a->total_tokens == 0) {
        *empty = true;
        return PPLHIP_RC_SUCCESS;
    }
    if (!a->d_query || !a->d_key || !a->d_seqstarts || !a->d_start_pos || !a->d_rotated_query || !a->d_rotated_key)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null tensor pointer");
    if (((uintptr_t)a->d_query & 15) || ((uintptr_t)a->d_key & 15) || ((uintptr_t)a->d_rotated_query & 15) ||
        ((uintptr_t)a->d_rotated_key & 15))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "query/key tensors must be 16-byte aligned");
    return PPLHIP_RC_SUCCESS;
}

pplhip_retcode pplhip_rope_forward(const pplhip_rope_args* a, void* stream) {
    bool empty;
    const pplhip_retcode rc = validate_rope(a, &empty);
    if (rc != PPLHIP_RC_SUCCESS || empty) return rc;
    return launch_rope(a, nullptr, (hipStream_t)stream);
}

pplhip_retcode pplhip_rope_kv_write_forward(const pplhip_rope_args* a, const pplhip_kv_write_args* w, void* stream) {
    bool empty;
    pplhip_retcode rc = validate_rope(a, &empty);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    if (!w) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block");
    {
        pplhip_kv_write_args checked = *w; // (the keys that are quantised are the rotated ones: current_key is not read)
        checked.d_current_key = a->d_rotated_key;
        rc = validate_write(&checked);
        if (rc != PPLHIP_RC_SUCCESS) return rc;
    }
    // one pass over the new tokens serves both operators: they must describe the same tokens
    if (w->batch != a->batch || w->total_new_tokens != a->total_tokens || w->num_kv_heads != a->num_key_heads ||
        w->head_dim != a->head_dim)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE,
                    "rotary embedding + cache write: batch %lld/%lld, tokens %lld/%lld, key heads %d/%d, head_dim %d/%d differ",
                    (long long)a->batch, (long long)w->batch, (long long)a->total_tokens, (long long)w->total_new_tokens,
                    a->num_key_heads, w->num_kv_heads, a->head_dim, w->head_dim);
    if (empty) return PPLHIP_RC_SUCCESS;
    if (w->d_seqstarts != a->d_seqstarts || w->d_start_pos != a->d_start_pos)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "rotary embedding + cache write: both must use the same seqstarts / start_pos");
    if (a->head_dim > 256) PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "rotary embedding + cache write: head_dim at most 256");
    return launch_rope(a, w, (hipStream_t)stream);
}

pplhip_retcode pplhip_position_index(const int64_t* d_start_pos, const int64_t* d_seqstarts, int64_t batch,
                                     int64_t total_tokens, int64_t max_seqlen, int64_t* d_position_idx, void* stream) {
    (void)max_seqlen;
    if (batch < 0 || total_tokens < 0) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "negative batch or token count");
    if (batch == 0 || total_tokens == 0) return PPLHIP_RC_SUCCESS;
    if (!d_start_pos || !d_seqstarts || !d_position_idx) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null tensor pointer");
    return launch_position_index(d_seqstarts, d_start_pos, batch, total_tokens, d_position_idx, (hipStream_t)stream);
}

pplhip_retcode pplhip_kv_quantize_write(const pplhip_kv_write_args* a, void* stream) {
    pplhip_retcode rc = validate_write(a);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    return launch_kv_quantize_write(a, (hipStream_t)stream);
}

pplhip_retcode pplhip_kv_cache_forward(const pplhip_kv_cache_args* a, void* stream) {
    if (!a) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block");
    if (a->cache_layout != 0) PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "currently only support cache_layout == 0");
    if (a->cache_mode != 0) PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "currently only support cache_mode == 0");
    if (a->num_repeat != 1) PPLHIP_FAIL(PPLHIP_RC_UNSUPPORTED, "currently only support num_repeat == 1");
    pplhip_retcode rc = validate_write(&a->write);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    if (a->total_kv_tokens < 0) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "negative total_kv_tokens");
    if (a->total_kv_tokens > 0 && (!a->d_kvstarts || !a->d_key_out || !a->d_value_out))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null tensor pointer");
    if (((uintptr_t)a->d_key_out & 15) || ((uintptr_t)a->d_value_out & 15))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "key/value outputs must be 16-byte aligned");
    rc = launch_kv_quantize_write(&a->write, (hipStream_t)stream);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    return launch_kv_gather_dequant(a, (hipStream_t)stream);
}

pplhip_retcode pplhip_pack_tables(const pplhip_pack_args* a, void* stream) {
    if (!a) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block");
    if (!a->d_slot_kvlen || !a->d_slot_newlen || !a->d_slot_cachestart || !a->d_seqstarts || !a->d_kvstarts ||
        !a->d_cachestarts || !a->d_start_pos || !a->d_batch_slots || !a->d_header)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null table pointer");
    return launch_pack_tables(a, (hipStream_t)stream);
}

static pplhip_retcode validate_check_tables(const pplhip_mhca_args* a, int64_t max_slab_tokens, const int32_t* flag) {
    if (!a || !flag) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null argument block or flag pointer");
    if (a->batch < 0 || a->decoding_batches < 0 || a->decoding_batches > a->batch || max_slab_tokens < 0)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "check_tables: batch %lld, decoding_batches %lld, max_slab_tokens %lld",
                    (long long)a->batch, (long long)a->decoding_batches, (long long)max_slab_tokens);
    if (a->batch >= (int64_t(1) << 31)) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "check_tables: too many sequences");
    if (a->batch > 0 && (!a->d_seqstarts || !a->d_kvstarts || !a->d_cachestarts || !a->d_start_pos))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "null table pointer");
    return validate_cache_mode(a->cache_mode, a->page_size, a->cachestart_stride_b);
}

pplhip_retcode pplhip_check_tables(const pplhip_mhca_args* a, int64_t max_slab_tokens, int32_t* d_flag, void* stream) {
    const pplhip_retcode rc = validate_check_tables(a, max_slab_tokens, d_flag);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    return launch_check_tables(a, max_slab_tokens, d_flag, (hipStream_t)stream);
}

pplhip_retcode pplhip_check_tables_host(const pplhip_mhca_args* a, int64_t max_slab_tokens, int32_t* flag) {
    const pplhip_retcode rc = validate_check_tables(a, max_slab_tokens, flag);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    check_tables_host(a, max_slab_tokens, flag);
    return PPLHIP_RC_SUCCESS;
}

pplhip_retcode pplhip_advance_slots(int64_t* d_slot_kvlen, const int64_t* d_slot_newlen, int32_t num_slots,
                                    void* stream) {
    if (num_slots < 0 || (num_slots > 0 && (!d_slot_kvlen || !d_slot_newlen)))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "bad slot arrays");
    return launch_advance_slots(d_slot_kvlen, d_slot_newlen, num_slots, (hipStream_t)stream);
}

} // extern "C"
