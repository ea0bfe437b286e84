// MultiHeadCacheAttention's kernels in one translation unit: the decode sequences' attention (decode.hip), the prompts'
// attention (prefill.hip), and -- for a call that has both -- ONE launch that carries the workgroups of both.
//
// Why one launch: kernels of one stream never overlap and every launch boundary costs a few microseconds of idle chip;
// two streams overlap the two parts, but the fork and the join are two dependencies between hardware queues that cost
// more than the overlap gains (Llama-3-8B mixed batch: 17 us). In one grid the decode workgroups come first and all run
// at once; the prompts' tile workgroups sit behind them and take the slots as they become free. Measured on that batch:
// 187 us per call instead of 199 (the launch itself takes about as long as the two kernels one after the other -- the
// tile workgroups that move in share their CUs' memory pipes with the decode workgroups still running -- what is saved is
// two launches and their gaps).
#include "decode.hip"
#include "prefill.hip"

namespace pplhip {

static_assert(kDecodeLdsBytes >= 4 * kDmaTile, "the prompt workgroups use the decode workgroups' LDS allocation");

template <bool PAGED, bool DIRECT>
__global__ __launch_bounds__(256, 2) void mixed_attention_kernel(const DecodeParams dp, const PrefillParams pp,
                                                                 uint32_t decode_blocks) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    if (blockIdx.x < decode_blocks)
        decode_workgroup<PAGED, DIRECT>(dp, blockIdx.x, smem);
    else
        prefill_workgroup(pp, blockIdx.x - decode_blocks, gridDim.x - decode_blocks, smem);
}

// Decode sequences and prompts of one call. The single launch serves the default path (prompts read from
// current_key / current_value, or from staged rows); prompts that are read from the int8 slab by their own kernel keep
// the two launches.
pplhip_retcode launch_decode_and_prefill(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* ws,
                                         hipStream_t stream) {
    const bool has_decode = a->decoding_batches > 0;
    const bool has_prefill = a->batch > a->decoding_batches && plan->prefill_num_q_tiles > 0;
    if (!has_decode || !has_prefill) {
        const pplhip_retcode rc = launch_decode(a, plan, ws, stream);
        return rc != PPLHIP_RC_SUCCESS ? rc : launch_prefill(a, plan, ws, stream);
    }
    DecodeParams dp;
    PrefillParams pp;
    int64_t dblocks, pblocks;
    bool from_slab;
    pplhip_retcode rc = decode_setup(a, plan, ws, &dp, &dblocks);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    if (a->enable_cache_prefill && !plan->prefill_staging) { // (decided before prefill_setup enqueues anything)
        rc = launch_decode(a, plan, ws, stream);
        return rc != PPLHIP_RC_SUCCESS ? rc : launch_prefill(a, plan, ws, stream);
    }
    // the prompts' write-only workgroups (dispatched last, into the launch's tail) take the decode sequences' new
    // tokens as well: stores from the middle of a decode wave's stream stall it
    rc = prefill_setup(a, plan, ws, stream, true, &pp, &pblocks, &from_slab);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    dp.new_tokens_written_elsewhere = pp.w_cache != nullptr && pp.w_first_token == 0;
    if (dblocks + pblocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "attention: too many workgroups in one call");
    static std::atomic<uint64_t> lds_opted_in{0};
    rc = reserve_decode_lds(lds_opted_in, {reinterpret_cast<const void*>(mixed_attention_kernel<false, false>),
                                           reinterpret_cast<const void*>(mixed_attention_kernel<true, false>),
                                           reinterpret_cast<const void*>(mixed_attention_kernel<false, true>),
                                           reinterpret_cast<const void*>(mixed_attention_kernel<true, true>)});
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    // the decode workgroups come first: they are dispatched at once. The prompts' numbering relies on workgroups that
    // are 8 apart sharing an XCD, which holds behind any number of decode workgroups.
    const dim3 grid((unsigned)(dblocks + pblocks)), block(256);
    const uint32_t nd_blocks = (uint32_t)dblocks;
    const bool direct = dp.hpb == kDecodeWaves;
    if (dp.page_shift && direct)
        hipLaunchKernelGGL((mixed_attention_kernel<true, true>), grid, block, kDecodeLdsBytes, stream, dp, pp, nd_blocks);
    else if (dp.page_shift)
        hipLaunchKernelGGL((mixed_attention_kernel<true, false>), grid, block, kDecodeLdsBytes, stream, dp, pp, nd_blocks);
    else if (direct)
        hipLaunchKernelGGL((mixed_attention_kernel<false, true>), grid, block, kDecodeLdsBytes, stream, dp, pp, nd_blocks);
    else
        hipLaunchKernelGGL((mixed_attention_kernel<false, false>), grid, block, kDecodeLdsBytes, stream, dp, pp, nd_blocks);
    PPLHIP_CHECK_LAUNCH("mixed_attention");
    return launch_decode_merge(dp, stream);
}

} // namespace pplhip
