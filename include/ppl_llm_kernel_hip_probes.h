/*
 * Measurement and verification aids of the gfx950 kernel library, built into a library of their own
 * (libppl_llm_kernel_hip_probes.so). They are NOT part of the drop-in ABI of ppl_llm_kernel_hip.h and have no
 * counterpart in the reference: a benchmark uses the two roofline probes to report the rates this chip sustains beside
 * the published peaks, and a test uses the quantiser enumeration to pin the library's rounding rule on the GPU it runs
 * on. Return codes are those of ppl_llm_kernel_hip.h.
 */
#ifndef PPL_LLM_KERNEL_HIP_PROBES_H_
#define PPL_LLM_KERNEL_HIP_PROBES_H_

#include "ppl_llm_kernel_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Human-readable text of the last error a probe raised on the calling thread ("" if none). Never NULL. */
const char* pplhip_probe_last_error(void);

/*
 * Measurement aid (no counterpart in the reference): enqueues `workgroups` x 4 wavefronts that each issue
 * `iterations` x 16 independent v_mfma_f32_32x32x16_f16 on the operands at `d_operands` (2048 x 16 bytes of fp16,
 * device, 16-byte aligned) and write one float per lane to `d_out` (workgroups x 256 floats). `*flops` (host, may be
 * NULL) receives the floating-point operations of the launch. Timing it gives the matrix-core rate this chip sustains
 * for THAT operand data: with random operands the clock is held well below the one the published peak assumes.
 */
pplhip_retcode pplhip_probe_mfma_f16(const void* d_operands, void* d_out, int32_t workgroups, int32_t iterations,
                                     double* flops, void* stream);

/*
 * Measurement aid (no counterpart in the reference): `workgroups` workgroups each stream their own contiguous share
 * of the `bytes` at `d_src` (device, 16-byte aligned) with plain 16-byte loads, eight in flight per lane, and write one
 * word per lane to `d_out` (workgroups x 256 words). `*bytes_read` (host, may be NULL) receives what the launch read
 * (shares are rounded down to whole rounds of 32 KiB). Timed over a buffer much larger than the memory-side cache it
 * gives the streaming-read rate the chip sustains, the practical ceiling beside the published 8 TB/s.
 */
pplhip_retcode pplhip_probe_hbm_read(const void* d_src, uint64_t bytes, void* d_out, int32_t workgroups,
                                     uint64_t* bytes_read, void* stream);

/*
 * Verification aid (no counterpart in the reference): the quantiser forms x / s as x * (1 / s), one division per
 * group instead of eight. This call enumerates every absmax (all positive fp16 up to +inf, i.e. every scale the rule
 * max(fp16(absmax / 127), fp16(1e-5)) can produce) with every fp16 x of no larger magnitude or NaN, runs each pair through
 * the library's own quantiser and ADDS to `*d_mismatches` (device, 8 bytes, cleared by the caller) the number of pairs
 * whose int8 differs from int8(rint(fp16(x / s))) formed by a correctly rounded division. 0 is the contract.
 */
pplhip_retcode pplhip_probe_quantizer(uint64_t* d_mismatches, void* stream);

/*
 * Verification aid, host only (no device call): the element offset of row (token, kv, head) of layer `layer` in the
 * int8 slab and of the row's first scale in the scale tensor, formed by the library's own addressing (the struct every
 * kernel folds its slab offsets with). A test compares it with arbitrary-precision arithmetic over strides up to
 * 2^34, i.e. slabs far beyond 4 GiB: tok*stride_s + layer*stride_l + kv*stride_kv + head*stride_h, and that / 8.
 */
pplhip_retcode pplhip_probe_slab_row(int64_t stride_s, int64_t stride_l, int64_t stride_h, int64_t stride_kv, int32_t layer,
                                     int64_t token, int32_t kv, int32_t head, int64_t* cache_element,
                                     int64_t* scale_element);

#ifdef __cplusplus
}
#endif

#endif
