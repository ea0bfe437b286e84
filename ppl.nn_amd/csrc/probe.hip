// Calibration probes for the two rooflines.
// fp16 matrix cores: a bare loop of independent v_mfma_f32_32x32x16_f16 over operands
// the caller supplies. The rate this chip SUSTAINS depends on the operand data (power management lowers the clock when
// the operands toggle many bits): the benchmark reports the prefill kernel next to the published peak and next to
// this measured figure for random fp16 operands.
// Built into a library of its own (the probes are not part of the drop-in ABI); quantize_group8 is the kernel library's
// own inline quantiser, compiled here with the same flags.
#include <stdarg.h>

#include "common.h"
#include "../../include/ppl_llm_kernel_hip_probes.h"

namespace pplhip {

static thread_local char g_probe_error[256] = "";
void set_error(const char* fmt, ...) { // (this library's copy: PPLHIP_FAIL writes here)
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_probe_error, sizeof(g_probe_error), fmt, ap);
    va_end(ap);
}

constexpr int kProbeMfmaPerIter = 16;

__global__ __launch_bounds__(256) void probe_mfma_f16_kernel(const half8_t* __restrict__ in, float* __restrict__ out,
                                                             int iters) {
    half8_t a[4], b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        a[j] = in[threadIdx.x + 256 * j];
        b[j] = in[threadIdx.x + 256 * (4 + j)];
    }
    float16_t c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) c[j][i] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < kProbeMfmaPerIter; ++s) {
            c[s & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[s & 3], b[s >> 2], c[s & 3], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) s += c[j][i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// HBM: every workgroup streams its own contiguous share of a buffer with 16-byte loads, eight in flight per lane, and
// folds what it read into one word per lane (so that no load can be dropped). The benchmark runs it over a buffer far
// larger than the 256 MB memory-side cache and reports the decode kernel next to the published 8 TB/s and next to
// this measured streaming rate.
constexpr int kProbeLoadsInFlight = 8;

typedef uint32_t u32x4_probe_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void probe_hbm_read_kernel(const u32x4_probe_t* __restrict__ src, uint64_t chunk16,
                                                             uint32_t* __restrict__ out) {
    const u32x4_probe_t* p = src + (uint64_t)blockIdx.x * chunk16;
    uint32_t acc = 0;
    for (uint64_t i = threadIdx.x; i + (kProbeLoadsInFlight - 1) * 256 < chunk16; i += kProbeLoadsInFlight * 256) {
        u32x4_probe_t v[kProbeLoadsInFlight];
#pragma unroll
        for (int j = 0; j < kProbeLoadsInFlight; ++j) v[j] = __builtin_nontemporal_load(p + i + j * 256);
#pragma unroll
        for (int j = 0; j < kProbeLoadsInFlight; ++j) acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = acc;
}

} // namespace pplhip

using namespace pplhip;

extern "C" const char* pplhip_probe_last_error(void) {
    return g_probe_error;
}

// The slab addressing every kernel uses (CacheAddr::row, compiled here for the host): element offset of a row of the
// int8 slab and of its first scale. Host only, no device call.
extern "C" pplhip_retcode pplhip_probe_slab_row(int64_t stride_s, int64_t stride_l, int64_t stride_h, int64_t stride_kv,
                                                int32_t layer, int64_t token, int32_t kv, int32_t head,
                                                int64_t* cache_element, int64_t* scale_element) {
    if (!cache_element || !scale_element) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "probe: null result pointer");
    const CacheAddr addr{stride_s, stride_l, stride_h, stride_kv, layer};
    *cache_element = addr.row(token, kv, head);
    *scale_element = *cache_element / kQuantGroup;
    return PPLHIP_RC_SUCCESS;
}

extern "C" pplhip_retcode pplhip_probe_hbm_read(const void* d_src, uint64_t bytes, void* d_out, int32_t workgroups,
                                                uint64_t* bytes_read, void* stream) {
    if (!d_src || !d_out || workgroups <= 0) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "probe: null buffer or no workgroups");
    if (((uintptr_t)d_src & 15)) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "probe: source must be 16-byte aligned");
    // whole rounds of 256 lanes x 8 loads x 16 bytes per workgroup
    const uint64_t round16 = 256ull * kProbeLoadsInFlight;
    const uint64_t chunk16 = bytes / 16 / (uint64_t)workgroups / round16 * round16;
    if (chunk16 == 0) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "probe: buffer too small for %d workgroups", workgroups);
    hipLaunchKernelGGL(probe_hbm_read_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4_probe_t*)d_src, chunk16, (uint32_t*)d_out);
    PPLHIP_CHECK_LAUNCH("probe_hbm_read");
    if (bytes_read) *bytes_read = chunk16 * 16 * (uint64_t)workgroups;
    return PPLHIP_RC_SUCCESS;
}

extern "C" pplhip_retcode pplhip_probe_mfma_f16(const void* d_operands, void* d_out, int32_t workgroups,
                                                int32_t iterations, double* flops, void* stream) {
    if (!d_operands || !d_out || workgroups <= 0 || iterations <= 0)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "probe: null buffer or non-positive size");
    if (((uintptr_t)d_operands & 15)) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "probe: operands must be 16-byte aligned");
    hipLaunchKernelGGL(probe_mfma_f16_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream,
                       (const half8_t*)d_operands, (float*)d_out, iterations);
    PPLHIP_CHECK_LAUNCH("probe_mfma_f16");
    // 4 waves per workgroup, 32 x 32 x 16 multiply-adds per wave-level instruction
    if (flops) *flops = (double)workgroups * 4.0 * iterations * kProbeMfmaPerIter * (2.0 * 32 * 32 * 16);
    return PPLHIP_RC_SUCCESS;
}

// ---- the quantiser's quotients, enumerated
// quantize_group8 forms x / s as x * (1 / s). For every absmax A (all positive fp16 up to +inf: every scale the rule
// can produce) and every fp16 x of no larger magnitude (and every NaN, which the maximum ignores), the group
// {A, x, 0, ...} goes through quantize_group8 and the int8 it gives x is compared with int8(rint(fp16(x / s))) formed
// by a correctly rounded fp32 division.
__global__ __launch_bounds__(256) void probe_quantizer_kernel(unsigned long long* mismatches) {
    const uint32_t a_bits = blockIdx.x + 1; // 0x0001 .. 0x7c00
    unsigned long long bad = 0;
    for (uint32_t xb = threadIdx.x; xb < 65536; xb += 256) {
        const uint32_t mag = xb & 0x7fffu;
        if (mag > a_bits && mag <= 0x7c00u) continue; // larger magnitude than the absmax
        uint2 q;
        half_t s;
        quantize_group8(make_uint4(a_bits | xb << 16, 0, 0, 0), &q, &s);
        const uint16_t x16 = (uint16_t)xb;
        half_t x;
        __builtin_memcpy(&x, &x16, 2);
        float r = rintf((float)(half_t)((float)x / (float)s));
        r = fminf(fmaxf(r, -128.f), 127.f);
        if ((uint32_t)((int)r & 0xff) != ((q.x >> 8) & 0xffu)) ++bad;
    }
    if (bad) atomicAdd(mismatches, bad);
}

extern "C" pplhip_retcode pplhip_probe_quantizer(uint64_t* d_mismatches, void* stream) {
    if (!d_mismatches) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "probe: null counter");
    hipLaunchKernelGGL(probe_quantizer_kernel, dim3(0x7c00), dim3(256), 0, (hipStream_t)stream,
                       (unsigned long long*)d_mismatches);
    PPLHIP_CHECK_LAUNCH("probe_quantizer");
    return PPLHIP_RC_SUCCESS;
}

