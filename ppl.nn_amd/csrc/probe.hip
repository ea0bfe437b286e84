// Calibration probe for the fp16 matrix-core roofline: a bare loop of independent v_mfma_f32_32x32x16_f16 over operands
// the caller supplies. The rate this chip SUSTAINS depends on the operand data (power management lowers the clock when
// the operands toggle many bits): the benchmark reports the prefill kernel next to the published peak and next to
// this measured figure for random fp16 operands.
#include "common.h"

namespace pplhip {

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

} // namespace pplhip

using namespace pplhip;

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
