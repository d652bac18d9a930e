// Measurement aid for the benchmark (not part of the kernel library): the MFMA rate and core clock that the GPU
// sustains on a loop of nothing but matrix instructions whose operands come from a caller-supplied buffer.
// On MI355X the matrix pipe is power-managed: with random fp16 operands the core clock drops well below the
// 2.4 GHz behind the published 2.5 PFLOP/s, so this rate, not the published peak, is what a GEMM can approach.
#include <hip/hip_runtime.h>

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Each lane loads 8 operand vectors (64 halves) once, then issues 4 independent MFMAs per iteration.
// clocks[2 b] / clocks[2 b + 1]: shader-clock and 100 MHz constant-clock ticks workgroup b spent in the loop.
template <bool k16x16x32>
__global__ void __launch_bounds__(512)
    mfma_rate_kernel(const _Float16* __restrict__ operands, unsigned long long* __restrict__ clocks, float* sink, int iters) {
    const f16x8* p = reinterpret_cast<const f16x8*>(operands) + (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
    const f16x8 a0 = p[0], a1 = p[1], a2 = p[2], a3 = p[3], b0 = p[4], b1 = p[5], b2 = p[6], b3 = p[7];
    float s = 0.f;
    const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    if constexpr (k16x16x32) {
        f32x4 c0 = {0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
        for (int it = 0; it < iters; ++it) {
            c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b0, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, b1, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, b2, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a3, b3, c3, 0, 0, 0);
        }
        for (int i = 0; i < 4; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
    } else {
        f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
        for (int it = 0; it < iters; ++it) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b0, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b1, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2, b2, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a3, b3, c3, 0, 0, 0);
        }
        for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
    }
    const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    if (threadIdx.x == 0) {
        clocks[2 * blockIdx.x] = t1 - t0;
        clocks[2 * blockIdx.x + 1] = r1 - r0;
    }
    if (s == 12345.678f) *sink = s;  // keeps the accumulators alive
}

}  // namespace

// operands: at least workgroups * waves_per_workgroup * 64 lanes * 64 halves of fp16; clocks: 2 * workgroups u64;
// sink: one float. shape 0 = 32x32x16, 1 = 16x16x32. Launches one kernel on `stream`; returns the hipError_t value.
// FLOPs of the launch: workgroups * waves_per_workgroup * iters * 4 * (32768 for shape 0, 16384 for shape 1).
extern "C" int tcu_probe_mfma_f16(const void* operands, void* clocks, void* sink, int shape, int workgroups,
                                  int waves_per_workgroup, int iters, void* stream) {
    if (workgroups <= 0 || waves_per_workgroup <= 0 || waves_per_workgroup > 8 || iters <= 0) return int(hipErrorInvalidValue);
    const dim3 grid(workgroups), block(waves_per_workgroup * 64);
    auto* ops = static_cast<const _Float16*>(operands);
    auto* clk = static_cast<unsigned long long*>(clocks);
    auto* snk = static_cast<float*>(sink);
    if (shape == 1)
        hipLaunchKernelGGL(mfma_rate_kernel<true>, grid, block, 0, static_cast<hipStream_t>(stream), ops, clk, snk, iters);
    else
        hipLaunchKernelGGL(mfma_rate_kernel<false>, grid, block, 0, static_cast<hipStream_t>(stream), ops, clk, snk, iters);
    return int(hipGetLastError());
}
