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

// The register-level pattern of the one-wavefront-per-SIMD kernels: a wavefront alone on its SIMD holds a grid of
// accumulator tiles (all 256 AGPRs) and multiplies every A fragment with every B fragment, so each operand register
// feeds 8 (16x16x32: 8 x 8 tiles) or 4 (32x32x16: 4 x 4 tiles) matrix instructions and each accumulator is touched
// once per pass - the operand-reuse and accumulator-traffic pattern of gemm_w128 / flash_attention_fwd_w64, without
// their LDS reads, loads and vector-ALU work. One pass = 64 or 16 instructions = 2^20 / 2^19 FLOP per wavefront.
template <bool k16x16x32>
__global__ void __launch_bounds__(256)
    mfma_reuse_kernel(const _Float16* __restrict__ operands, unsigned long long* __restrict__ clocks, float* sink, int iters) {
    constexpr int kT = k16x16x32 ? 8 : 4;
    const f16x8* p = reinterpret_cast<const f16x8*>(operands) + (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * 16;
    f16x8 a[kT], b[kT];
#pragma unroll
    for (int i = 0; i < kT; ++i) {
        a[i] = p[i];
        b[i] = p[8 + i];
    }
    float s = 0.f;
    const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    if constexpr (k16x16x32) {
        f32x4 c[kT][kT];
#pragma unroll
        for (int i = 0; i < kT; ++i)
#pragma unroll
            for (int j = 0; j < kT; ++j) c[i][j] = f32x4{0, 0, 0, 0};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < kT; ++i)
#pragma unroll
                for (int j = 0; j < kT; ++j) c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], b[j], c[i][j], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < kT; ++i)
#pragma unroll
            for (int j = 0; j < kT; ++j) s += c[i][j][0] + c[i][j][3];
    } else {
        f32x16 c[kT][kT];
#pragma unroll
        for (int i = 0; i < kT; ++i)
#pragma unroll
            for (int j = 0; j < kT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) c[i][j][e] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < kT; ++i)
#pragma unroll
                for (int j = 0; j < kT; ++j) c[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], c[i][j], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < kT; ++i)
#pragma unroll
            for (int j = 0; j < kT; ++j) s += c[i][j][0] + c[i][j][15];
    }
    const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    if (threadIdx.x == 0) {
        clocks[2 * blockIdx.x] = t1 - t0;
        clocks[2 * blockIdx.x + 1] = r1 - r0;
    }
    if (s == 12345.678f) *sink = s;
}

}  // namespace

// The one-wavefront-per-SIMD pattern (see mfma_reuse_kernel): 4 wavefronts per workgroup, one workgroup per CU.
// operands: at least workgroups * 256 lanes * 128 halves of fp16; shape 0 = 32x32x16 (16 instructions per pass),
// 1 = 16x16x32 (64 per pass). FLOPs of the launch: workgroups * 4 * iters * (2^19 for shape 0, 2^20 for shape 1).
extern "C" int tcu_probe_mfma_f16_reuse(const void* operands, void* clocks, void* sink, int shape, int workgroups, int iters,
                                        void* stream) {
    if (workgroups <= 0 || iters <= 0) return int(hipErrorInvalidValue);
    const dim3 grid(workgroups), block(256);
    auto* ops = static_cast<const _Float16*>(operands);
    auto* clk = static_cast<unsigned long long*>(clocks);
    auto* snk = static_cast<float*>(sink);
    if (shape == 1)
        hipLaunchKernelGGL(mfma_reuse_kernel<true>, grid, block, 0, static_cast<hipStream_t>(stream), ops, clk, snk, iters);
    else
        hipLaunchKernelGGL(mfma_reuse_kernel<false>, grid, block, 0, static_cast<hipStream_t>(stream), ops, clk, snk, iters);
    return int(hipGetLastError());
}

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
