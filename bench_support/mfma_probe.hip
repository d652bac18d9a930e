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

// What a wavefront alone on its SIMD pays for the instructions it places between two matrix instructions: a loop of
// 8 independent matrix instructions, each followed by the same filler. kFill: 0 nothing, 1..4 that many v_add_f32,
// 5 v_exp_f32, 6 v_exp_f32 + v_add_f32, 7 v_exp_f32 + 2 v_add_f32, 8 ds_read_b128, 9 v_add_u32 feeding the address of a
// ds_read_b128, 10 two ds_read_b64_tr_b16, 11 v_cvt_pk_f16_f32 + v_add_f32, 12 a ds_read_b128 behind every second matrix
// instruction only. clocks[b]: shader-clock ticks workgroup b spent in the loop (8 * iters matrix instructions).
template <int kFill, bool k32x32>
__global__ void __launch_bounds__(256)
    mfma_gap_kernel(const _Float16* __restrict__ operands, unsigned long long* __restrict__ clocks, float* sink, int iters) {
    __shared__ __align__(16) char lds[16384];
    for (int i = threadIdx.x; i < 1024; i += 256) reinterpret_cast<uint4*>(lds)[i] = reinterpret_cast<const uint4*>(operands)[i];
    __syncthreads();
    const f16x8* p = reinterpret_cast<const f16x8*>(operands) + threadIdx.x * 4;
    const f16x8 a = p[0], b = p[1];
    f32x4 acc[8];
    f32x16 acc32[4];
    for (int i = 0; i < 8; ++i) acc[i] = f32x4{0, 0, 0, 0};
    for (int i = 0; i < 4; ++i)
        for (int e = 0; e < 16; ++e) acc32[i][e] = 0.f;
    float x0 = float(p[2][0]), x1 = float(p[2][1]), x2 = float(p[2][2]), s = 0.f;
    unsigned int addr = (threadIdx.x & 63) * 16, u = threadIdx.x;
    f16x8 frag = p[3];
    const unsigned long long t0 = __builtin_amdgcn_s_memtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            if constexpr (k32x32) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc32[m % 4]) : "v"(a), "v"(b));
            else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[m]) : "v"(a), "v"(b));
            if constexpr (kFill == 1) asm volatile("v_add_f32 %0, %0, %1" : "+v"(x0) : "v"(x1));
            if constexpr (kFill == 2) asm volatile("v_add_f32 %0, %0, %2\n\tv_add_f32 %1, %1, %2" : "+v"(x0), "+v"(x1) : "v"(x2));
            if constexpr (kFill == 3)
                asm volatile("v_add_f32 %0, %0, %2\n\tv_add_f32 %1, %1, %2\n\tv_add_f32 %3, %3, %2" : "+v"(x0), "+v"(x1) : "v"(x2), "v"(s));
            if constexpr (kFill == 4)
                asm volatile("v_add_f32 %0, %0, %2\n\tv_add_f32 %1, %1, %2\n\tv_add_f32 %3, %3, %2\n\tv_add_f32 %4, %4, %2"
                             : "+v"(x0), "+v"(x1)
                             : "v"(x2), "v"(s), "v"(u));
            if constexpr (kFill == 5) asm volatile("v_exp_f32 %0, %1" : "=v"(x0) : "v"(x1));
            if constexpr (kFill == 6) asm volatile("v_exp_f32 %0, %1\n\tv_add_f32 %2, %2, %3" : "=v"(x0), "+v"(s) : "v"(x1), "v"(x2));
            if constexpr (kFill == 7)
                asm volatile("v_exp_f32 %0, %1\n\tv_add_f32 %2, %2, %3\n\tv_add_f32 %4, %4, %3" : "=v"(x0), "+v"(s) : "v"(x1), "v"(x2), "v"(u));
            if constexpr (kFill == 8) asm volatile("ds_read_b128 %0, %1" : "=v"(frag) : "v"(addr));
            if constexpr (kFill == 9) asm volatile("v_add_u32 %1, %1, %2\n\tds_read_b128 %0, %1" : "=v"(frag), "+v"(addr) : "s"(0));
            if constexpr (kFill == 10)
                asm volatile("ds_read_b64_tr_b16 %0, %1\n\tds_read_b64_tr_b16 %0, %1 offset:512" : "=v"(*reinterpret_cast<uint2*>(&frag)) : "v"(addr));
            if constexpr (kFill == 11) asm volatile("v_cvt_pk_f16_f32 %0, %1, %2\n\tv_add_f32 %3, %3, %2" : "=v"(u), "+v"(s) : "v"(x1), "v"(x2));
            if constexpr (kFill == 12) {
                if (m % 2 == 0) asm volatile("ds_read_b128 %0, %1" : "=v"(frag) : "v"(addr));
            }
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)");
    const unsigned long long t1 = __builtin_amdgcn_s_memtime();
    if (threadIdx.x == 0) clocks[blockIdx.x] = t1 - t0;
    for (int i = 0; i < 8; ++i) s += acc[i][0];
    for (int i = 0; i < 4; ++i) s += acc32[i][0];
    s += x0 + x1 + float(frag[0]) + float(u) + float(addr);
    if (s == 12345.678f) *sink = s;
}

template <bool k32x32>
int launch_gap(int fill, const _Float16* ops, unsigned long long* clk, float* snk, int workgroups, int iters, hipStream_t st) {
    const dim3 grid(workgroups), block(256);
    switch (fill) {
#define TCU_GAP_CASE(n)                                                                              \
    case n:                                                                                          \
        hipLaunchKernelGGL((mfma_gap_kernel<n, k32x32>), grid, block, 0, st, ops, clk, snk, iters); \
        break;
        TCU_GAP_CASE(0) TCU_GAP_CASE(1) TCU_GAP_CASE(2) TCU_GAP_CASE(3) TCU_GAP_CASE(4) TCU_GAP_CASE(5) TCU_GAP_CASE(6)
        TCU_GAP_CASE(7) TCU_GAP_CASE(8) TCU_GAP_CASE(9) TCU_GAP_CASE(10) TCU_GAP_CASE(11) TCU_GAP_CASE(12)
#undef TCU_GAP_CASE
        default: return int(hipErrorInvalidValue);
    }
    return int(hipGetLastError());
}

}  // namespace

// Issue cost of what sits between two matrix instructions (see mfma_gap_kernel). operands: at least 16 KiB + 256 lanes x
// 32 halves of fp16; clocks: `workgroups` u64; shape 0 = 32x32x16, 1 = 16x16x32; fill 0..12.
extern "C" int tcu_probe_mfma_gap(const void* operands, void* clocks, void* sink, int shape, int fill, int workgroups, int iters,
                                  void* stream) {
    if (workgroups <= 0 || iters <= 0) return int(hipErrorInvalidValue);
    auto* ops = static_cast<const _Float16*>(operands);
    auto* clk = static_cast<unsigned long long*>(clocks);
    auto* snk = static_cast<float*>(sink);
    return shape == 1 ? launch_gap<false>(fill, ops, clk, snk, workgroups, iters, static_cast<hipStream_t>(stream))
                      : launch_gap<true>(fill, ops, clk, snk, workgroups, iters, static_cast<hipStream_t>(stream));
}

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
