// Back-to-back GEMM D = f16(A·B)·C for gfx950 with every operand resident in LDS: the tuned counterpart of
// kernels/b2b_gemm.hpp (which follows the reference's examples/cpp/02_fused_two_gemms/fused_gemm.hpp:107-181).
// A [M, K] and D [M, P] row-major; B column-major [K, N] (stored [N, K]); C column-major [N, P] (stored [P, N]).
//
// With K = P = 128 and N = 256 the two weight matrices are 64 KiB each, so a workgroup can hold both in the CU's
// 160 KiB of LDS next to its 32 rows of A and its 32 x 256 intermediate; nothing is streamed:
//   * all loads (A, B, C: 136 KiB) are issued at once as direct-to-LDS loads, one memory round trip for the whole
//     kernel; the first product starts when A and B have landed, C is awaited before the second one;
//   * first product, split over the 8 wavefronts by n: wavefront w computes (A·B)ᵀ[n, m] for its 32 values of n with
//     v_mfma_f32_16x16x32_f16 (operands swapped, so a lane holds 4 consecutive n of one row m), rounds to f16 and
//     writes its slice of the intermediate to LDS;
//   * second product, split by p: wavefront w computes Dᵀ[p, m] for its 16 values of p over all 256 n, reading the
//     intermediate as the other operand; a lane ends up with 4 consecutive p of one row m and stores them;
//   * LDS rows are 256 B (A, B) or 512 B (C, intermediate); the 16-byte chunks are XOR-ed with row % 16 inside
//     every aligned group of 16 chunks, which makes the ds_read_b128 of 16 consecutive rows at one k-offset
//     conflict-free; for the loads the permutation is applied on the global-address side.
// Longer N (any multiple of 256, the reference's example also runs N = 1024 and 2048,
// examples/cpp/02_fused_two_gemms/fused_gemm.cu:236-259) is processed in blocks of 256 columns of B / rows of C through
// the same LDS buffers: the B buffer is refilled with the next block while the second product of the current block
// runs, the C buffer while the first product of the next block runs; the f32 accumulators of D stay in registers.
// The intermediate never leaves the chip. M % 32 == 0 and N % 256 == 0 are required (checked by the host launcher).
#pragma once

#include "config.hpp"
#include "hip_utils.hpp"
#include "kernels/gemm_pipelined.hpp"  // detail::load_lds_16B_untracked

namespace tiledcuda::kernels {

struct B2bResidentTraits {
    static constexpr int kN = 256, kK = 128, kP = 128;
    static constexpr int kTM = 32;  // rows of A / D per workgroup
    static constexpr int kWaves = 8, kThreads = kWaves * kWaveSize;
    static constexpr int kRowBytesK = 2 * kK;  // rows of A and B
    static constexpr int kRowBytesN = 2 * kN;  // rows of C and of the intermediate
    static constexpr int kAOff = 0;
    static constexpr int kBOff = kAOff + kTM * kRowBytesK;
    static constexpr int kCOff = kBOff + kN * kRowBytesK;
    static constexpr int kSOff = kCOff + kP * kRowBytesN;
    static constexpr int kLdsBytes = kSOff + kTM * kRowBytesN;
    static_assert(kLdsBytes <= kMaxLdsBytes);
    /// Physical 16-byte chunk of logical chunk c in row `row` (rows of 16 or 32 chunks).
    HOST_DEVICE static constexpr int swz(int c, int row) { return (c & 16) | ((c & 15) ^ (row & 15)); }
};

/// grid = (M / 32, batch), block = 512, dynamic LDS = B2bResidentTraits::kLdsBytes. N: columns of B = rows of C.
template <typename OutType>
__global__ void __launch_bounds__(B2bResidentTraits::kThreads)
    b2b_gemm_resident(const __half* __restrict__ A, const __half* __restrict__ B, const __half* __restrict__ C,
                      OutType* __restrict__ D, int M, int N) {
    using T = B2bResidentTraits;
    constexpr int kN = T::kN, kK = T::kK, kP = T::kP;  // kN: the block of N held in LDS at a time
    extern __shared__ __align__(1024) unsigned char lds[];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int L = lane & 15, g = lane >> 4;
    const int m0 = blockIdx.x * T::kTM;
    const size_t batch = blockIdx.y;
    const __half* Ab = A + (batch * M + m0) * kK;
    const __half* Bb = B + batch * size_t(N) * kK;
    const __half* Cb = C + batch * size_t(kP) * N;
    OutType* Db = D + (batch * M + m0) * kP;
    const int nblocks = N / kN;

    // block nb of B: rows 256 nb .. of the stored [N, K] array (8 instructions of 1 KiB per wavefront)
    auto load_b = [&](int nb) {
        const int r4 = lane >> 4, c16 = lane & 15;  // 256-byte rows: 4 rows x 16 chunks per instruction
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int q = 8 * wave + j;
            const int row = 4 * q + r4;
            detail::load_lds_16B_untracked(Bb + (size_t(nb) * kN + row) * kK + (c16 ^ (row & 15)) * 8,
                                           lds + T::kBOff + q * 1024);
        }
    };
    // block nb of C: columns 256 nb .. of the stored [P, N] array (8 instructions per wavefront)
    auto load_c = [&](int nb) {
        const int r2 = lane >> 5, c32 = lane & 31;  // 512-byte rows: 2 rows x 32 chunks per instruction
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int q = 8 * wave + j;
            const int row = 2 * q + r2;
            detail::load_lds_16B_untracked(Cb + size_t(row) * N + size_t(nb) * kN + T::swz(c32, row) * 8,
                                           lds + T::kCOff + q * 1024);
        }
    };
    // ---- everything of the first block in flight at once: A (1 instruction per wavefront), B (8), C (8)
    {
        const int r4 = lane >> 4, c16 = lane & 15;
        const int row = 4 * wave + r4;
        detail::load_lds_16B_untracked(Ab + size_t(row) * kK + (c16 ^ (row & 15)) * 8, lds + T::kAOff + wave * 1024);
    }
    load_b(0);
    load_c(0);

    f32x4 acc2[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
    for (int nb = 0; nb < nblocks; ++nb) {
    // the B block (and A) have landed - this wavefront's share (the 8 younger loads, of the C block, may still be in
    // flight), then everyone's; everyone is done with the previous block's C and intermediate
    detail::lds_barrier<8>();

    // ---- first product: acc1[nt][mt][r] = (A·B)[m = 16 mt + L][n = 32 wave + 16 nt + 4 g + r]
    f32x4 acc1[2][2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) acc1[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < kK / 32; ++s) {
        f16x8 fb[2], fa[2];
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
            const int n = 32 * wave + 16 * nt + L;
            fb[nt] = *reinterpret_cast<const f16x8*>(lds + T::kBOff + n * T::kRowBytesK + T::swz(4 * s + g, n) * 16);
        }
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            const int m = 16 * mt + L;
            fa[mt] = *reinterpret_cast<const f16x8*>(lds + T::kAOff + m * T::kRowBytesK + T::swz(4 * s + g, m) * 16);
        }
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
                acc1[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[nt], fa[mt], acc1[nt][mt], 0, 0, 0);
    }
    // the intermediate, rounded to f16 (part of the specification of this operation), to LDS: 8 bytes per lane
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            const int m = 16 * mt + L;
            const int chunk = 4 * wave + 2 * nt + (g >> 1);  // n / 8 with n = 32 wave + 16 nt + 4 g
            f16x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = static_cast<_Float16>(acc1[nt][mt][e]);
            *reinterpret_cast<f16x4*>(lds + T::kSOff + m * T::kRowBytesN + T::swz(chunk, m) * 16 + (g & 1) * 8) = v;
        }
    detail::lds_barrier<0>();  // C has landed, the intermediate is written, the B buffer is free; for everyone
    if (nb + 1 < nblocks) load_b(nb + 1);  // under the second product

    // ---- second product: acc2[mt][r] += D[m = 16 mt + L][p = 16 wave + 4 g + r] over this block's n
    const int p_row = 16 * wave + L;
#pragma unroll
    for (int s = 0; s < kN / 32; ++s) {
        const f16x8 fc =
            *reinterpret_cast<const f16x8*>(lds + T::kCOff + p_row * T::kRowBytesN + T::swz(4 * s + g, p_row) * 16);
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            const int m = 16 * mt + L;
            const f16x8 fs =
                *reinterpret_cast<const f16x8*>(lds + T::kSOff + m * T::kRowBytesN + T::swz(4 * s + g, m) * 16);
            acc2[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fc, fs, acc2[mt], 0, 0, 0);
        }
    }
    if (nb + 1 < nblocks) {
        // everyone is done with this block's C and intermediate: the C buffer is refilled under the next first product
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's LDS reads have returned
        __builtin_amdgcn_s_barrier();
        load_c(nb + 1);
    }
    }  // blocks of N
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
        OutType* dst = Db + size_t(16 * mt + L) * kP + 16 * wave + 4 * g;
        if constexpr (sizeof(OutType) == 4) {
            *reinterpret_cast<f32x4*>(dst) = acc2[mt];
        } else {
            f16x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = static_cast<_Float16>(acc2[mt][e]);
            *reinterpret_cast<f16x4*>(dst) = v;
        }
    }
}

}  // namespace tiledcuda::kernels
