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
#include "kernels/gemm_w128.hpp"       // detail::mfma_16x16x32_agpr

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
    static constexpr int kDOff = kSOff + kTM * kRowBytesN;  // the f16 output tile on its way out: 32 rows of 256 bytes
    static constexpr int kLdsBytes = kDOff + kTM * kP * 2;  // 160 KiB
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
    if constexpr (sizeof(OutType) == 4) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
            *reinterpret_cast<f32x4*>(Db + size_t(16 * mt + L) * kP + 16 * wave + 4 * g) = acc2[mt];
    } else {
        // f16: the tile is gathered in LDS (8-byte slots of a row XOR-ed with twice the row) and leaves as whole 256-byte
        // rows, one 16-byte piece per lane, through non-temporal stores - a wavefront's own share is 32 bytes of every
        // row, which the L2 would have to gather into lines and write back after the kernel's last wavefront
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            f16x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = static_cast<_Float16>(acc2[mt][e]);
            const int row = 16 * mt + L;
            *reinterpret_cast<f16x4*>(lds + T::kDOff + row * (kP * 2) + (((4 * wave + g) ^ (2 * row)) & 31) * 8) = v;
        }
        __syncthreads();
        const int row = threadIdx.x >> 4, c = threadIdx.x & 15;
        const u32x4 v = *reinterpret_cast<const u32x4*>(lds + T::kDOff + row * (kP * 2) + (((2 * c) ^ (2 * row)) & 31) * 8);
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(Db + size_t(row) * kP + 8 * c));
    }
}

/// The same product for many rows (M x batch in the tens of thousands and more), N = 256: with 32 rows per
/// workgroup every workgroup re-reads both weight blocks (128 KiB) from the L2 for 16 KiB of A and D, and every
/// wavefront re-reads the whole A tile and the whole intermediate from LDS. Here a workgroup (4 wavefronts, one per
/// SIMD, 512 registers each) keeps B and C in LDS for its whole life and walks over blocks of 256 rows; inside a block
/// every wavefront owns 64 rows outright:
///   * its A fragments come straight from global memory into registers (16 bytes per lane, fetched one block ahead);
///   * first product for 128 n at a time: 32 ds_read_b128 of B for 128 MFMAs, accumulators = 128 registers;
///   * the accumulators, rounded to f16, are the second product's operand without leaving the lane: a lane holds
///     n = 4 g .. + 3 of two adjacent 16-wide n-tiles, which are declared to be the 8 contraction slots of lane group
///     g; the C fragment is read in the same slot order (two 8-byte reads per fragment);
///   * no barrier after the first one and no LDS traffic for A or the intermediate: per 64 rows 128 KiB of LDS reads
///     for 512 MFMAs, i.e. half of the CU's LDS bandwidth (128 B/clk) at the full rate of its matrix pipes.
/// grid = (row blocks a workgroup strides over, batch), block = 256, dynamic LDS = B2bRowsTraits::kLdsBytes.
/// M % 64 == 0 (a wavefront's 64 rows exist or do not).
namespace detail {
/// acc = a · b on the matrix pipe (no accumulator input), result in AGPRs.
DEVICE void mfma_16x16x32_agpr_zero(f32x4& acc, const f16x8& a, const f16x8& b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
}
/// LDS reads as assembly the compiler does not track, with the kernel's own lgkmcnt waits (with one wavefront per SIMD
/// nothing else covers the LDS latency, and the compiler's own waits come directly before the first use).
template <int kOff>
DEVICE f16x8 lds_read_b128_at(unsigned int addr) {
    f16x8 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(kOff));
    return r;
}
/// Two 8-byte reads forming one 16-byte MFMA operand.
template <int kOff>
DEVICE f16x8 lds_read_b64_pair_at(unsigned int addr_lo, unsigned int addr_hi) {
    f16x4 lo, hi;
    asm volatile("ds_read_b64 %0, %2 offset:%4\n\tds_read_b64 %1, %3 offset:%4"
                 : "=&v"(lo), "=&v"(hi)
                 : "v"(addr_lo), "v"(addr_hi), "n"(kOff));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
/// Wait until at most kOutstanding of this wavefront's LDS reads are outstanding (they return in order).
template <int kOutstanding>
DEVICE void lds_wait_outstanding() {
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kOutstanding) : "memory");
}
}  // namespace detail

struct B2bRowsTraits {
    static constexpr int kN = 256, kK = 128, kP = 128;
    static constexpr int kRowsPerWave = 64, kWaves = 4, kThreads = kWaves * kWaveSize;
    static constexpr int kMT = kRowsPerWave / 16;
    static_assert(kMT == 4, "the waiting statements name four accumulators per row of tiles");
    static constexpr int kRowsPerBlock = kRowsPerWave * kWaves;
    static constexpr int kFragAhead = 3;  // weight fragments requested ahead of their MFMAs (4 MFMAs = 64 cycles each)
    static constexpr int kRowBytesK = 2 * kK, kRowBytesN = 2 * kN;
    static constexpr int kBOff = 0;
    static constexpr int kCOff = kBOff + kN * kRowBytesK;
    static constexpr int kStageOff = kCOff + kP * kRowBytesN;   // 128 KiB of weights, then the f16 output staging:
    static constexpr int kStageBytesPerWave = 16 * kP * 2;      // 16 rows of D per wavefront
    static constexpr int kLdsBytes = kStageOff + kWaves * kStageBytesPerWave;  // 144 KiB
    static_assert(kLdsBytes <= kMaxLdsBytes);
};

template <typename OutType>
__global__ void __launch_bounds__(B2bRowsTraits::kThreads)
    b2b_gemm_rows(const __half* __restrict__ A, const __half* __restrict__ B, const __half* __restrict__ C,
                  OutType* __restrict__ D, int M) {
    using T = B2bRowsTraits;
    using R = B2bResidentTraits;  // the swizzle of the weight blocks
    constexpr int kN = T::kN, kK = T::kK, kP = T::kP, kMT = T::kMT;
    constexpr int kAhead = T::kFragAhead, kRing = kAhead + 1;
    extern __shared__ __align__(1024) unsigned char lds[];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int L = lane & 15, g = lane >> 4;
    const size_t batch = blockIdx.y;
    const __half* Ab = A + batch * size_t(M) * kK;
    const __half* Bb = B + batch * size_t(kN) * kK;
    const __half* Cb = C + batch * size_t(kP) * kN;
    OutType* Db = D + batch * size_t(M) * kP;

    // ---- both weight blocks, once: 16 + 16 direct-to-LDS instructions of 1 KiB per wavefront
    {
        const int r4 = lane >> 4, c16 = lane & 15;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int q = 16 * wave + j;
            const int row = 4 * q + r4;
            detail::load_lds_16B_untracked(Bb + size_t(row) * kK + (c16 ^ (row & 15)) * 8, lds + T::kBOff + q * 1024);
        }
        const int r2 = lane >> 5, c32 = lane & 31;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int q = 16 * wave + j;
            const int row = 2 * q + r2;
            detail::load_lds_16B_untracked(Cb + size_t(row) * kN + R::swz(c32, row) * 8, lds + T::kCOff + q * 1024);
        }
    }
    // fragment (mt, s) of the wavefront's rows: row 16 mt + L, k = 32 s + 8 g .. + 7
    auto load_a = [&](int row0, f16x8(&fa)[kMT][4]) {
#pragma unroll
        for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                fa[mt][s] = *reinterpret_cast<const f16x8*>(Ab + size_t(row0 + 16 * mt + L) * kK + 32 * s + 8 * g);
            }
    };
    // LDS addresses of the weight fragments, per lane: B row L (+ an immediate per n-tile), chunk 4 s + g; C row L (+ an
    // immediate per p-tile), the 8-byte halves at n = 128 half + 32 s2 + 4 g and 16 further
    const unsigned int lds_base = static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds));
    unsigned int b_addr[4], c_addr_lo[2][4], c_addr_hi[2][4];
#pragma unroll
    for (int s = 0; s < 4; ++s) b_addr[s] = lds_base + T::kBOff + L * T::kRowBytesK + R::swz(4 * s + g, L) * 16;
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2) {
            const int c0 = 16 * half + 4 * s2 + (g >> 1);  // 16-byte chunk of n = 128 half + 32 s2 + 4 g
            c_addr_lo[half][s2] = lds_base + T::kCOff + L * T::kRowBytesN + (g & 1) * 8 + R::swz(c0, L) * 16;
            c_addr_hi[half][s2] = lds_base + T::kCOff + L * T::kRowBytesN + (g & 1) * 8 + R::swz(c0 + 2, L) * 16;
        }
    const int blocks = (M + T::kRowsPerBlock - 1) / T::kRowsPerBlock;
    f16x8 fa[kMT][4];
    {
        const int row0 = blockIdx.x * T::kRowsPerBlock + wave * T::kRowsPerWave;
        if (row0 < M) load_a(row0, fa);
    }
    detail::lds_barrier<0>();  // B and C have landed, for everyone

    for (int blk = blockIdx.x; blk < blocks; blk += gridDim.x) {
        const int row0 = blk * T::kRowsPerBlock + wave * T::kRowsPerWave;
        const int next0 = (blk + int(gridDim.x)) * T::kRowsPerBlock + wave * T::kRowsPerWave;
        f16x8 fa_next[kMT][4];
        if (next0 < M) load_a(next0, fa_next);
        if (row0 < M) {
            // acc2[pt][mt][r] = D[m = row0 + 16 mt + L][p = 16 pt + 4 g + r]
            f32x4 acc2[8][kMT];
            // N in two halves of 128, so that the first product's accumulators are 128 registers, not 256.
            // (The MFMAs are assembly with accumulators constrained to AGPRs: left to the compiler, 256 accumulator
            // registers next to 128 of A fragments wander between the register files and spill. The LDS reads are
            // assembly too, issued kAhead fragments ahead of the MFMAs that use them.)
            detail::static_for<2>([&](auto half_c) {
                constexpr int half = decltype(half_c)::value;
                // ---- first product: acc1[nt][mt][r] = (A.B)[m = row0 + 16 mt + L][n = 128 half + 16 nt + 4 g + r];
                // fragment idx = 8 s + nt of B: row n = 128 half + 16 nt + L, chunk 4 s + g
                f32x4 acc1[8][kMT];
                f16x8 fb[kRing];
                auto read_b = [&](auto idx_c) {
                    constexpr int idx = decltype(idx_c)::value, s = idx >> 3, nt = idx & 7;
                    fb[idx % kRing] = detail::lds_read_b128_at<(128 * half + 16 * nt) * T::kRowBytesK>(b_addr[s]);
                };
                detail::static_for<kAhead>([&](auto i_c) { read_b(i_c); });
                detail::static_for<32>([&](auto idx_c) {
                    constexpr int idx = decltype(idx_c)::value, s = idx >> 3, nt = idx & 7;
                    if constexpr (idx + kAhead < 32) read_b(std::integral_constant<int, idx + kAhead>{});
                    detail::lds_wait_outstanding<(idx + kAhead < 32 ? kAhead : 31 - idx)>();
#pragma unroll
                    for (int mt = 0; mt < kMT; ++mt) {
                        if (s == 0) detail::mfma_16x16x32_agpr_zero(acc1[nt][mt], fb[idx % kRing], fa[mt][s]);
                        else detail::mfma_16x16x32_agpr(acc1[nt][mt], fb[idx % kRing], fa[mt][s]);
                    }
                });
                // the compiler does not know the statements above are MFMAs: wait once for the last results, then pass every
                // accumulator through a statement that comes after the wait
                detail::mfma_results_wait();
#pragma unroll
                for (int nt = 0; nt < 8; ++nt)
                    asm volatile("" : "+a"(acc1[nt][0]), "+a"(acc1[nt][1]), "+a"(acc1[nt][2]), "+a"(acc1[nt][3]));

                // ---- second product over this half's n: contraction step s2 covers n = 128 half + 32 s2 .. + 31, lane
                // group g holding n = .. + 4 g .. + 3 and .. + 16 + 4 g .. + 3 (the two halves of its operand); fragment
                // idx = 8 s2 + pt of C: row p = 16 pt + L, the 8 bytes at n = .. + 4 g and at n = .. + 16 + 4 g
                f16x8 fs[2][kMT], fc[kRing];
                auto convert = [&](auto s2_c) {
                    constexpr int s2 = decltype(s2_c)::value;
#pragma unroll
                    for (int mt = 0; mt < kMT; ++mt) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            fs[s2 & 1][mt][e] = static_cast<_Float16>(acc1[2 * s2][mt][e]);  // the f16 rounding of the intermediate
                            fs[s2 & 1][mt][4 + e] = static_cast<_Float16>(acc1[2 * s2 + 1][mt][e]);
                        }
                        asm volatile("" : "+v"(fs[s2 & 1][mt]));  // here, not at the first use
                    }
                };
                auto read_c = [&](auto idx_c) {
                    constexpr int idx = decltype(idx_c)::value, s2 = idx >> 3, pt = idx & 7;
                    fc[idx % kRing] = detail::lds_read_b64_pair_at<16 * pt * T::kRowBytesN>(c_addr_lo[half][s2], c_addr_hi[half][s2]);
                };
                detail::static_for<kAhead>([&](auto i_c) { read_c(i_c); });
                convert(std::integral_constant<int, 0>{});
                asm volatile("s_nop 4" ::: "memory");  // the conversions' results are read by MFMAs the compiler does not see
                detail::static_for<32>([&](auto idx_c) {
                    constexpr int idx = decltype(idx_c)::value, s2 = idx >> 3, pt = idx & 7;
                    if constexpr (idx + kAhead < 32) read_c(std::integral_constant<int, idx + kAhead>{});
                    detail::lds_wait_outstanding<(idx + kAhead < 32 ? 2 * kAhead : 2 * (31 - idx))>();
#pragma unroll
                    for (int mt = 0; mt < kMT; ++mt) {
                        if (half == 0 && s2 == 0) detail::mfma_16x16x32_agpr_zero(acc2[pt][mt], fc[idx % kRing], fs[s2 & 1][mt]);
                        else detail::mfma_16x16x32_agpr(acc2[pt][mt], fc[idx % kRing], fs[s2 & 1][mt]);
                    }
                    // the next step's operand is converted under this step's MFMAs
                    if constexpr (pt == 2 && s2 + 1 < 4) convert(std::integral_constant<int, s2 + 1>{});
                });
            });
            detail::mfma_results_wait();
#pragma unroll
            for (int pt = 0; pt < 8; ++pt)
                asm volatile("" : "+a"(acc2[pt][0]), "+a"(acc2[pt][1]), "+a"(acc2[pt][2]), "+a"(acc2[pt][3]));
            if constexpr (sizeof(OutType) == 4) {
#pragma unroll
                for (int pt = 0; pt < 8; ++pt)
#pragma unroll
                    for (int mt = 0; mt < kMT; ++mt)
                        *reinterpret_cast<f32x4*>(Db + size_t(row0 + 16 * mt + L) * kP + 16 * pt + 4 * g) = acc2[pt][mt];
            } else {
                // f16: 16 rows at a time through 4 KiB of LDS of this wavefront's own (the 8-byte slots of a row XOR-ed with
                // twice the row), so that D leaves as whole 256-byte rows, 16 bytes per lane, through non-temporal stores:
                // 8-byte pieces would have to be gathered into lines by the L2, and lines left dirty there are written
                // back after the kernel's last wavefront
                using lds_f16x4_ptr = __attribute__((address_space(3))) f16x4*;
                using lds_u32x4_ptr = __attribute__((address_space(3))) const u32x4*;
                const unsigned int stg = lds_base + T::kStageOff + wave * T::kStageBytesPerWave;
                const int q4 = lane >> 4, c = lane & 15;  // read-back: row 4 it + q4, 16-byte piece c
#pragma unroll
                for (int mt = 0; mt < kMT; ++mt) {
#pragma unroll
                    for (int pt = 0; pt < 8; ++pt) {
                        f16x4 v;
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = static_cast<_Float16>(acc2[pt][mt][e]);
                        *reinterpret_cast<lds_f16x4_ptr>(stg + L * (kP * 2) + (((4 * pt + g) ^ (2 * L)) & 31) * 8) = v;
                    }
                    // LDS operations of one wavefront execute in order: the reads see the writes above, the next
                    // row group's writes come behind them
#pragma unroll
                    for (int it = 0; it < 4; ++it) {
                        const int q = 4 * it + q4;
                        const u32x4 v = *reinterpret_cast<lds_u32x4_ptr>(stg + q * (kP * 2) + (((2 * c) ^ (2 * q)) & 31) * 8);
                        __builtin_nontemporal_store(
                            v, reinterpret_cast<u32x4*>(Db + size_t(row0 + 16 * mt + q) * kP + 8 * c));
                    }
                }
            }
        }
        if (next0 < M) {
#pragma unroll
            for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
                for (int s = 0; s < 4; ++s) fa[mt][s] = fa_next[mt][s];
        }
    }
}

}  // namespace tiledcuda::kernels
