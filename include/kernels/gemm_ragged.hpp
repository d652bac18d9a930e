// GEMM C[M, N] = A[M, K] · B[K, N] for shapes that are whole 16 x 16 BaseTiles and nothing more: M, N and K any
// multiples of 16, known at run time. A row-major, B column-major (stored [N, K]), C row-major.
//
// The reference's kernels take their shapes as template arguments in multiples of the 16 x 16 BaseTile
// (examples/cpp/01_gemm/01_gemm_global_reg/gemm.hpp:40-68, include/types/register.hpp:108-112), so any such shape can
// be instantiated there; behind a C interface the shape arrives at run time, and this kernel is where shapes go that
// the tiled kernels' 64-element granularity does not cover. It is the global -> register GEMM of that example with
// run-time extents: register tiles of MFMA operand tiles (types/mfma_tile.hpp) filled straight from global memory -
// one lane's share of a 16 x 32 operand tile is 16 consecutive bytes of one row - and cell::compute::gemm() on them.
// A workgroup of 4 wavefronts owns a 64 x 64 block of C, a wavefront 32 x 32 of it (2 x 2 BaseTiles); BaseTiles
// beyond M or N are not loaded (their operand tiles stay zero) and not stored. A last k-step of 16 is the upper half
// of a 32-wide operand tile left zero.
#pragma once

#include "cell/mod.hpp"
#include "types/mod.hpp"

namespace tiledcuda::kernels {
using namespace tiledcuda::cell;
namespace tl = tile_layout;

struct RaggedGemmTraits {
    static constexpr int kBM = 64, kBN = 64;
    static constexpr int kWaves = 4, kThreads = kWaves * kWaveSize;
    using RegA = RegTile<MfmaTileA16x32<__half>, tl::RowMajor<2, 1>>;
    using RegB = RegTile<MfmaTileB32x16<__half>, tl::ColMajor<1, 2>>;
    using RegC = RegTile<BaseTileRowMajor<float>, tl::RowMajor<2, 2>>;
};

/// grid = ceil(M / 64) * ceil(N / 64) workgroups of 256 threads, no LDS. M, N, K multiples of 16.
template <typename OutType>
__global__ void __launch_bounds__(RaggedGemmTraits::kThreads)
    gemm_ragged(const __half* __restrict__ A, const __half* __restrict__ B, OutType* __restrict__ C, int M, int N,
                int K) {
    using T = RaggedGemmTraits;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int blocks_n = (N + T::kBN - 1) / T::kBN;
    const int m0 = (blockIdx.x / blocks_n) * T::kBM + 32 * (wave >> 1);
    const int n0 = (blockIdx.x % blocks_n) * T::kBN + 32 * (wave & 1);
    const int line = lane & 15, group = lane >> 4;  // operand tiles: line = row of A / column of B, k = 8 group ..

    const __half* a_line[2];
    const __half* b_line[2];
    bool a_in[2], b_in[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        a_in[t] = m0 + 16 * t < M;  // uniform over the wavefront: whole BaseTiles only
        b_in[t] = n0 + 16 * t < N;
        a_line[t] = A + size_t(a_in[t] ? m0 + 16 * t + line : 0) * K + 8 * group;
        b_line[t] = B + size_t(b_in[t] ? n0 + 16 * t + line : 0) * K + 8 * group;
    }

    typename T::RegA a;
    typename T::RegB b;
    typename T::RegC acc;
    for (int k = 0; k < K; k += 32) {
        // the upper 16 of a 32-wide step may lie beyond K (K % 32 == 16): lanes holding it keep zeros
        const bool k_in = k + 8 * group < K;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            f16x8 av = {0, 0, 0, 0, 0, 0, 0, 0}, bv = {0, 0, 0, 0, 0, 0, 0, 0};
            if (a_in[t] && k_in) av = *reinterpret_cast<const f16x8*>(a_line[t] + k);
            if (b_in[t] && k_in) bv = *reinterpret_cast<const f16x8*>(b_line[t] + k);
            __builtin_memcpy(a(t, 0).mutable_data(), &av, sizeof(av));
            __builtin_memcpy(b(0, t).mutable_data(), &bv, sizeof(bv));
        }
        compute::gemm(a, b, acc);
    }

    // a lane of a row-major accumulator BaseTile holds row `line`, columns 4 group .. + 3
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (!a_in[i] || !b_in[j]) continue;
            OutType* dst = C + size_t(m0 + 16 * i + line) * N + n0 + 16 * j + 4 * group;
            f32x4 v;
            __builtin_memcpy(&v, acc(i, j).data(), sizeof(v));
            if constexpr (sizeof(OutType) == 4) {
                *reinterpret_cast<f32x4*>(dst) = v;
            } else {
                f16x4 h;
#pragma unroll
                for (int e = 0; e < 4; ++e) h[e] = static_cast<_Float16>(v[e]);
                *reinterpret_cast<f16x4*>(dst) = h;
            }
        }
    }
}

}  // namespace tiledcuda::kernels
