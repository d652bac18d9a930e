// One time step of the fused LSTM layer for any batch, input and hidden size in multiples of 16, known at run time:
// the fallback for shapes the tuned step kernel (kernels/lstm_fwd.hpp) is not instantiated for. Same contract:
// gates = concat(x_t, h_{t-1}) · Wᵀ + bias (W [4H, I + H], gate rows i, f, g, o), c_t = σ(f) c_{t-1} + σ(i) tanh(g),
// h_t = σ(o) tanh(c_t); f16 operands, f32 gates and cell state. The reference has no LSTM kernel (its Makefile:3 only
// names a test); its tile types come in whole 16 x 16 BaseTiles, which is the granularity kept here.
//
// Like kernels/gemm_ragged.hpp it is the global -> register composition: a wavefront owns 16 batch rows x 16 hidden
// units and all four gates of them - four accumulator BaseTiles filled by cell::compute::gemm() on MFMA operand tiles
// read straight from global memory (16 bytes of one row per lane: rows of [x_t | h_{t-1}] as the A operand, the four
// weight rows gate * H + unit as B operands). The accumulators are row-major BaseTiles, so a lane holds the four gates
// of (batch row lane % 16, units 4 (lane / 16) .. + 3) in the same positions of the four tiles: the cell update is
// lane-local. A workgroup is 4 wavefronts = 64 hidden units of one 16-row batch block. The k loop runs over the I
// columns of x_t, then over the H columns of h_{t-1}; a last step of 16 leaves the upper half of the 32-wide operand
// tiles zero.
#pragma once

#include "cell/mod.hpp"
#include "kernels/lstm_fwd.hpp"  // detail::sigmoid_fast, tanh_fast
#include "types/mod.hpp"

namespace tiledcuda::kernels {
using namespace tiledcuda::cell;
namespace tl = tile_layout;

struct RaggedLstmTraits {
    static constexpr int kRows = 16;                  // batch rows per workgroup
    static constexpr int kWaves = 4, kThreads = kWaves * kWaveSize;
    static constexpr int kUnits = 16 * kWaves;        // hidden units per workgroup
    using RegA = RegTile<MfmaTileA16x32<__half>, tl::RowMajor<1, 1>>;
    using RegB = RegTile<MfmaTileB32x16<__half>, tl::ColMajor<1, 4>>;  // the four gates
    using RegAcc = RegTile<BaseTileRowMajor<float>, tl::RowMajor<1, 4>>;
};

/// grid = (ceil(H / 64), B / 16), block = 256. h_in / c_in may be null (zeros). B, I, H multiples of 16.
__global__ void __launch_bounds__(RaggedLstmTraits::kThreads)
    lstm_cell_ragged(const __half* __restrict__ x_t, const __half* __restrict__ h_in, const __half* __restrict__ W,
                     const __half* __restrict__ bias, const float* __restrict__ c_in, float* __restrict__ c_out,
                     __half* __restrict__ h_out, int B, int I, int H) {
    using T = RaggedLstmTraits;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int unit0 = blockIdx.x * T::kUnits + 16 * wave;
    if (unit0 >= H) return;  // whole BaseTiles only: uniform over the wavefront
    const int row0 = blockIdx.y * T::kRows;
    const int line = lane & 15, group = lane >> 4;
    const int KK = I + H;

    const __half* x_line = x_t + size_t(row0 + line) * I + 8 * group;
    const __half* h_line = h_in ? h_in + size_t(row0 + line) * H + 8 * group : nullptr;
    const __half* w_line[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) w_line[g] = W + size_t(g * H + unit0 + line) * KK + 8 * group;

    typename T::RegA a;
    typename T::RegB b;
    typename T::RegAcc acc;
    auto k_range = [&](const __half* src_line, int k_len, int w_col0) {
        for (int k = 0; k < k_len; k += 32) {
            const bool k_in = k + 8 * group < k_len;  // the upper 16 of the last step may lie beyond the range
            f16x8 av = {0, 0, 0, 0, 0, 0, 0, 0};
            if (k_in) av = *reinterpret_cast<const f16x8*>(src_line + k);
            __builtin_memcpy(a(0, 0).mutable_data(), &av, sizeof(av));
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f16x8 bv = {0, 0, 0, 0, 0, 0, 0, 0};
                if (k_in) bv = *reinterpret_cast<const f16x8*>(w_line[g] + w_col0 + k);
                __builtin_memcpy(b(0, g).mutable_data(), &bv, sizeof(bv));
            }
            compute::gemm(a, b, acc);
        }
    };
    k_range(x_line, I, 0);
    if (h_line) k_range(h_line, H, I);

    // acc(0, g)(e): gate g of batch row row0 + line, hidden unit unit0 + 4 group + e
    const int brow = row0 + line, hid = unit0 + 4 * group;
    f32x4 c_prev = {0.f, 0.f, 0.f, 0.f};
    if (c_in) c_prev = *reinterpret_cast<const f32x4*>(c_in + size_t(brow) * H + hid);
    f32x4 c_new;
    f16x4 h_new;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float gate[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) gate[g] = acc(0, g)(0, e) + __half2float(bias[g * H + hid + e]);
        const float cn = detail::sigmoid_fast(gate[1]) * c_prev[e] + detail::sigmoid_fast(gate[0]) * detail::tanh_fast(gate[2]);
        c_new[e] = cn;
        h_new[e] = static_cast<_Float16>(detail::sigmoid_fast(gate[3]) * detail::tanh_fast(cn));
    }
    *reinterpret_cast<f32x4*>(c_out + size_t(brow) * H + hid) = c_new;
    *reinterpret_cast<f16x4*>(h_out + size_t(brow) * H + hid) = h_new;
}

}  // namespace tiledcuda::kernels
