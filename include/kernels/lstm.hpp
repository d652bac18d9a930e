// One time step of a fused LSTM layer, composed from the tile primitives:
//   gates[B, 4H] = concat(x_t, h_{t-1})[B, I+H] · W^T + bias,   W [4H, I+H] row-major,
//   gate order i, f, g, o;  c_t = sigmoid(f)·c_{t-1} + sigmoid(i)·tanh(g);
//   h_t = sigmoid(o)·tanh(c_t).  Weights, x, h, bias are f16; gates and c are f32.
// The gate GEMM and the cell update are one kernel: a workgroup owns kTM batch rows and kTH
// hidden units and computes all four gates for them, so the update happens in registers and
// the [B, 4H] gate matrix never reaches memory.
//
// The reference snapshot has no LSTM kernel (only Makefile:3 names a test_lstm_cell); the
// structure follows the library's own GEMM kernels (global -> LDS -> register -> MFMA).
#pragma once

#include "cell/mod.hpp"
#include "types/mod.hpp"

namespace tiledcuda::kernels {

using namespace tiledcuda::cell;
using namespace tiledcuda::cell::copy;
namespace tl = tile_layout;

/// kI, kH: input and hidden width (compile-time: every leading dimension depends on them).
template <typename InType, typename AccType, const int kI_, const int kH_, const int kTM_ = 64, const int kTH_ = 16,
          const int kTK_ = 64, typename WarpLayout_ = tl::RowMajor<4, 1>>
struct LstmCellTraits {
    using BaseShape = traits::BaseTileShape<InType>;
    using WarpLayout = WarpLayout_;
    static constexpr int kI = kI_, kH = kH_, kTM = kTM_, kTH = kTH_, kTK = kTK_;
    static constexpr int kKK = kI + kH;  // reduction length
    static constexpr int kTG = 4 * kTH;  // gate columns per workgroup

    static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
    static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;
    static_assert(kWarpPerCol == 1, "wavefronts are stacked along the batch rows");
    static_assert(kI % kTK == 0 && kH % kTK == 0, "a K chunk must not straddle x and h");
    static constexpr int kThreads = tl::get_numel<WarpLayout> * kWaveSize;

    // A operand: a [kTM, kTK] block of x_t (leading dimension kI) or h_{t-1} (kH)
    using GlobalX = GlobalTile<InType, tl::RowMajor<kTM, kTK, kI>>;
    using GlobalHin = GlobalTile<InType, tl::RowMajor<kTM, kTK, kH>>;
    using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, true>;
    static constexpr int kAMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kAKs = kTK / BaseShape::kTileSize;
    using RegA = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAMs, kAKs>>;
    using G2SLoaderA = GlobalToSharedLoader<SharedA, WarpLayout>;
    using S2RLoaderA = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

    // B operand: four [kTK, kTH] column-major blocks of W^T (one per gate), side by side in LDS
    using GlobalW = GlobalTile<InType, tl::ColMajor<kTK, kTH, kKK>>;
    using SharedW = SharedTile<InType, tl::ColMajor<kTK, kTG>, true>;
    using SIteratorW = STileIterator<SharedW, TileShape<kTK, kTH>>;
    using SharedWGate = SharedTile<InType, tl::MatrixLayout<kTK, kTH, 1, kTK>, true>;
    using G2SLoaderW = GlobalToSharedLoader<SharedWGate, WarpLayout>;
    static constexpr int kBKs = kTK / BaseShape::kTileSize;
    static constexpr int kBNs = kTG / BaseShape::kTileSize;
    using RegB = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kBKs, kBNs>>;
    using S2RLoaderB = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

    // gate accumulators [kTM, 4*kTH] and the per-gate [kTM, kTH] state tiles
    static constexpr int kHs = kTH / BaseShape::kTileSize;
    using RegAcc = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kAMs, kBNs>>;
    using RegState = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kAMs, kHs>>;
    using RegHout = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAMs, kHs>>;

    using GlobalState = GlobalTile<AccType, tl::RowMajor<kTM, kTH, kH>>;
    using GlobalHout = GlobalTile<InType, tl::RowMajor<kTM, kTH, kH>>;
    using StateLoader = GlobalToRegLoader<RegState, WarpLayout, WarpReuse::kCont>;
    using StateStorer = RegToGlobalStorer<GlobalState, RegState, WarpLayout>;
    using HoutStorer = RegToGlobalStorer<GlobalHout, RegHout, WarpLayout>;

    static constexpr int kShmBytes = (kTM * kTK + kTK * kTG) * sizeof(InType);
};

namespace detail {
DEVICE float sigmoid_f32(float x) { return 1.0f / (1.0f + __expf(-x)); }
DEVICE float tanh_f32(float x) {
    // tanh(x) = 1 - 2 / (exp(2x) + 1); exact limits at +-inf, no cancellation blow-up near 0 beyond 1 ulp of 1
    const float e = __expf(2.0f * x);
    return 1.0f - 2.0f / (e + 1.0f);
}
}  // namespace detail

/// grid = (B / kTM, H / kTH), block = Traits::kThreads, dynamic LDS = Traits::kShmBytes.
/// x_t [B, I], h_in [B, H] f16 (nullptr = zeros); W [4H, I+H], bias [4H] f16; c_in (nullptr = zeros) / c_out [B, H] f32 (may alias);
/// h_out [B, H] f16 (must not alias h_in: other workgroups still read h_in).
template <typename InType, typename Traits>
__global__ void __launch_bounds__(Traits::kThreads)
    lstm_cell(const InType* x_t, const InType* h_in, const InType* W, const InType* bias, const float* c_in,
              float* c_out, InType* h_out) {
    constexpr int kI = Traits::kI, kH = Traits::kH, kKK = Traits::kKK;
    constexpr int kTM = Traits::kTM, kTH = Traits::kTH, kTK = Traits::kTK;

    const int row0 = blockIdx.x * kTM;  // first batch row
    const int hid0 = blockIdx.y * kTH;  // first hidden unit

    extern __shared__ __align__(16) unsigned char buf[];
    InType* sA_ptr = reinterpret_cast<InType*>(buf);
    InType* sW_ptr = sA_ptr + Traits::SharedA::kNumel;

    typename Traits::SharedA sA(sA_ptr);
    typename Traits::SharedW sW(sW_ptr);
    typename Traits::SIteratorW sWs(sW_ptr);
    typename Traits::RegA rA;
    typename Traits::RegB rB;
    typename Traits::RegAcc acc;

    typename Traits::G2SLoaderA g2s_a;
    typename Traits::G2SLoaderW g2s_w;
    typename Traits::S2RLoaderA s2r_a;
    typename Traits::S2RLoaderB s2r_b;

    // h_in == nullptr means h_{t-1} = 0: its half of the reduction contributes nothing
    const int k_end = h_in ? kKK : kI;
    for (int k0 = 0; k0 < k_end; k0 += kTK) {
        if (k0 < kI) {
            typename Traits::GlobalX gX(x_t + size_t(row0) * kI + k0);
            g2s_a(gX, sA);
        } else {
            typename Traits::GlobalHin gH(h_in + size_t(row0) * kH + (k0 - kI));
            g2s_a(gH, sA);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            typename Traits::GlobalW gW(W + (size_t(g) * kH + hid0) * kKK + k0);
            auto sWg = sWs(g);
            g2s_w(gW, sWg);
        }
        __copy_async();
        __syncthreads();

        s2r_a(sA, rA);
        s2r_b(sW, rB);
        compute::gemm(rA, rB, acc);
        __syncthreads();
    }

    // cell update in registers
    typename Traits::RegState c;
    typename Traits::RegHout h;
    if (c_in) {  // c_in == nullptr means c_{t-1} = 0 (RegTile starts zeroed)
        typename Traits::GlobalState gCin(const_cast<float*>(c_in) + size_t(row0) * kH + hid0);
        typename Traits::StateLoader load_c;
        load_c(gCin, c);
    }

    const int col_in_tile = traits::lane_minor();
#pragma unroll
    for (int i = 0; i < Traits::kAMs; ++i) {
#pragma unroll
        for (int j = 0; j < Traits::kHs; ++j) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int hid = hid0 + j * 16 + col_in_tile + e;
                const float gi = acc(i, 0 * Traits::kHs + j)(0, e) + __half2float(bias[0 * kH + hid]);
                const float gf = acc(i, 1 * Traits::kHs + j)(0, e) + __half2float(bias[1 * kH + hid]);
                const float gg = acc(i, 2 * Traits::kHs + j)(0, e) + __half2float(bias[2 * kH + hid]);
                const float go = acc(i, 3 * Traits::kHs + j)(0, e) + __half2float(bias[3 * kH + hid]);
                const float cn =
                    detail::sigmoid_f32(gf) * c(i, j)(0, e) + detail::sigmoid_f32(gi) * detail::tanh_f32(gg);
                c(i, j)(0, e) = cn;
                h(i, j)(0, e) = __float2half(detail::sigmoid_f32(go) * detail::tanh_f32(cn));
            }
        }
    }

    typename Traits::GlobalState gCout(c_out + size_t(row0) * kH + hid0);
    typename Traits::StateStorer store_c;
    store_c(c, gCout);

    typename Traits::GlobalHout gHout(h_out + size_t(row0) * kH + hid0);
    typename Traits::HoutStorer store_h;
    store_h(h, gHout);
}

}  // namespace tiledcuda::kernels
