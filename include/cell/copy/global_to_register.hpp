// Global memory <-> register tiles, in BaseTile lane order.
// Same functors as the reference's include/cell/copy/global_to_register.hpp:309-379
// (GlobalToRegLoader<Reg, WarpLayout, WarpReuse>, RegToGlobalStorer<Global, Reg, WarpLayout>).
// Where the reference issues eight 2-byte accesses per lane per BaseTile in mma.sync
// fragment order (:34-43), a lane here moves its 4 contiguous elements with one 64-bit
// (f16) or 128-bit (f32) access when the BaseTile orientation matches the memory layout.
#pragma once

#include "cell/copy/constants.hpp"
#include "cell/copy/vec.hpp"
#include "cell/copy/warp.hpp"
#include "types/mod.hpp"

namespace tiledcuda::cell::copy {

using namespace traits;
namespace tl = tile_layout;

namespace detail {

/// Moves the share of one lane of one BaseTile whose top-left element sits at `tile_ptr`
/// (pitched by kRowStride / kColStride). kLoad: memory -> registers, else registers -> memory.
template <typename DType, typename BaseTile, const int kRowStride, const int kColStride, const bool kLoad>
DEVICE void move_base_tile(DType* tile_ptr, BaseTile& reg) {
    constexpr bool kRegRowMajor = BaseTile::kType == tl::Layout::kRowMajor;
    // (row, col) of the first of the lane's 4 elements and the direction they run in
    const int row = kRegRowMajor ? lane_major() : lane_minor();
    const int col = kRegRowMajor ? lane_minor() : lane_major();
    constexpr int kStep = kRegRowMajor ? kColStride : kRowStride;

    DType* p = tile_ptr + row * kRowStride + col * kColStride;
    if constexpr (kStep == 1 && (kRegRowMajor ? kRowStride : kColStride) % 4 == 0) {
        if constexpr (kLoad)
            vec_load<4>(p, reg.mutable_data());
        else
            vec_store<4>(reg.data(), p);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (kLoad)
                reg.mutable_data()[e] = p[e * kStep];
            else
                p[e * kStep] = reg.data()[e];
        }
    }
}

/// The same for any tile described by TileGeometry (16 x 16 BaseTile or MFMA-shaped tile): every run of the lane
/// moves as one vector access when it lies along the contiguous dimension of the memory tile.
template <typename DType, typename BaseTile, const int kRowStride, const int kColStride, const bool kLoad>
DEVICE void move_tile(DType* tile_ptr, BaseTile& reg) {
    using G = TileGeometry<std::remove_const_t<BaseTile>>;
    using E = std::remove_const_t<DType>;
    const int lane = lane_id();
    const int major = lane % G::kLaneMajor;
    const int minor0 = (lane / G::kLaneMajor) * G::kRunLen;
    constexpr int kStep = G::kRowMajor ? kColStride : kRowStride;
    constexpr int kLinePitch = G::kRowMajor ? kRowStride : kColStride;
    constexpr int kPiece = G::kRunLen * sizeof(E) > 16 ? int(16 / sizeof(E)) : G::kRunLen;
    auto* r = const_cast<E*>(reg.data());
#pragma unroll
    for (int run = 0; run < G::kRuns; ++run) {
        const int minor = minor0 + run * G::kRunStride;
        DType* p = tile_ptr + (G::kRowMajor ? major * kRowStride + minor * kColStride
                                            : minor * kRowStride + major * kColStride);
        if constexpr (kStep == 1 && kLinePitch % kPiece == 0) {
#pragma unroll
            for (int e = 0; e < G::kRunLen; e += kPiece) {
                if constexpr (kLoad)
                    vec_load<kPiece>(p + e, r + run * G::kRunLen + e);
                else
                    vec_store<kPiece>(r + run * G::kRunLen + e, const_cast<E*>(p) + e);
            }
        } else {
#pragma unroll
            for (int e = 0; e < G::kRunLen; ++e) {
                if constexpr (kLoad)
                    r[run * G::kRunLen + e] = p[e * kStep];
                else
                    const_cast<E*>(p)[e * kStep] = r[run * G::kRunLen + e];
            }
        }
    }
}

}  // namespace detail

/// Load this wavefront's share of a global tile into a register tile.
template <typename Reg_, typename WarpLayout_, const WarpReuse kMode_,
          typename Base = warp::CopyBase<WarpLayout_, kMode_>>
struct GlobalToRegLoader : public Base {
    using Reg = Reg_;
    using BaseTile = typename Reg::DType;
    using DType = typename BaseTile::DType;
    using BaseShape = TileExtent<BaseTile>;

    using WarpLayout = WarpLayout_;
    static constexpr WarpReuse kMode = kMode_;

    template <typename Global>
    DEVICE void operator()(const Global& src, Reg& dst) {
        static constexpr int kRowExec = Base::template row_exec_count<BaseShape, Global::kRows>();
        static constexpr int kColExec = Base::template col_exec_count<BaseShape, Global::kCols>();
        static_assert(kRowExec == Reg::kRows && kColExec == Reg::kCols,
                      "the register tile must hold exactly this wavefront's share of the global tile");

        const DType* warp_ptr = src.data() + Base::template get_warp_offset<Global>();
#pragma unroll
        for (int i = 0; i < kRowExec; ++i) {
#pragma unroll
            for (int j = 0; j < kColExec; ++j) {
                const DType* tile_ptr = warp_ptr + i * BaseShape::kRows * Global::kRowStride +
                                        j * BaseShape::kCols * Global::kColStride;
                detail::move_tile<const DType, BaseTile, Global::kRowStride, Global::kColStride, true>(
                    tile_ptr, dst(i, j));
            }
        }
    }
};

/// Store a register tile into this wavefront's share of a global tile.
template <typename Global_, typename Reg_, typename WarpLayout_,
          typename Base = warp::CopyBase<WarpLayout_, WarpReuse::kCont>>
struct RegToGlobalStorer : public Base {
    using Global = Global_;
    using Reg = Reg_;
    using BaseTile = typename Reg::DType;
    using DType = typename Global::DType;
    using BaseShape = TileExtent<BaseTile>;

    using WarpLayout = WarpLayout_;

    static_assert(std::is_same_v<typename BaseTile::DType, DType>,
                  "the register tile and the global tile must hold the same element type");

    DEVICE void operator()(const Reg& src, Global& dst) {
        static constexpr int kRowExec = Base::template row_exec_count<BaseShape, Global::kRows>();
        static constexpr int kColExec = Base::template col_exec_count<BaseShape, Global::kCols>();
        static_assert(kRowExec == Reg::kRows && kColExec == Reg::kCols,
                      "the register tile must hold exactly this wavefront's share of the global tile");

        DType* warp_ptr = dst.mutable_data() + Base::template get_warp_offset<Global>();
#pragma unroll
        for (int i = 0; i < kRowExec; ++i) {
#pragma unroll
            for (int j = 0; j < kColExec; ++j) {
                DType* tile_ptr = warp_ptr + i * BaseShape::kRows * Global::kRowStride +
                                  j * BaseShape::kCols * Global::kColStride;
                detail::move_tile<DType, const BaseTile, Global::kRowStride, Global::kColStride, false>(
                    tile_ptr, src(i, j));
            }
        }
    }
};

}  // namespace tiledcuda::cell::copy
