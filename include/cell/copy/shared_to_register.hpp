// LDS <-> register tile copies in BaseTile lane order.
// Same functors as the reference's include/cell/copy/shared_to_register.hpp:194-301
// (SharedToRegLoader<Reg, WarpLayout, WarpReuse>, RegToSharedStorer<Reg, WarpLayout>).
// The reference reads with ldmatrix.x4 (copy_atom.hpp:55-64) and scatters mma C-fragments
// in 2-element segments (:71-288); here a lane reads or writes its 4 contiguous elements of
// each BaseTile with one ds_read_b64 / ds_write_b64 (f16) or b128 (f32). Addresses are taken
// from logical coordinates of the (possibly swizzled, possibly sub-) shared tile.
#pragma once

#include "cell/copy/constants.hpp"
#include "cell/copy/vec.hpp"
#include "cell/copy/warp.hpp"
#include "types/mod.hpp"

namespace tiledcuda::cell::copy {

using namespace traits;
namespace tl = tile_layout;

namespace detail {

/// Move one lane's share of the BaseTile whose top-left element is (row0, col0) of `tile`.
template <typename Shared, typename BaseTile, const bool kLoad>
DEVICE void move_shared_base_tile(Shared& tile, int row0, int col0, BaseTile& reg) {
    using DType = typename Shared::DType;
    constexpr bool kRegRowMajor = BaseTile::kType == tl::Layout::kRowMajor;
    const int row = row0 + (kRegRowMajor ? lane_major() : lane_minor());
    const int col = col0 + (kRegRowMajor ? lane_minor() : lane_major());
    auto* base = const_cast<DType*>(tile.data());

    if constexpr (kRegRowMajor == Shared::kIsRowMajor) {
        // the lane's 4 elements are one contiguous chunk of a line
        DType* p = base + tile.offset(row, col);
        if constexpr (kLoad)
            vec_load<4>(p, reg.mutable_data());
        else
            vec_store<4>(reg.data(), p);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            DType* p = base + (kRegRowMajor ? tile.offset(row, col + e) : tile.offset(row + e, col));
            if constexpr (kLoad)
                reg.mutable_data()[e] = *p;
            else
                *p = reg.data()[e];
        }
    }
}

}  // namespace detail

/// Load this wavefront's share of a shared tile into a register tile.
template <typename Reg_, typename WarpLayout_, const WarpReuse kMode_,
          typename Base = warp::CopyBase<WarpLayout_, kMode_>>
struct SharedToRegLoader : public Base {
    using Reg = Reg_;
    using BaseTile = typename Reg::DType;
    using DType = typename BaseTile::DType;
    using BaseShape = BaseTileShape<DType>;

    using WarpLayout = WarpLayout_;
    static constexpr WarpReuse kMode = kMode_;

    template <typename Shared>
    DEVICE void operator()(const Shared& src, Reg& dst) {
        static_assert(std::is_same_v<typename Shared::DType, DType>,
                      "The data type of Shared and Reg must be the same.");
        static constexpr int kRowExec = Base::template row_exec_count<BaseShape, Shared::kRows>();
        static constexpr int kColExec = Base::template col_exec_count<BaseShape, Shared::kCols>();
        static_assert(kRowExec == Reg::kRows && kColExec == Reg::kCols,
                      "the register tile must hold exactly this wavefront's share of the shared tile");

        const int row0 = Base::template warp_row0<Shared::kRows>();
        const int col0 = Base::template warp_col0<Shared::kCols>();
#pragma unroll
        for (int i = 0; i < kRowExec; ++i) {
#pragma unroll
            for (int j = 0; j < kColExec; ++j) {
                detail::move_shared_base_tile<const Shared, BaseTile, true>(src, row0 + i * BaseShape::kRows,
                                                                            col0 + j * BaseShape::kCols, dst(i, j));
            }
        }
    }
};

/// Store a register tile into this wavefront's share of a shared tile (even split).
template <typename Reg_, typename WarpLayout_>
struct RegToSharedStorer : public warp::CopyBase<WarpLayout_, WarpReuse::kCont> {
    using Base = warp::CopyBase<WarpLayout_, WarpReuse::kCont>;
    using Reg = Reg_;
    using BaseTile = typename Reg::DType;
    using DType = typename BaseTile::DType;
    using BaseShape = BaseTileShape<DType>;
    using WarpLayout = WarpLayout_;

    template <typename Shared>
    DEVICE void operator()(const Reg& src, Shared& dst) {
        static_assert(std::is_same_v<typename Shared::DType, DType>,
                      "The element data type of Shared and Register tile must be the same.");
        static_assert((Reg::kNumel * BaseTile::kNumel * kWaveSize * tl::get_numel<WarpLayout>) == Shared::kNumel,
                      "The number of elements held in the register files of all lanes of the workgroup "
                      "must equal the number held in the shared memory tile.");
        static constexpr int kRowExec = Base::template row_exec_count<BaseShape, Shared::kRows>();
        static constexpr int kColExec = Base::template col_exec_count<BaseShape, Shared::kCols>();
        static_assert(kRowExec == Reg::kRows && kColExec == Reg::kCols,
                      "the register tile must hold exactly this wavefront's share of the shared tile");

        const int row0 = Base::template warp_row0<Shared::kRows>();
        const int col0 = Base::template warp_col0<Shared::kCols>();
#pragma unroll
        for (int i = 0; i < kRowExec; ++i) {
#pragma unroll
            for (int j = 0; j < kColExec; ++j) {
                detail::move_shared_base_tile<Shared, const BaseTile, false>(dst, row0 + i * BaseShape::kRows,
                                                                             col0 + j * BaseShape::kCols, src(i, j));
            }
        }
    }
};

}  // namespace tiledcuda::cell::copy
