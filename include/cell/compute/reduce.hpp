// Row / column reductions of a register tile of BaseTiles.
// Same functors as the reference's include/cell/compute/reduce.hpp:146-166
// (SumReduce / MaxReduce<RegTile, kLayout>, result written to dst(i, .)).
//
// The reference's mma fragment gives each lane two rows of a BaseTile, reduced over a quad of
// lanes with two shfl_down and one broadcast shfl (reduce.hpp:66-77), and stores them as
// dst(i, 0), dst(i, 1). In the MFMA BaseTile distribution a lane holds 4 consecutive
// elements of ONE row (row-major) or column (column-major); that line is spread over lanes
// l, l^16, l^32, l^48, so the reduction is 3 in-lane steps per BaseTile and a two-step XOR
// butterfly, after which all four lanes hold the result. The destination is therefore a
// RegTile<DType, RowMajor<kRows, 1>> (row-major) or RegTile<DType, RowMajor<1, kCols>>
// (column-major): one value per BaseTile row / column per lane.
#pragma once

#include "cell/compute/math_functor.hpp"
#include "cell/warp.hpp"
#include "types/layout.hpp"
#include "types/tile_shape.hpp"

namespace tiledcuda::cell::compute {
namespace tl = tile_layout;

namespace detail {

template <typename DType, typename Reduce>
DEVICE DType butterfly_16_32(DType v, Reduce reduce) {
    v = reduce(v, shuffle_xor(v, 16));
    v = reduce(v, shuffle_xor(v, 32));
    return v;
}

template <typename RegTile, const tl::Layout kLayout>
struct Reduce;

template <typename RegTile>
struct Reduce<RegTile, tl::Layout::kRowMajor> {
    using DType = typename RegTile::DType::DType;
    static_assert(RegTile::kType == tl::Layout::kRowMajor, "row reduction needs row-major BaseTiles");

    template <typename DstTile, typename ReduceOp>
    DEVICE void operator()(const RegTile& src, DstTile& dst, ReduceOp reduce) {
#pragma unroll
        for (int i = 0; i < RegTile::kRows; ++i) {
            DType acc = src(i, 0)(0, 0);
#pragma unroll
            for (int j = 0; j < RegTile::kCols; ++j) {
#pragma unroll
                for (int e = (j == 0 ? 1 : 0); e < 4; ++e) acc = reduce(acc, src(i, j)(0, e));
            }
            dst(i, 0) = butterfly_16_32(acc, reduce);
        }
    }
};

template <typename RegTile>
struct Reduce<RegTile, tl::Layout::kColMajor> {
    using DType = typename RegTile::DType::DType;
    static_assert(RegTile::kType == tl::Layout::kColMajor, "column reduction needs column-major BaseTiles");

    template <typename DstTile, typename ReduceOp>
    DEVICE void operator()(const RegTile& src, DstTile& dst, ReduceOp reduce) {
#pragma unroll
        for (int j = 0; j < RegTile::kCols; ++j) {
            DType acc = src(0, j)(0, 0);
#pragma unroll
            for (int i = 0; i < RegTile::kRows; ++i) {
#pragma unroll
                for (int e = (i == 0 ? 1 : 0); e < 4; ++e) acc = reduce(acc, src(i, j)(e, 0));
            }
            dst(0, j) = butterfly_16_32(acc, reduce);
        }
    }
};

}  // namespace detail

template <typename RegTile, const tl::Layout kLayout>
struct SumReduce {
    using DType = typename RegTile::DType::DType;

    template <typename DstTile>
    DEVICE void operator()(const RegTile& src, DstTile& dst) {
        detail::Reduce<RegTile, kLayout> reduce;
        reduce(src, dst, Add<DType>{});
    }
};

template <typename RegTile, const tl::Layout kLayout>
struct MaxReduce {
    using DType = typename RegTile::DType::DType;

    template <typename DstTile>
    DEVICE void operator()(const RegTile& src, DstTile& dst) {
        detail::Reduce<RegTile, kLayout> reduce;
        reduce(src, dst, Max<DType>{});
    }
};

}  // namespace tiledcuda::cell::compute
