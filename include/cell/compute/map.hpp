// Element-wise maps over register tiles. Same template names as the reference's
// include/cell/compute/map.hpp:84-133: BaseTileX applies a scalar functor to a tile of
// scalars, RegTileX applies BaseTileX to every BaseTile of a tile of BaseTiles.
#pragma once

#include "cell/compute/math_functor.hpp"
#include "types/layout.hpp"

namespace tiledcuda::cell::compute {

namespace tl = tile_layout;

namespace detail {

template <typename RegTile, typename Functor>
struct ElementWise {
    DEVICE void operator()(const RegTile& src, RegTile& dst) {
        Functor f;
#pragma unroll
        for (int i = 0; i < RegTile::kRows; ++i) {
#pragma unroll
            for (int j = 0; j < RegTile::kCols; ++j) f(src(i, j), dst(i, j));
        }
    }
};

template <typename SrcRegTile, typename DstRegTile, typename Functor>
struct ElementWise2 {
    static_assert(SrcRegTile::kRows == DstRegTile::kRows, "kRows must be equal");
    static_assert(SrcRegTile::kCols == DstRegTile::kCols, "kCols must be equal");

    DEVICE void operator()(const SrcRegTile& src, DstRegTile& dst) {
        Functor f;
#pragma unroll
        for (int i = 0; i < SrcRegTile::kRows; ++i) {
#pragma unroll
            for (int j = 0; j < SrcRegTile::kCols; ++j) f(src(i, j), dst(i, j));
        }
    }
};

template <typename RegTile, typename Functor>
struct Binary {
    DEVICE void operator()(const RegTile& lhs, const RegTile& rhs, RegTile& dst) {
        Functor f;
#pragma unroll
        for (int i = 0; i < RegTile::kRows; ++i) {
#pragma unroll
            for (int j = 0; j < RegTile::kCols; ++j) f(lhs(i, j), rhs(i, j), dst(i, j));
        }
    }
};

}  // namespace detail

#define TCU_UNARY_TILE_OP(Name)                                                             \
    template <typename RegTile>                                                              \
    using BaseTile##Name = detail::ElementWise<RegTile, Name<typename RegTile::DType>>;      \
    template <typename RegTile>                                                              \
    using RegTile##Name = detail::ElementWise<RegTile, BaseTile##Name<typename RegTile::DType>>

TCU_UNARY_TILE_OP(Exp);
TCU_UNARY_TILE_OP(Log);
TCU_UNARY_TILE_OP(Relu);
#undef TCU_UNARY_TILE_OP

#define TCU_BINARY_TILE_OP(Name)                                                          \
    template <typename RegTile>                                                            \
    using BaseTile##Name = detail::Binary<RegTile, Name<typename RegTile::DType>>;         \
    template <typename RegTile>                                                            \
    using RegTile##Name = detail::Binary<RegTile, BaseTile##Name<typename RegTile::DType>>

TCU_BINARY_TILE_OP(Add);
TCU_BINARY_TILE_OP(Sub);
TCU_BINARY_TILE_OP(Mul);
TCU_BINARY_TILE_OP(Div);
TCU_BINARY_TILE_OP(Max);
TCU_BINARY_TILE_OP(Min);
#undef TCU_BINARY_TILE_OP

template <typename SrcRegTile, typename DstRegTile>
using BaseTileConvert =
    detail::ElementWise2<SrcRegTile, DstRegTile, Convert<typename SrcRegTile::DType, typename DstRegTile::DType>>;
template <typename SrcRegTile, typename DstRegTile>
using RegTileConvert = detail::ElementWise2<SrcRegTile, DstRegTile,
                                            BaseTileConvert<typename SrcRegTile::DType, typename DstRegTile::DType>>;

}  // namespace tiledcuda::cell::compute
