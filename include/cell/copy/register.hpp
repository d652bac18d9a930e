// Register-to-register copies; same functors as the reference's
// include/cell/copy/register.hpp:33-38.
#pragma once

#include "config.hpp"

namespace tiledcuda::cell::copy {

namespace detail {
template <typename Element>
struct DataCopy {
    DEVICE void operator()(const Element& src, Element& dst) { dst = src; }
};

template <typename RegTile, typename Copy>
struct RegCopy {
    DEVICE void operator()(const RegTile& src, RegTile& dst) {
        Copy c;
#pragma unroll
        for (int i = 0; i < RegTile::kRows; ++i) {
#pragma unroll
            for (int j = 0; j < RegTile::kCols; ++j) c(src(i, j), dst(i, j));
        }
    }
};
}  // namespace detail

/// Copies a tile of scalars (a BaseTile, or a per-row vector).
template <typename RegTile>
using BaseTileCopy = detail::RegCopy<RegTile, detail::DataCopy<typename RegTile::DType>>;

/// Copies a tile of BaseTiles.
template <typename RegTile>
using RegTileCopy = detail::RegCopy<RegTile, BaseTileCopy<typename RegTile::DType>>;

}  // namespace tiledcuda::cell::copy
