// Chunk a global tile into sub-tiles. Same surface as the reference's
// include/types/global_tile_iterator.hpp:29-152 (sc0/sc1 strip counts; 1-D index when one
// strip count is 1, 2-D index, `_` slicing). Offsets are always taken from the parent's
// strides, i.e. from logical (row, col) coordinates.
#pragma once

#include "types/global.hpp"
#include "types/tile_shape.hpp"

#include <cassert>
#include <ostream>

namespace tiledcuda::cell {
namespace tl = tile_layout;

template <class Tile_, class ChunkShape_>
class GTileIterator {
  public:
    using Tile = Tile_;
    using DType = typename Tile::DType;
    using ChunkShape = ChunkShape_;

    static_assert(Tile::kRows >= dim_size<0, ChunkShape>, "Tile::kRows must be >= dim_size<0, ChunkShape>");
    static_assert(Tile::kCols >= dim_size<1, ChunkShape>, "Tile::kCols must be >= dim_size<1, ChunkShape>");

    static constexpr int kStride0 = dim_size<0, ChunkShape>;
    static constexpr int kStride1 = dim_size<1, ChunkShape>;

    static constexpr int sc0 = Tile::kRows / kStride0;
    static constexpr int sc1 = Tile::kCols / kStride1;

    HOST_DEVICE GTileIterator() : data_(nullptr) {}

    HOST_DEVICE GTileIterator(DType* data) : data_(data) {}

    HOST_DEVICE GTileIterator(const DType* data) : data_(const_cast<DType*>(data)) {}

    /// Sub-tile `i` along the only dimension that is actually chunked.
    HOST_DEVICE auto operator()(int i) const {
        static_assert(sc0 == 1 || sc1 == 1,
                      "A single index is supported only when the strip count of one of the iterator's "
                      "dimensions is 1.");
        return sc0 == 1 ? (*this)(0, i) : (*this)(i, 0);
    }

    /// Sub-tile at strip (x, y).
    HOST_DEVICE auto operator()(int x, int y) const {
        using SubLayout = tl::MatrixLayout<kStride0, kStride1, Tile::kRowStride, Tile::kColStride>;
        using NewTile = GlobalTile<DType, SubLayout>;
        return NewTile(data_ + origin(x * kStride0, y * kStride1));
    }

    /// Row strip x, still to be iterated along the columns.
    HOST_DEVICE auto operator()(int x, const Underscore&) const {
        using SubLayout = tl::MatrixLayout<kStride0, Tile::kCols, Tile::kRowStride, Tile::kColStride>;
        using Iter = GTileIterator<GlobalTile<DType, SubLayout>, ChunkShape>;
        static_assert(Iter::sc0 == 1);
        return Iter(data_ + origin(x * kStride0, 0));
    }

    /// Column strip y, still to be iterated along the rows.
    HOST_DEVICE auto operator()(const Underscore&, int y) const {
        using SubLayout = tl::MatrixLayout<Tile::kRows, kStride1, Tile::kRowStride, Tile::kColStride>;
        using Iter = GTileIterator<GlobalTile<DType, SubLayout>, ChunkShape>;
        static_assert(Iter::sc1 == 1);
        return Iter(data_ + origin(0, y * kStride1));
    }

    HOST_DEVICE auto to_tile() const { return Tile(data_); }

  private:
    HOST_DEVICE static constexpr int origin(int row, int col) {
        return row * Tile::kRowStride + col * Tile::kColStride;
    }

    DType* data_;
};

/// Host-only pretty printer of the iterator's static shape.
template <typename Tile, typename ChunkShape>
static HOST std::ostream& operator<<(std::ostream& out, const GTileIterator<Tile, ChunkShape>&) {
    using It = GTileIterator<Tile, ChunkShape>;
    out << "numel = " << Tile::kNumel << ", ChunkShape[" << It::kStride0 << ", " << It::kStride1
        << "], sc0 = " << It::sc0 << ", sc1 = " << It::sc1;
    return out;
}

}  // namespace tiledcuda::cell
