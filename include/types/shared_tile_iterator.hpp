// Chunk a shared (LDS) tile into sub-tiles. Same surface as the reference's
// include/types/shared_tile_iterator.hpp:31-129 (1-D index when one strip count is 1); the
// 2-D index and `_` slices, which the reference leaves as assert(false), are implemented.
// A sub-tile is a view (base pointer + origin) into the parent's pitched allocation.
#pragma once

#include "cell/traits/base.hpp"
#include "types/shared.hpp"
#include "types/tile_shape.hpp"

#include <ostream>

namespace tiledcuda::cell {
namespace tl = tile_layout;

template <class Tile_, class ChunkShape_>
class STileIterator {
  public:
    using Tile = Tile_;
    using DType = typename Tile::DType;
    using ChunkShape = ChunkShape_;
    using BaseShape = traits::BaseTileShape<DType>;

    static_assert(Tile::kRows >= dim_size<0, ChunkShape>, "Tile::kRows must be >= dim_size<0, ChunkShape>");
    static_assert(Tile::kCols >= dim_size<1, ChunkShape>, "Tile::kCols must be >= dim_size<1, ChunkShape>");

    static constexpr int kChunkRow = dim_size<0, ChunkShape>;
    static constexpr int kChunkCol = dim_size<1, ChunkShape>;

    static constexpr int sc0 = Tile::kRows / kChunkRow;
    static constexpr int sc1 = Tile::kCols / kChunkCol;

    HOST_DEVICE STileIterator() : data_(nullptr), line0_(0), elem0_(0) {}

    HOST_DEVICE STileIterator(DType* data) : data_(data), line0_(0), elem0_(0) {}

    HOST_DEVICE STileIterator(const DType* data) : data_(const_cast<DType*>(data)), line0_(0), elem0_(0) {}

    HOST_DEVICE STileIterator(DType* base, int line0, int elem0) : data_(base), line0_(line0), elem0_(elem0) {}

    HOST_DEVICE auto operator()(int i) const {
        static_assert(sc0 == 1 || sc1 == 1,
                      "A single index is supported only when the strip count of one of the iterator's "
                      "dimensions is 1.");
        return sc0 == 1 ? (*this)(0, i) : (*this)(i, 0);
    }

    HOST_DEVICE auto operator()(int x, int y) const {
        using SubLayout = tl::MatrixLayout<kChunkRow, kChunkCol, Tile::kRowStride, Tile::kColStride>;
        using NewTile = SharedTile<DType, SubLayout, Tile::kSwizzled, typename Tile::SwizzlePolicy>;
        const int row = x * kChunkRow, col = y * kChunkCol;
        return Tile::kIsRowMajor ? NewTile(data_, line0_ + row, elem0_ + col)
                                 : NewTile(data_, line0_ + col, elem0_ + row);
    }

    HOST_DEVICE auto operator()(int x, const Underscore&) const {
        using SubLayout = tl::MatrixLayout<kChunkRow, Tile::kCols, Tile::kRowStride, Tile::kColStride>;
        using Iter = STileIterator<SharedTile<DType, SubLayout, Tile::kSwizzled, typename Tile::SwizzlePolicy>, ChunkShape>;
        const int row = x * kChunkRow;
        return Tile::kIsRowMajor ? Iter(data_, line0_ + row, elem0_) : Iter(data_, line0_, elem0_ + row);
    }

    HOST_DEVICE auto operator()(const Underscore&, int y) const {
        using SubLayout = tl::MatrixLayout<Tile::kRows, kChunkCol, Tile::kRowStride, Tile::kColStride>;
        using Iter = STileIterator<SharedTile<DType, SubLayout, Tile::kSwizzled, typename Tile::SwizzlePolicy>, ChunkShape>;
        const int col = y * kChunkCol;
        return Tile::kIsRowMajor ? Iter(data_, line0_, elem0_ + col) : Iter(data_, line0_ + col, elem0_);
    }

    HOST_DEVICE auto to_tile() const { return Tile(data_, line0_, elem0_); }

  private:
    DType* data_;
    int line0_;
    int elem0_;
};

template <typename Tile, typename ChunkShape>
static HOST std::ostream& operator<<(std::ostream& out, const STileIterator<Tile, ChunkShape>&) {
    using It = STileIterator<Tile, ChunkShape>;
    out << "numel = " << Tile::kNumel << ", ChunkShape[" << It::kChunkRow << ", " << It::kChunkCol
        << "], sc0 = " << It::sc0 << ", sc1 = " << It::sc1;
    return out;
}

}  // namespace tiledcuda::cell
