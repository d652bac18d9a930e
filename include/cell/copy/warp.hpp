// Which part of a tile each wavefront of a workgroup owns, per WarpReuse mode.
// Same role as the reference's include/cell/copy/warp.hpp:47-203 (CopyBase: warp offset and
// execution counts; warp_row_id / warp_col_id), expressed in logical (row, col) coordinates
// so that it serves global, shared and swizzled tiles alike.
#pragma once

#include "cell/copy/constants.hpp"
#include "cell/traits/base.hpp"
#include "types/layout.hpp"

namespace tiledcuda::cell::copy::warp {

namespace tl = tile_layout;
using namespace tiledcuda::cell::traits;

template <typename WarpLayout_, const WarpReuse kMode_>
struct CopyBase {
    static constexpr WarpReuse kMode = kMode_;
    using WarpLayout = WarpLayout_;

    static_assert(kMode == WarpReuse::kCont || kMode == WarpReuse::kRowReuseCont ||
                      kMode == WarpReuse::kColReuseCont,
                  "Only the three `Cont` reuse modes are implemented.");

    static constexpr int kWarpsPerRow = tl::num_rows<WarpLayout>;  // wavefronts along the rows
    static constexpr int kWarpsPerCol = tl::num_cols<WarpLayout>;  // wavefronts along the columns
    static constexpr bool kRowsShared = kMode == WarpReuse::kColReuseCont;  // every wavefront-row loads all rows
    static constexpr bool kColsShared = kMode == WarpReuse::kRowReuseCont;

    /// Row of this wavefront in the wavefront layout.
    DEVICE static int warp_row_id() {
        const int wid = wave_id();
        if constexpr (tl::layout_type<WarpLayout> == tl::Layout::kRowMajor)
            return wid / kWarpsPerCol;
        else
            return wid % kWarpsPerRow;
    }

    /// Column of this wavefront in the wavefront layout.
    DEVICE static int warp_col_id() {
        const int wid = wave_id();
        if constexpr (tl::layout_type<WarpLayout> == tl::Layout::kRowMajor)
            return wid % kWarpsPerCol;
        else
            return wid / kWarpsPerRow;
    }

    /// Rows / columns of a kRows x kCols tile handled by one wavefront.
    template <const int kRows>
    static constexpr int rows_per_warp() {
        static_assert(kRows % (kRowsShared ? 1 : kWarpsPerRow) == 0, "rows must divide over the wavefront rows");
        return kRowsShared ? kRows : kRows / kWarpsPerRow;
    }
    template <const int kCols>
    static constexpr int cols_per_warp() {
        static_assert(kCols % (kColsShared ? 1 : kWarpsPerCol) == 0, "cols must divide over the wavefront columns");
        return kColsShared ? kCols : kCols / kWarpsPerCol;
    }

    /// First row / column of this wavefront's share of the tile.
    template <const int kRows>
    DEVICE static int warp_row0() {
        if constexpr (kRowsShared) return 0; else return warp_row_id() * rows_per_warp<kRows>();
    }
    template <const int kCols>
    DEVICE static int warp_col0() {
        if constexpr (kColsShared) return 0; else return warp_col_id() * cols_per_warp<kCols>();
    }

    /// Number of BaseTiles this wavefront handles along the rows / columns.
    template <typename BaseTile, const int kRows>
    static constexpr int row_exec_count() {
        static_assert(rows_per_warp<kRows>() % BaseTile::kRows == 0 && rows_per_warp<kRows>() >= BaseTile::kRows,
                      "each wavefront must own a whole number (>= 1) of BaseTile rows");
        return rows_per_warp<kRows>() / BaseTile::kRows;
    }
    template <typename BaseTile, const int kCols>
    static constexpr int col_exec_count() {
        static_assert(cols_per_warp<kCols>() % BaseTile::kCols == 0 && cols_per_warp<kCols>() >= BaseTile::kCols,
                      "each wavefront must own a whole number (>= 1) of BaseTile columns");
        return cols_per_warp<kCols>() / BaseTile::kCols;
    }

    /// Element offset of this wavefront's share inside a pitched (global) tile.
    template <typename Tile>
    DEVICE static int get_warp_offset() {
        return warp_row0<Tile::kRows>() * Tile::kRowStride + warp_col0<Tile::kCols>() * Tile::kColStride;
    }
};

}  // namespace tiledcuda::cell::copy::warp
