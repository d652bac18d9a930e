// Printers that show a register tile as the matrix it stands for. The role of the reference's RegTilePrinter /
// RegVecPrinter (include/util/print.hpp:67-175), which walk the mma.sync fragment order of a 32-lane warp, lanes
// printing in turn. Device printf gives no ordering between lanes, so here the wavefront gathers each element from
// the lane that owns it (one cross-lane read per element, taken from TileGeometry, so 16 x 16 BaseTiles and
// MFMA-shaped tiles print alike) and lane 0 prints the rows in order. All 64 lanes of the wavefront must call the
// printer (it shuffles); `tid` is the thread index, as in the reference, and only the wavefront with tid / 64 == 0
// prints unless kAllWaves is set.
#pragma once

#include "types/mfma_tile.hpp"
#include "types/register.hpp"
#include "util/print.hpp"

namespace tiledcuda::cell {
namespace tl = tile_layout;

/// Value of element (row, col) of a BaseTile spread over the wavefront, delivered to every lane.
template <typename BaseTile>
DEVICE float gather_tile_element(const BaseTile& tile, int row, int col) {
    using G = traits::TileGeometry<BaseTile>;
    const int major = G::kRowMajor ? row : col;
    const int minor = G::kRowMajor ? col : row;
    const int owner = major + G::kLaneMajor * ((minor % G::kRunStride) / G::kRunLen);
    const int index = (minor / G::kRunStride) * G::kRunLen + minor % G::kRunLen;
    float mine = 0.f;
#pragma unroll
    for (int e = 0; e < G::kRuns * G::kRunLen; ++e)
        if (e == index) mine = print_cast(tile.data()[e]);
    return __shfl(mine, owner, kWaveSize);
}

/// Print a register tile of BaseTiles (any orientation) in matrix order. kLayout is kept for source compatibility
/// with the reference's RegTilePrinter<RegTile, kLayout>; the orientation is read from the tile itself.
template <typename RegTile, const tl::Layout kLayout = RegTile::kType, const bool kAllWaves = false>
struct RegTilePrinter {
    using BaseTile = typename RegTile::DType;
    using G = traits::TileGeometry<BaseTile>;
    static constexpr int kRows = RegTile::kRows, kCols = RegTile::kCols;

    DEVICE void operator()(const RegTile& tile, int tid) {
        const bool printing = (tid % kWaveSize) == 0 && (kAllWaves || tid / kWaveSize == 0);
        for (int i = 0; i < kRows; ++i) {
            for (int r = 0; r < G::kRows; ++r) {
                for (int j = 0; j < kCols; ++j) {
                    for (int c = 0; c < G::kCols; ++c) {
                        const float v = gather_tile_element(tile(i, j), r, c);
                        if (printing) printf("%.3f, ", v);
                    }
                }
                if (printing) printf("\n");
            }
        }
        if (printing) printf("\n");
    }
};

/// Print a per-line vector as the reductions produce it (RegTile<Element, RowMajor<kRows, 1>> for row-wise results:
/// one value per BaseTile line per lane, every lane group holding a copy): the 16 values of each BaseTile, in order.
template <typename RegTile, const bool kAllWaves = false>
struct RegVecPrinter {
    static constexpr int kLines = RegTile::kNumel;

    DEVICE void operator()(const RegTile& tile, int tid) {
        const bool printing = (tid % kWaveSize) == 0 && (kAllWaves || tid / kWaveSize == 0);
        for (int i = 0; i < kLines; ++i) {
            for (int r = 0; r < 16; ++r) {
                const float v = __shfl(print_cast(tile.data()[i]), r, kWaveSize);
                if (printing) printf("%.3f, ", v);
            }
        }
        if (printing) printf("\n\n");
    }
};

}  // namespace tiledcuda::cell
