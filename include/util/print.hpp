// Scalar tile printers (device printf); the role of the reference's util/print.hpp:15-65. The printers that show a
// register tile in matrix order (the reference's RegTilePrinter / RegVecPrinter, :67-175) are in util/tile_print.hpp.
#pragma once

#include "config.hpp"

#include <cstdio>

namespace tiledcuda::cell {

DEVICE float print_cast(float v) { return v; }
DEVICE float print_cast(__half v) { return __half2float(v); }
DEVICE float print_cast(_Float16 v) { return static_cast<float>(v); }

/// Print a tile of scalars element by element through its layout.
template <typename DType, typename Layout>
DEVICE void print_tile(const DType* data, const Layout& layout) {
    for (int i = 0; i < Layout::kRows; ++i) {
        for (int j = 0; j < Layout::kCols; ++j) printf("%.3f, ", print_cast(data[layout(i, j)]));
        printf("\n");
    }
}

}  // namespace tiledcuda::cell
