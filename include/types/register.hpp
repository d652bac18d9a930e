// Register tiles. Same surface as the reference's include/types/register.hpp:65-126:
// a RegTile is a small array living in one lane's registers; nesting a BaseTile inside a
// RegTile gives the per-lane share of a block of 16x16 tiles held by one wavefront.
//
// What changed for gfx950: a BaseTile is 4 elements per lane (64 lanes), laid out
// RowMajor<1, 4> (row-major: 4 consecutive columns of one row) or ColMajor<4, 1>
// (column-major: 4 consecutive rows of one column) instead of the reference's
// RowMajor<2, 4> / ColMajor<4, 2> mma.sync fragments (register.hpp:108-112).
#pragma once

#include <utility>

#include "hip_utils.hpp"
#include "types/layout.hpp"
#include "util/print.hpp"

#include <ostream>

namespace tiledcuda::cell {
namespace tl = tile_layout;

namespace detail {

template <typename T>
struct IsScalar : std::bool_constant<traits::BaseType<T>> {};

template <typename DType>
constexpr int elem_rows() {
    if constexpr (IsScalar<DType>::value) return 1; else return 16;
}

HOST_DEVICE constexpr int reg_align(size_t bytes) {
    return bytes >= 16 ? 16 : (bytes >= 8 ? 8 : (bytes >= 4 ? 4 : 2));
}

/// Host-only pretty printer of a register tile's static shape.
struct RegTilePrettyPrinter {
    template <typename Tile>
    static HOST void print(std::ostream& out, const Tile&) {
        constexpr int scale = IsScalar<typename Tile::DType>::value ? 1 : 16;
        out << tl::layout_type_to_str(Tile::kType) << "[" << Tile::kRows * scale << ", " << Tile::kCols * scale
            << "]";
    }
};

}  // namespace detail

template <typename Element_, typename Layout_>
class RegTile {
  public:
    using DType = Element_;
    using Layout = Layout_;

    static constexpr int kNumel = tl::get_numel<Layout>;
    static constexpr int kRows = tl::num_rows<Layout>;
    static constexpr int kCols = tl::num_cols<Layout>;

    static constexpr bool kIsBaseTile = detail::IsScalar<DType>::value;

    // For a tile of BaseTiles the type is that of the BaseTile (so a 1x1 block still
    // reports the right orientation); for a tile of scalars it is the layout's own.
    static constexpr tl::Layout kType = [] {
        if constexpr (kIsBaseTile) return tl::layout_type<Layout>; else return DType::kType;
    }();

    /// Every element zero. The elements are initialised one by one in the member initialiser (a pack expansion), not by
    /// the loop a compiler generates for an array of class-type elements: that loop is not unrolled for large tiles,
    /// and one dynamic index is enough to keep a whole register tile in scratch memory.
    HOST_DEVICE RegTile() : RegTile(std::make_integer_sequence<int, kNumel>{}) {}

    HOST_DEVICE DType* mutable_data() { return data_; }

    HOST_DEVICE const DType* data() const { return data_; }

    HOST_DEVICE constexpr Layout layout() const { return Layout{}; }

    HOST_DEVICE DType& operator()(int x, int y) { return data_[Layout{}(x, y)]; }

    HOST_DEVICE const DType& operator()(int x, int y) const { return data_[Layout{}(x, y)]; }

    /// Zero every element.
    HOST_DEVICE void clear() {
        if constexpr (kIsBaseTile) {
#pragma unroll
            for (int i = 0; i < kNumel; ++i) data_[i] = DType(0.f);
        } else {
#pragma unroll
            for (int i = 0; i < kNumel; ++i) data_[i].clear();
        }
    }

    DEVICE void dump_value() const {
        if constexpr (kIsBaseTile) {
            print_tile(data_, Layout{});
        } else {
            for (int i = 0; i < kRows; ++i)
                for (int j = 0; j < kCols; ++j) (*this)(i, j).dump_value();
        }
    }

  private:
    template <int... kIs>
    HOST_DEVICE explicit RegTile(std::integer_sequence<int, kIs...>) : data_{zero_element<kIs>()...} {}
    template <int>
    HOST_DEVICE static DType zero_element() {
        if constexpr (kIsBaseTile) return DType(0.f); else return DType();
    }

    alignas(detail::reg_align(sizeof(DType) * kNumel)) DType data_[kNumel];
};

template <typename Element>
using BaseTileRowMajor = RegTile<Element, tl::RowMajor<1, 4>>;

template <typename Element>
using BaseTileColMajor = RegTile<Element, tl::ColMajor<4, 1>>;

/// Host-only pretty printer (prints the outer layout name and the element extents).
template <typename T, typename Layout>
static HOST std::ostream& operator<<(std::ostream& out, const RegTile<T, Layout>& tile) {
    detail::RegTilePrettyPrinter::print(out, tile);
    return out;
}

}  // namespace tiledcuda::cell
