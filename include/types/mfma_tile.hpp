// Register tiles shaped like the operands of the gfx950 matrix instructions.
//
// The reference has one BaseTile shape, 16x16, the operand of mma.sync.m16n8k16 issued twice
// (include/cell/traits/base.hpp:24-39, include/types/register.hpp:108-112). The CDNA4 matrix instructions for f16
// take operands that are not square, and the shape depends on which operand it is:
//
//   instruction                 A tile (row-major)   B tile (column-major)   C tile (row-major, f32)
//   v_mfma_f32_16x16x32_f16     16 x 32              32 x 16                 16 x 16
//   v_mfma_f32_32x32x16_f16     32 x 16              16 x 32                 32 x 32
//
// An MfmaTile is one lane's share of such a tile. Operand tiles: the lane holds ONE run of 8 consecutive elements
// along the contraction index - major index (row of A, column of B) lane % kLaneMajor, contraction indices
// 8 (lane / kLaneMajor) .. + 7 - which is one ds_read_b128 from a shared tile whose lines run along the contraction
// index, and is the distribution the instruction expects. The 16 x 16 accumulator is the ordinary row-major BaseTile
// (types/register.hpp). The 32 x 32 accumulator holds row lane % 32 and, for q = 0..3, the 4 consecutive columns
// 8 q + 4 (lane / 32) .. + 3 (what the instruction produces when the operands are passed swapped, so that the lane's
// values are consecutive along a row of C and can be stored 16 bytes at a time).
//
// RegTile<MfmaTile<...>, Layout> nests them exactly like RegTile<BaseTileRowMajor<...>, Layout>; the loaders, storers
// and gemm() read the geometry from TileGeometry<BaseTile>.
#pragma once

#include "hip_utils.hpp"
#include "types/layout.hpp"
#include "types/register.hpp"
#include "util/print.hpp"

namespace tiledcuda::cell {
namespace tl = tile_layout;

template <typename Element_, const int kTileRows_, const int kTileCols_, const tl::Layout kType_>
class MfmaTile {
  public:
    using DType = Element_;
    static constexpr int kTileRows = kTileRows_;
    static constexpr int kTileCols = kTileCols_;
    static constexpr tl::Layout kType = kType_;
    static_assert(kType == tl::Layout::kRowMajor || kType == tl::Layout::kColMajor);

    static constexpr int kNumel = kTileRows * kTileCols / kWaveSize;  // elements per lane
    // rows / cols as a RegTile of scalars would report them (one line of kNumel values)
    static constexpr int kRows = kType == tl::Layout::kRowMajor ? 1 : kNumel;
    static constexpr int kCols = kType == tl::Layout::kRowMajor ? kNumel : 1;

    HOST_DEVICE MfmaTile() { clear(); }

    HOST_DEVICE DType* mutable_data() { return data_; }
    HOST_DEVICE const DType* data() const { return data_; }

    HOST_DEVICE DType& operator()(int i) { return data_[i]; }
    HOST_DEVICE const DType& operator()(int i) const { return data_[i]; }

    HOST_DEVICE void clear() {
#pragma unroll
        for (int i = 0; i < kNumel; ++i) data_[i] = DType(0.f);
    }

    DEVICE void dump_value() const {
        for (int i = 0; i < kNumel; ++i) printf("%.3f, ", print_cast(data_[i]));
        printf("\n");
    }

  private:
    alignas(16) DType data_[kNumel];
};

/// Operands and accumulator of v_mfma_f32_16x16x32_f16.
template <typename Element>
using MfmaTileA16x32 = MfmaTile<Element, 16, 32, tl::Layout::kRowMajor>;
template <typename Element>
using MfmaTileB32x16 = MfmaTile<Element, 32, 16, tl::Layout::kColMajor>;
/// Operands and accumulator of v_mfma_f32_32x32x16_f16.
template <typename Element>
using MfmaTileA32x16 = MfmaTile<Element, 32, 16, tl::Layout::kRowMajor>;
template <typename Element>
using MfmaTileB16x32 = MfmaTile<Element, 16, 32, tl::Layout::kColMajor>;
template <typename Element>
using MfmaTileC32x32 = MfmaTile<Element, 32, 32, tl::Layout::kRowMajor>;

namespace traits {

/// Where the elements of one lane sit inside its BaseTile: kRuns runs of kRunLen consecutive elements along the minor
/// index (columns of a row-major tile, rows of a column-major one); the lane's major index is lane % kLaneMajor, run r
/// starts at minor index r * kRunStride + (lane / kLaneMajor) * kRunLen.
template <typename BaseTile>
struct TileGeometry;

/// The 16 x 16 BaseTile of types/register.hpp: one run of 4.
template <typename Element, typename Layout>
    requires BaseType<Element>
struct TileGeometry<RegTile<Element, Layout>> {
    using DType = Element;
    static constexpr int kRows = 16, kCols = 16;
    static constexpr bool kRowMajor = RegTile<Element, Layout>::kType == tl::Layout::kRowMajor;
    static constexpr int kLaneMajor = 16, kRunLen = 4, kRuns = 1, kRunStride = 16;
};

template <typename Element, const int kTileRows, const int kTileCols, const tl::Layout kType>
struct TileGeometry<MfmaTile<Element, kTileRows, kTileCols, kType>> {
    using DType = Element;
    static constexpr int kRows = kTileRows, kCols = kTileCols;
    static constexpr bool kRowMajor = kType == tl::Layout::kRowMajor;
    static constexpr int kMajor = kRowMajor ? kTileRows : kTileCols;
    static constexpr int kMinor = kRowMajor ? kTileCols : kTileRows;
    static constexpr int kLaneMajor = kMajor;                 // 16 or 32 lanes along the major index
    static constexpr int kLaneGroups = kWaveSize / kMajor;    // 4 or 2 lane groups along the minor index
    static constexpr int kPerLane = kTileRows * kTileCols / kWaveSize;
    // operand tiles: one run of 8; the 32 x 32 accumulator: 4 runs of 4, 8 apart
    static constexpr int kRunLen = kMinor / kLaneGroups <= 8 ? kMinor / kLaneGroups : 4;
    static constexpr int kRuns = kPerLane / kRunLen;
    static constexpr int kRunStride = kRunLen * kLaneGroups;
    static_assert(kRuns * kRunLen == kPerLane && kRuns * kRunStride == kMinor);
};

/// Extent of a BaseTile, in the form the copy layer's execution counts expect (kRows, kCols).
template <typename BaseTile>
struct TileExtent {
    static constexpr int kRows = TileGeometry<BaseTile>::kRows;
    static constexpr int kCols = TileGeometry<BaseTile>::kCols;
};

/// Shapes of the two f16 matrix instructions, per operand (the reference's BaseTileShape has one square shape).
enum class MfmaShape { k16x16x32 = 0, k32x32x16 = 1 };

template <typename Element, const MfmaShape kShape>
struct MfmaTileShape {
    static constexpr int kM = kShape == MfmaShape::k16x16x32 ? 16 : 32;
    static constexpr int kN = kM;
    static constexpr int kK = kShape == MfmaShape::k16x16x32 ? 32 : 16;
    using TileA = MfmaTile<Element, kM, kK, tl::Layout::kRowMajor>;
    using TileB = MfmaTile<Element, kK, kN, tl::Layout::kColMajor>;
    using TileC = std::conditional_t<kShape == MfmaShape::k16x16x32, BaseTileRowMajor<float>, MfmaTileC32x32<float>>;
};

}  // namespace traits

namespace detail {
template <typename Element, const int kR, const int kC, const tl::Layout kT>
struct IsScalar<MfmaTile<Element, kR, kC, kT>> : std::false_type {};
}  // namespace detail

}  // namespace tiledcuda::cell
