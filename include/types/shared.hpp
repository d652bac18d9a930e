// View of a tile in LDS. Same members as the reference's include/types/shared.hpp:9-46,
// plus an origin: a sub-tile produced by STileIterator keeps the base pointer of the tile it
// was cut from and its (line, element) origin inside it, because the XOR swizzle is a
// function of absolute coordinates within the pitched allocation.
#pragma once

#include <type_traits>

#include "types/layout.hpp"
#include "util/print.hpp"

namespace tiledcuda::cell {
namespace tl = tile_layout;

/// SwizzlePolicy_: which XOR permutation a swizzled tile uses (void = tl::LdsSwizzle, the one for plain vector reads
/// along a line; tl::LdsSwizzleTr for tiles read across lines with the transposing LDS read). Sub-tiles cut by
/// STileIterator keep their tile's policy.
template <typename Element_, typename Layout_, const bool kSwizzled_ = false, typename SwizzlePolicy_ = void>
class SharedTile {
  public:
    using DType = Element_;
    using Layout = Layout_;
    using SwizzlePolicy = SwizzlePolicy_;

    static constexpr int kNumel = tl::get_numel<Layout>;

    static constexpr int kRows = tl::num_rows<Layout>;
    static constexpr int kCols = tl::num_cols<Layout>;

    static constexpr int kRowStride = tl::row_stride<Layout>;
    static constexpr int kColStride = tl::col_stride<Layout>;

    static constexpr tl::Layout kType = tl::layout_type<Layout>;
    static constexpr bool kSwizzled = kSwizzled_;

    static constexpr bool kIsRowMajor = kType == tl::Layout::kRowMajor;
    // distance between consecutive lines (rows if row-major, columns otherwise)
    static constexpr int kPitch = kIsRowMajor ? kRowStride : kColStride;
    // number of lines / elements per line of this view
    static constexpr int kLines = kIsRowMajor ? kRows : kCols;
    static constexpr int kLineLen = kIsRowMajor ? kCols : kRows;

    using Swizzle = std::conditional_t<std::is_void_v<SwizzlePolicy_>, tl::LdsSwizzle<kPitch, sizeof(DType)>, SwizzlePolicy_>;

    HOST_DEVICE SharedTile(DType* data) : data_(data), line0_(0), elem0_(0) {}

    /// A view whose logical (0, 0) sits at (line0, elem0) of the allocation starting at `base`.
    HOST_DEVICE SharedTile(DType* base, int line0, int elem0) : data_(base), line0_(line0), elem0_(elem0) {}

    /// Base pointer of the allocation this view addresses into.
    HOST_DEVICE DType* mutable_data() { return data_; }
    HOST_DEVICE const DType* data() const { return data_; }

    HOST_DEVICE int line0() const { return line0_; }
    HOST_DEVICE int elem0() const { return elem0_; }

    HOST_DEVICE constexpr Layout layout() const { return Layout{}; }

    /// Element offset (from the base pointer) of the element at line `line`, position `elem`
    /// of this view. Four consecutive positions starting at a multiple of 4 are contiguous.
    HOST_DEVICE int line_offset(int line, int elem) const {
        const int l = line + line0_;
        const int e = elem + elem0_;
        if constexpr (kSwizzled) {
            return l * kPitch + Swizzle::apply(l, e);
        } else {
            return l * kPitch + e;
        }
    }

    /// Element offset of logical element (row x, column y).
    HOST_DEVICE int offset(int x, int y) const { return kIsRowMajor ? line_offset(x, y) : line_offset(y, x); }

    HOST_DEVICE DType& operator()(int x, int y) { return data_[offset(x, y)]; }

    HOST_DEVICE const DType& operator()(int x, int y) const { return data_[offset(x, y)]; }

    DEVICE void dump_value() {
        for (int i = 0; i < kRows; ++i) {
            for (int j = 0; j < kCols; ++j) printf("%.3f, ", print_cast((*this)(i, j)));
            printf("\n");
        }
    }

  private:
    DType* data_;
    int line0_;
    int elem0_;
};

/// kStages copies of a shared tile laid out back to back: the LDS side of a multi-stage global -> LDS pipeline
/// (the reference's kernels have one stage and wait for every load, examples/cpp/01_gemm/02_gemm_all_mem/gemm.hpp:139-143).
/// ring[s] is a whole-tile view of stage s; stages advance modulo kStages. kStrideNumel_: elements from one stage to
/// the next (0 = the tile's own size: stages back to back); larger when the stages of two rings are interleaved, e.g.
/// the K and V blocks of an attention kernel as [K0 V0 K1 V1 ...].
template <typename Shared_, const int kStages_, const int kStrideNumel_ = 0>
class SharedRing {
  public:
    using Shared = Shared_;
    using DType = typename Shared::DType;
    static constexpr int kStages = kStages_;
    static constexpr int kTileNumel = Shared::kLines * Shared::kPitch;
    static constexpr int kStageNumel = kStrideNumel_ == 0 ? kTileNumel : kStrideNumel_;
    static_assert(kStageNumel >= kTileNumel, "stages must not overlap");
    static constexpr int kStageBytes = kStageNumel * int(sizeof(DType));
    // bytes from the first stage's start to the last stage's end
    static constexpr int kBytes = ((kStages - 1) * kStageNumel + kTileNumel) * int(sizeof(DType));

    HOST_DEVICE explicit SharedRing(DType* base) : base_(base) {}

    HOST_DEVICE Shared operator[](int stage) const { return Shared(base_ + stage * kStageNumel); }
    HOST_DEVICE DType* stage_data(int stage) const { return base_ + stage * kStageNumel; }
    HOST_DEVICE static constexpr int next(int stage) { return stage + 1 == kStages ? 0 : stage + 1; }

  private:
    DType* base_;
};

}  // namespace tiledcuda::cell
