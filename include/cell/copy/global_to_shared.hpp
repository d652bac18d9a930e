// Global memory <-> LDS tile copies, cooperative over the wavefronts of a workgroup.
// Same functors as the reference's include/cell/copy/global_to_shared.hpp:250-341
// (GlobalToSharedLoader<Shared, WarpLayout>, SharedToGlobalStorer<Shared, WarpLayout>).
// The reference moves one 16x16 BaseTile per warp per cp.async (16 B per lane,
// copy_atom.hpp:326-356) into tile-contiguous shared memory; here each wavefront streams
// its share line by line, 16 B per lane (global_load_dwordx4 -> ds_write_b128), fully
// coalesced along the contiguous dimension, into the pitched / XOR-swizzled LDS tile.
#pragma once

#include "cell/copy/constants.hpp"
#include "cell/copy/vec.hpp"
#include "cell/copy/warp.hpp"
#include "types/mod.hpp"

namespace tiledcuda::cell::copy {

using namespace traits;
namespace tl = tile_layout;

namespace detail {

/// Per-wavefront line-by-line copy between a pitched global block and a shared tile view.
/// The block is kLines lines of kLineLen contiguous elements, starting at line `line0`,
/// element `elem0` of both tiles. kToShared selects the direction.
template <typename Global, typename Shared, const int kLines, const int kLineLen, const bool kToShared,
          const bool kStream = false>
struct LineCopy {
    using DType = typename Shared::DType;
    static constexpr int kVec = TraitsBase<DType>::kNumPerAccess;  // 8 x f16 or 4 x f32 = 16 B
    static_assert(kLineLen % kVec == 0, "a line must be a whole number of 16-byte accesses");

    static constexpr int kVecPerLine = kLineLen / kVec;
    static constexpr int kTotal = kLines * kVecPerLine;
    static constexpr int kIters = (kTotal + kWaveSize - 1) / kWaveSize;
    static constexpr int kGlobalPitch = Shared::kIsRowMajor ? Global::kRowStride : Global::kColStride;

    template <typename GPtr, typename STile>
    DEVICE void operator()(GPtr gptr, STile& stile, int line0, int elem0) const {
        const int lane = lane_id();
        auto* sbase = const_cast<DType*>(stile.data());
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            const int idx = lane + it * kWaveSize;
            if (kTotal % kWaveSize == 0 || idx < kTotal) {
                const int line = line0 + idx / kVecPerLine;
                const int elem = elem0 + (idx % kVecPerLine) * kVec;
                auto* g = gptr + line * kGlobalPitch + elem;
                DType* s = sbase + stile.line_offset(line, elem);
                if constexpr (kToShared) {
                    DType tmp[kVec];
                    vec_load<kVec>(g, tmp);
                    vec_store<kVec>(tmp, s);
                } else {
                    DType tmp[kVec];
                    vec_load<kVec>(s, tmp);
                    if constexpr (kStream) vec_store_stream<kVec>(tmp, const_cast<DType*>(g));
                    else vec_store<kVec>(tmp, const_cast<DType*>(g));
                }
            }
        }
    }
};

template <typename Global, typename Shared>
constexpr void check_g2s_shapes() {
    static_assert(Global::kRows == Shared::kRows && Global::kCols == Shared::kCols,
                  "Global and shared memory tiles must have the same shape.");
    static_assert(Global::kType == Shared::kType, "Global and shared memory tiles must have the same layout.");
    static_assert(std::is_same_v<typename Shared::DType, typename Global::DType>,
                  "Global and shared memory tiles must have the same element type.");
}

}  // namespace detail

/// Copy a global tile into a shared tile of the same shape; the tile is split evenly over
/// the wavefronts of WarpLayout.
template <typename Shared_, typename WarpLayout_, typename Base = warp::CopyBase<WarpLayout_, WarpReuse::kCont>>
struct GlobalToSharedLoader : public Base {
    using Shared = Shared_;
    using DType = typename Shared::DType;
    using WarpLayout = WarpLayout_;
    using BaseShape = BaseTileShape<DType>;

    static constexpr int kRowExec = Base::template row_exec_count<BaseShape, Shared::kRows>();
    static constexpr int kColExec = Base::template col_exec_count<BaseShape, Shared::kCols>();

    template <typename Global>
    DEVICE void operator()(const Global& src, Shared& dst) {
        detail::check_g2s_shapes<Global, Shared>();
        constexpr int kBlockRows = Base::template rows_per_warp<Shared::kRows>();
        constexpr int kBlockCols = Base::template cols_per_warp<Shared::kCols>();
        const int row0 = Base::template warp_row0<Shared::kRows>();
        const int col0 = Base::template warp_col0<Shared::kCols>();

        if constexpr (Shared::kIsRowMajor) {
            detail::LineCopy<Global, Shared, kBlockRows, kBlockCols, true> copy;
            copy(src.data(), dst, row0, col0);
        } else {
            detail::LineCopy<Global, Shared, kBlockCols, kBlockRows, true> copy;
            copy(src.data(), dst, col0, row0);
        }
    }
};

/// Copy a shared tile into a global tile of the same shape. kStream: with non-temporal stores (an output that the
/// kernel does not read again: nothing stays dirty in the L2 for the write-back at the kernel's end).
template <typename Shared_, typename WarpLayout_, typename Base = warp::CopyBase<WarpLayout_, WarpReuse::kCont>,
          const bool kStream = false>
struct SharedToGlobalStorer : public Base {
    using Shared = Shared_;
    using DType = typename Shared::DType;
    using WarpLayout = WarpLayout_;
    using BaseShape = BaseTileShape<DType>;

    static constexpr int kRowExec = Base::template row_exec_count<BaseShape, Shared::kRows>();
    static constexpr int kColExec = Base::template col_exec_count<BaseShape, Shared::kCols>();

    template <typename Global>
    DEVICE void operator()(const Shared& src, Global& dst) {
        detail::check_g2s_shapes<Global, Shared>();
        constexpr int kBlockRows = Base::template rows_per_warp<Shared::kRows>();
        constexpr int kBlockCols = Base::template cols_per_warp<Shared::kCols>();
        const int row0 = Base::template warp_row0<Shared::kRows>();
        const int col0 = Base::template warp_col0<Shared::kCols>();

        if constexpr (Shared::kIsRowMajor) {
            detail::LineCopy<Global, Shared, kBlockRows, kBlockCols, false, kStream> copy;
            copy(dst.mutable_data(), src, row0, col0);
        } else {
            detail::LineCopy<Global, Shared, kBlockCols, kBlockRows, false, kStream> copy;
            copy(dst.mutable_data(), src, col0, row0);
        }
    }
};

/// SharedToGlobalStorer with non-temporal stores.
template <typename Shared_, typename WarpLayout_>
using SharedToGlobalStreamStorer =
    SharedToGlobalStorer<Shared_, WarpLayout_, warp::CopyBase<WarpLayout_, WarpReuse::kCont>, true>;

}  // namespace tiledcuda::cell::copy
