// Broadcast a per-row (or per-column) vector over a register tile, optionally fused with a
// binary op. Same functors as the reference's include/cell/compute/broadcast.hpp:21-160
// (Broadcast, BroadcastAdd/Sub/Mul/Div<SrcTile, DstTile, kLayout>; fused form computes
// dst = op(dst, src_broadcast)). The source holds one value per BaseTile row (column) per
// lane, as produced by the reductions.
#pragma once

#include "cell/compute/math_functor.hpp"
#include "types/layout.hpp"
#include "types/tile_shape.hpp"

namespace tiledcuda::cell::compute {
namespace tl = tile_layout;

template <typename SrcTile, typename DstTile, const tl::Layout kLayout>
struct Broadcast;

template <typename SrcTile, typename DstTile>
struct Broadcast<SrcTile, DstTile, tl::Layout::kRowMajor> {
    using DType = typename DstTile::DType::DType;

    DEVICE void operator()(const SrcTile& src, DstTile& dst) {
#pragma unroll
        for (int i = 0; i < DstTile::kRows; ++i) {
            const DType v = src(i, 0);
#pragma unroll
            for (int j = 0; j < DstTile::kCols; ++j) {
#pragma unroll
                for (int e = 0; e < 4; ++e) dst(i, j)(0, e) = v;
            }
        }
    }
};

template <typename SrcTile, typename DstTile>
struct Broadcast<SrcTile, DstTile, tl::Layout::kColMajor> {
    using DType = typename DstTile::DType::DType;

    DEVICE void operator()(const SrcTile& src, DstTile& dst) {
#pragma unroll
        for (int j = 0; j < DstTile::kCols; ++j) {
            const DType v = src(0, j);
#pragma unroll
            for (int i = 0; i < DstTile::kRows; ++i) {
#pragma unroll
                for (int e = 0; e < 4; ++e) dst(i, j)(e, 0) = v;
            }
        }
    }
};

template <typename SrcTile, typename DstTile, typename Functor, const tl::Layout kLayout>
struct BroadcastFuse;

template <typename SrcTile, typename DstTile, typename Functor>
struct BroadcastFuse<SrcTile, DstTile, Functor, tl::Layout::kRowMajor> {
    using DType = typename DstTile::DType::DType;

    DEVICE void operator()(const SrcTile& src, DstTile& dst) {
        Functor f;
#pragma unroll
        for (int i = 0; i < DstTile::kRows; ++i) {
            const DType v = src(i, 0);
#pragma unroll
            for (int j = 0; j < DstTile::kCols; ++j) {
#pragma unroll
                for (int e = 0; e < 4; ++e) f(dst(i, j)(0, e), v, dst(i, j)(0, e));
            }
        }
    }
};

template <typename SrcTile, typename DstTile, typename Functor>
struct BroadcastFuse<SrcTile, DstTile, Functor, tl::Layout::kColMajor> {
    using DType = typename DstTile::DType::DType;

    DEVICE void operator()(const SrcTile& src, DstTile& dst) {
        Functor f;
#pragma unroll
        for (int j = 0; j < DstTile::kCols; ++j) {
            const DType v = src(0, j);
#pragma unroll
            for (int i = 0; i < DstTile::kRows; ++i) {
#pragma unroll
                for (int e = 0; e < 4; ++e) f(dst(i, j)(e, 0), v, dst(i, j)(e, 0));
            }
        }
    }
};

template <typename SrcTile, typename DstTile, const tl::Layout kLayout>
using BroadcastAdd = BroadcastFuse<SrcTile, DstTile, Add<typename SrcTile::DType>, kLayout>;

template <typename SrcTile, typename DstTile, const tl::Layout kLayout>
using BroadcastSub = BroadcastFuse<SrcTile, DstTile, Sub<typename SrcTile::DType>, kLayout>;

template <typename SrcTile, typename DstTile, const tl::Layout kLayout>
using BroadcastMul = BroadcastFuse<SrcTile, DstTile, Mul<typename SrcTile::DType>, kLayout>;

template <typename SrcTile, typename DstTile, const tl::Layout kLayout>
using BroadcastDiv = BroadcastFuse<SrcTile, DstTile, Div<typename SrcTile::DType>, kLayout>;

}  // namespace tiledcuda::cell::compute
