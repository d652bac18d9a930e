// LDS <-> register tile copies in BaseTile lane order.
// Same functors as the reference's include/cell/copy/shared_to_register.hpp:194-301
// (SharedToRegLoader<Reg, WarpLayout, WarpReuse>, RegToSharedStorer<Reg, WarpLayout>).
// The reference reads with ldmatrix.x4 (copy_atom.hpp:55-64) and scatters mma C-fragments
// in 2-element segments (:71-288); here a lane reads or writes its 4 contiguous elements of
// each BaseTile with one ds_read_b64 / ds_write_b64 (f16) or b128 (f32). Addresses are taken
// from logical coordinates of the (possibly swizzled, possibly sub-) shared tile.
// The same functors move MFMA-shaped operand tiles (types/mfma_tile.hpp): a lane's 8 consecutive f16 along the
// contraction index are one ds_read_b128, half the LDS instructions per MFMA of the 16 x 16 BaseTile path.
// SharedToRegLoaderTr reads a column-major operand out of a ROW-major shared tile (contraction index along the rows,
// e.g. V of an attention layer stored [keys, head_dim]) with the transposing read ds_read_b64_tr_b16; the reference
// has no counterpart (ldmatrix.trans plays that role inside its copy atoms, copy_atom.hpp:55-64).
#pragma once

#include "cell/copy/constants.hpp"
#include "cell/copy/vec.hpp"
#include "cell/copy/warp.hpp"
#include "types/mod.hpp"

namespace tiledcuda::cell::copy {

using namespace traits;
namespace tl = tile_layout;

namespace detail {

/// Move one lane's share of the BaseTile whose top-left element is (row0, col0) of `tile`.
template <typename Shared, typename BaseTile, const bool kLoad>
DEVICE void move_shared_base_tile(Shared& tile, int row0, int col0, BaseTile& reg) {
    using DType = typename Shared::DType;
    constexpr bool kRegRowMajor = BaseTile::kType == tl::Layout::kRowMajor;
    const int row = row0 + (kRegRowMajor ? lane_major() : lane_minor());
    const int col = col0 + (kRegRowMajor ? lane_minor() : lane_major());
    auto* base = const_cast<DType*>(tile.data());

    if constexpr (kRegRowMajor == Shared::kIsRowMajor) {
        // the lane's 4 elements are one contiguous chunk of a line
        DType* p = base + tile.offset(row, col);
        if constexpr (kLoad)
            vec_load<4>(p, reg.mutable_data());
        else
            vec_store<4>(reg.data(), p);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            DType* p = base + (kRegRowMajor ? tile.offset(row, col + e) : tile.offset(row + e, col));
            if constexpr (kLoad)
                reg.mutable_data()[e] = *p;
            else
                *p = reg.data()[e];
        }
    }
}

/// Move one lane's share of the tile (16 x 16 BaseTile or MFMA-shaped tile) whose top-left element is (row0, col0)
/// of `tile`. Runs that lie along a line of the shared tile move as vectors of up to 16 bytes (the swizzle keeps
/// 16-byte pieces of 2-byte elements and 8- or 16-byte pieces of 4-byte elements contiguous); runs across lines move
/// element by element.
template <typename Shared, typename BaseTile, const bool kLoad>
DEVICE void move_shared_tile(Shared& tile, int row0, int col0, BaseTile& reg) {
    using G = TileGeometry<std::remove_const_t<BaseTile>>;
    using DType = typename Shared::DType;
    const int lane = lane_id();
    const int major = lane % G::kLaneMajor;
    const int minor0 = (lane / G::kLaneMajor) * G::kRunLen;
    auto* base = const_cast<DType*>(tile.data());
    auto* r = const_cast<DType*>(reg.data());
    // longest piece of a line that stays contiguous under the swizzle
    constexpr int kPiece = (sizeof(DType) == 2 && G::kRunLen % 8 == 0) ? 8 : 4;
#pragma unroll
    for (int run = 0; run < G::kRuns; ++run) {
        const int minor = minor0 + run * G::kRunStride;
        const int row = row0 + (G::kRowMajor ? major : minor);
        const int col = col0 + (G::kRowMajor ? minor : major);
        if constexpr (G::kRowMajor == Shared::kIsRowMajor) {
#pragma unroll
            for (int e = 0; e < G::kRunLen; e += kPiece) {
                DType* p = base + (G::kRowMajor ? tile.offset(row, col + e) : tile.offset(row + e, col));
                if constexpr (kLoad)
                    vec_load<kPiece>(p, r + run * G::kRunLen + e);
                else
                    vec_store<kPiece>(r + run * G::kRunLen + e, p);
            }
        } else {
#pragma unroll
            for (int e = 0; e < G::kRunLen; ++e) {
                DType* p = base + (G::kRowMajor ? tile.offset(row, col + e) : tile.offset(row + e, col));
                if constexpr (kLoad)
                    r[run * G::kRunLen + e] = *p;
                else
                    *p = r[run * G::kRunLen + e];
            }
        }
    }
}

}  // namespace detail

/// Load this wavefront's share of a shared tile into a register tile.
template <typename Reg_, typename WarpLayout_, const WarpReuse kMode_,
          typename Base = warp::CopyBase<WarpLayout_, kMode_>>
struct SharedToRegLoader : public Base {
    using Reg = Reg_;
    using BaseTile = typename Reg::DType;
    using DType = typename BaseTile::DType;
    using BaseShape = TileExtent<BaseTile>;

    using WarpLayout = WarpLayout_;
    static constexpr WarpReuse kMode = kMode_;

    template <typename Shared>
    DEVICE void operator()(const Shared& src, Reg& dst) {
        static_assert(std::is_same_v<typename Shared::DType, DType>,
                      "The data type of Shared and Reg must be the same.");
        static constexpr int kRowExec = Base::template row_exec_count<BaseShape, Shared::kRows>();
        static constexpr int kColExec = Base::template col_exec_count<BaseShape, Shared::kCols>();
        static_assert(kRowExec == Reg::kRows && kColExec == Reg::kCols,
                      "the register tile must hold exactly this wavefront's share of the shared tile");

        const int row0 = Base::template warp_row0<Shared::kRows>();
        const int col0 = Base::template warp_col0<Shared::kCols>();
#pragma unroll
        for (int i = 0; i < kRowExec; ++i) {
#pragma unroll
            for (int j = 0; j < kColExec; ++j) {
                detail::move_shared_tile<const Shared, BaseTile, true>(src, row0 + i * BaseShape::kRows,
                                                                       col0 + j * BaseShape::kCols, dst(i, j));
            }
        }
    }
    /// BaseTile (i, j) of this wavefront's share only: for kernels that place each fragment read between particular
    /// matrix instructions (compute::gemm_scheduled) instead of reading a whole register tile at once.
    template <typename Shared>
    DEVICE void load_one(const Shared& src, Reg& dst, int i, int j) {
        static_assert(std::is_same_v<typename Shared::DType, DType>,
                      "The data type of Shared and Reg must be the same.");
        static_assert(Base::template row_exec_count<BaseShape, Shared::kRows>() == Reg::kRows &&
                          Base::template col_exec_count<BaseShape, Shared::kCols>() == Reg::kCols,
                      "the register tile must hold exactly this wavefront's share of the shared tile");
        detail::move_shared_tile<const Shared, BaseTile, true>(
            src, Base::template warp_row0<Shared::kRows>() + i * BaseShape::kRows,
            Base::template warp_col0<Shared::kCols>() + j * BaseShape::kCols, dst(i, j));
    }
};

/// Store a register tile into this wavefront's share of a shared tile (even split).
template <typename Reg_, typename WarpLayout_>
struct RegToSharedStorer : public warp::CopyBase<WarpLayout_, WarpReuse::kCont> {
    using Base = warp::CopyBase<WarpLayout_, WarpReuse::kCont>;
    using Reg = Reg_;
    using BaseTile = typename Reg::DType;
    using DType = typename BaseTile::DType;
    using BaseShape = TileExtent<BaseTile>;
    using WarpLayout = WarpLayout_;

    template <typename Shared>
    DEVICE void operator()(const Reg& src, Shared& dst) {
        static_assert(std::is_same_v<typename Shared::DType, DType>,
                      "The element data type of Shared and Register tile must be the same.");
        static_assert((Reg::kNumel * BaseTile::kNumel * kWaveSize * tl::get_numel<WarpLayout>) == Shared::kNumel,
                      "The number of elements held in the register files of all lanes of the workgroup "
                      "must equal the number held in the shared memory tile.");
        static constexpr int kRowExec = Base::template row_exec_count<BaseShape, Shared::kRows>();
        static constexpr int kColExec = Base::template col_exec_count<BaseShape, Shared::kCols>();
        static_assert(kRowExec == Reg::kRows && kColExec == Reg::kCols,
                      "the register tile must hold exactly this wavefront's share of the shared tile");

        const int row0 = Base::template warp_row0<Shared::kRows>();
        const int col0 = Base::template warp_col0<Shared::kCols>();
#pragma unroll
        for (int i = 0; i < kRowExec; ++i) {
#pragma unroll
            for (int j = 0; j < kColExec; ++j) {
                detail::move_shared_tile<Shared, const BaseTile, false>(dst, row0 + i * BaseShape::kRows,
                                                                        col0 + j * BaseShape::kCols, src(i, j));
            }
        }
    }
};

/// Load a column-major MFMA operand (B: contraction index along the rows of the tile) out of a ROW-major shared tile
/// of 2-byte elements, i.e. transpose on the way: ds_read_b64_tr_b16 hands each lane of a 16-lane group 4 consecutive
/// rows of ONE column of a 4 x 16 block whose rows the lanes address 4 x 8 bytes at a time. Two reads per operand tile
/// (8 contraction indices per lane). Same call shape as SharedToRegLoader.
template <typename Reg_, typename WarpLayout_, const WarpReuse kMode_,
          typename Base = warp::CopyBase<WarpLayout_, kMode_>>
struct SharedToRegLoaderTr : public Base {
    using Reg = Reg_;
    using BaseTile = typename Reg::DType;
    using DType = typename BaseTile::DType;
    using G = TileGeometry<BaseTile>;
    using BaseShape = TileExtent<BaseTile>;
    using WarpLayout = WarpLayout_;
    static constexpr WarpReuse kMode = kMode_;
    static_assert(sizeof(DType) == 2 && !G::kRowMajor && G::kRunLen == 8 && G::kRuns == 1,
                  "the transposing read serves column-major operand tiles of 2-byte elements");

    template <typename Shared>
    DEVICE void operator()(const Shared& src, Reg& dst) {
        static_assert(std::is_same_v<typename Shared::DType, DType> && Shared::kIsRowMajor,
                      "the transposing loader reads a row-major shared tile of the operand's element type");
        static constexpr int kRowExec = Base::template row_exec_count<BaseShape, Shared::kRows>();
        static constexpr int kColExec = Base::template col_exec_count<BaseShape, Shared::kCols>();
        static_assert(kRowExec == Reg::kRows && kColExec == Reg::kCols,
                      "the register tile must hold exactly this wavefront's share of the shared tile");
        using fp16x4 = __fp16 __attribute__((ext_vector_type(4)));
        using lds_ptr = fp16x4 __attribute__((address_space(3)))*;

        const int lane = lane_id();
        const int L = lane & 15;                                  // lane within its 16-lane group
        const int col_grp = ((lane >> 4) % (G::kLaneMajor / 16)) * 16;  // which 16 columns of the tile the group serves
        const int k0 = (lane / G::kLaneMajor) * 8;                // first contraction index of this lane
        const int row0 = Base::template warp_row0<Shared::kRows>();
        const int col0 = Base::template warp_col0<Shared::kCols>();
        const DType* base = src.data();
#pragma unroll
        for (int i = 0; i < kRowExec; ++i) {
#pragma unroll
            for (int j = 0; j < kColExec; ++j) {
                DType* r = dst(i, j).mutable_data();
#pragma unroll
                for (int part = 0; part < 2; ++part) {
                    const int row = row0 + i * BaseShape::kRows + k0 + 4 * part + (L >> 2);
                    const int col = col0 + j * BaseShape::kCols + col_grp + 4 * (L & 3);
                    const DType* p = base + src.offset(row, col);
                    const fp16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_ptr)(p));
                    __builtin_memcpy(r + 4 * part, &v, sizeof(v));
                }
            }
        }
    }
};

}  // namespace tiledcuda::cell::copy
