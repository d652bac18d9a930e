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

/// Wait until at most kOutstanding of this wavefront's LDS reads are still in flight (they return in order): the
/// companion of SharedToRegPieces / SharedToRegTrPieces, whose reads the compiler does not track.
template <int kOutstanding>
DEVICE void wait_shared_reads() {
    static_assert(kOutstanding >= 0 && kOutstanding < 16);
    __builtin_amdgcn_s_waitcnt(0xC07F | (kOutstanding << 8));  // lgkmcnt(kOutstanding), nothing else
}

namespace detail {
/// Wave-uniform LDS byte address of logical line 0, element 0 of a (sub-)tile whose origin lies a multiple of the
/// swizzle's line period into its allocation (the permutation then looks the same from the view as from the tile).
template <typename Shared>
DEVICE unsigned int shared_view_address(const Shared& tile) {
    // (through an LDS-qualified pointer: the cast back from the generic address space then folds away, where the
    // truncation of a generic address would keep a null check per use)
    using lds_cptr = __attribute__((address_space(3))) const void*;
    const unsigned int base = static_cast<unsigned int>(reinterpret_cast<uintptr_t>((lds_cptr)(tile.data())));
    return base + static_cast<unsigned int>(tile.line0() * Shared::kPitch + tile.elem0()) *
                      static_cast<unsigned int>(sizeof(typename Shared::DType));
}
}  // namespace detail

/// SharedToRegLoader a fragment at a time with the waits in the caller's hands, for kernels that run one wavefront
/// per SIMD and request each operand fragment a fixed number of matrix instructions before its use, also across loop
/// back-edges and between stages of a SharedRing. The compiler's own waits for LDS reads are exact only inside a basic
/// block; across a back-edge it waits for every read in flight, including those just requested for later
/// instructions. So the reads here are assembly the compiler does not track: read<i, j>() requests fragment (i, j) of
/// the register tile (one ds_read_b128 for an MFMA operand tile of 2-byte elements), and the caller places
/// wait_shared_reads<N>() before the first use. The per-lane byte offset of every fragment inside the tile (swizzle
/// included) is computed once, at construction, and kept in a register; a read adds the wave-uniform address of the
/// (sub-)tile it is pointed at: one vector addition per read.
/// Shared_ is the tile type the offsets are computed for (a whole stage of a ring, or the sub-tile a wavefront's
/// operand comes from); read() takes any view of that type whose origin is a multiple of the swizzle's line period.
/// kDealtLines: the lines (rows of A, columns of B) of a PAIR of neighbouring operand tiles are dealt to the two tiles
/// four at a time - tile 2 p + h holds lines 32 p + 8 q + 4 h + r (q, r = 0..3) as its lines 4 q + r - instead of 16
/// consecutive ones each. The two 16 x 16 accumulators of a product with such a pair then hold, per lane, 8 CONSECUTIVE
/// lines (accumulator 2 p: 8 g .. 8 g + 3, accumulator 2 p + 1: 8 g + 4 .. 8 g + 7 for lane group g): converted, they are
/// an A operand in the standard contraction order, and the other operand of the next product can be read with plain
/// 16-byte reads along its lines (a V stored column-major).
template <typename Reg_, typename Shared_, typename WarpLayout_, const WarpReuse kMode_, const bool kDealtLines = false,
          typename Base = warp::CopyBase<WarpLayout_, kMode_>>
struct SharedToRegPieces : public Base {
    using Reg = Reg_;
    using Shared = Shared_;
    using BaseTile = typename Reg::DType;
    using DType = typename BaseTile::DType;
    using G = TileGeometry<BaseTile>;
    using BaseShape = TileExtent<BaseTile>;
    static_assert(std::is_same_v<typename Shared::DType, DType> && sizeof(DType) == 2 && G::kRuns == 1 && G::kRunLen == 8 &&
                      G::kRowMajor == Shared::kIsRowMajor,
                  "one ds_read_b128 per fragment: MFMA operand tiles of 2-byte elements whose runs lie along the lines");
    static_assert(Base::template row_exec_count<BaseShape, Shared::kRows>() == Reg::kRows &&
                      Base::template col_exec_count<BaseShape, Shared::kCols>() == Reg::kCols,
                  "the register tile must hold exactly this wavefront's share of the shared tile");

    static_assert(!kDealtLines || (G::kLaneMajor == 16 && (G::kRowMajor ? Reg::kRows : Reg::kCols) % 2 == 0),
                  "lines are dealt to pairs of 16-line operand tiles");

    DEVICE SharedToRegPieces() {
        const int lane = lane_id();
        const int major = lane % G::kLaneMajor, minor = (lane / G::kLaneMajor) * G::kRunLen;
        // line of operand tile t (along the major index) that this lane holds
        auto line_of = [&](int t) {
            return kDealtLines ? (t / 2) * 32 + 8 * (major / 4) + 4 * (t % 2) + major % 4 : t * G::kLaneMajor + major;
        };
        const int row0 = Base::template warp_row0<Shared::kRows>();
        const int col0 = Base::template warp_col0<Shared::kCols>();
        const Shared whole(nullptr);
#pragma unroll
        for (int i = 0; i < Reg::kRows; ++i)
#pragma unroll
            for (int j = 0; j < Reg::kCols; ++j) {
                const int row = row0 + (G::kRowMajor ? line_of(i) : i * BaseShape::kRows + minor);
                const int col = col0 + (G::kRowMajor ? j * BaseShape::kCols + minor : line_of(j));
                offset_[i][j] = static_cast<unsigned int>(whole.offset(row, col)) * static_cast<unsigned int>(sizeof(DType));
                asm volatile("" : "+v"(offset_[i][j]));  // computed once, not again at every use
            }
    }

    /// Request fragment (kI, kJ) of this wavefront's share of `src` into dst(kI, kJ); not waited for.
    template <int kI, int kJ>
    DEVICE void read(const Shared& src, Reg& dst) const {
        f16x8 r;
        asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(offset_[kI][kJ] + detail::shared_view_address(src)));
        __builtin_memcpy(dst(kI, kJ).mutable_data(), &r, sizeof(r));
    }

    /// The same without an addition in front of every read (a vector addition directly in front of the LDS read that
    /// takes its result stalls the wavefront for several cycles, and every instruction between two matrix
    /// instructions costs issue time): bind() makes the kept offsets absolute addresses inside the view `src`, once;
    /// read_bound<i, j, kBytes>() then reads fragment (i, j) of the view that lies kBytes further on (an immediate of the
    /// instruction: a multiple of the swizzle's period in lines, below 64 KiB), and shift<i, j>(bytes) moves one
    /// fragment's address on to another view (another stage of a ring) - one addition per fragment and move, placed
    /// by the caller well ahead of the fragment's next read.
    DEVICE void bind(const Shared& src) {
        const unsigned int base = detail::shared_view_address(src);
#pragma unroll
        for (int i = 0; i < Reg::kRows; ++i)
#pragma unroll
            for (int j = 0; j < Reg::kCols; ++j) {
                offset_[i][j] += base;
                asm volatile("" : "+v"(offset_[i][j]));
            }
    }
    template <int kI, int kJ, int kBytes = 0>
    DEVICE void read_bound(Reg& dst) const {
        read_bound_to<kI, kJ, kBytes>(dst(kI, kJ));
    }
    /// ... into any operand tile (a kernel that keeps only the fragments in flight, as a ring of a few tiles).
    template <int kI, int kJ, int kBytes = 0>
    DEVICE void read_bound_to(BaseTile& dst) const {
        static_assert(kBytes >= 0 && kBytes < 65536 &&
                          kBytes % ((Shared::kSwizzled ? Shared::Swizzle::kLinePeriod : 1) * Shared::kPitch * int(sizeof(DType))) == 0,
                      "the immediate moves the view by whole periods of the swizzle");
        f16x8 r;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(offset_[kI][kJ]), "n"(kBytes));
        __builtin_memcpy(dst.mutable_data(), &r, sizeof(r));
    }
    template <int kI, int kJ>
    DEVICE void shift(int bytes) {
        offset_[kI][kJ] += static_cast<unsigned int>(bytes);
        asm volatile("" : "+v"(offset_[kI][kJ]));
    }

  private:
    unsigned int offset_[Reg::kRows][Reg::kCols];
};

/// The same for the transposing read (SharedToRegLoaderTr: a column-major operand out of a row-major shared tile):
/// read<i, j>() requests the two ds_read_b64_tr_b16 of operand tile (i, j). One per-lane offset per COLUMN of operand
/// tiles is kept; the contraction index (the tile's row i) is an immediate of the instruction, which requires a
/// swizzle whose line period divides 4 (tl::LdsSwizzleTr).
/// kAccumulatorOrder: which contraction indices a lane receives. false: the standard operand order (lane group
/// g = lane / 32 or lane / 16 holds indices 8 g .. 8 g + 7 of the tile). true: the order in which the accumulators of
/// a preceding product hold their columns, so that accumulator values converted to 2-byte elements ARE the A operand
/// of the next product without leaving the lane (the contraction index of a matrix instruction may be permuted as long
/// as both operands agree). For 16 x 32 tiles (B of v_mfma_f32_32x32x16_f16) that is one 32 x 32 accumulator: slot e of
/// lane half h is index 8 (e / 4) + 4 h + e % 4. For 32 x 16 tiles (B of v_mfma_f32_16x16x32_f16) it is two 16 x 16
/// accumulators side by side: slot e of lane group g is index 16 (e / 4) + 4 g + e % 4.
template <typename Reg_, typename Shared_, typename WarpLayout_, const WarpReuse kMode_, const bool kAccumulatorOrder = false,
          typename Base = warp::CopyBase<WarpLayout_, kMode_>>
struct SharedToRegTrPieces : public Base {
    using Reg = Reg_;
    using Shared = Shared_;
    using BaseTile = typename Reg::DType;
    using DType = typename BaseTile::DType;
    using G = TileGeometry<BaseTile>;
    using BaseShape = TileExtent<BaseTile>;
    static_assert(std::is_same_v<typename Shared::DType, DType> && sizeof(DType) == 2 && Shared::kIsRowMajor &&
                      !G::kRowMajor && G::kRunLen == 8 && G::kRuns == 1,
                  "the transposing read serves column-major operand tiles of 2-byte elements out of a row-major tile");
    static constexpr int kPeriod = Shared::kSwizzled ? Shared::Swizzle::kLinePeriod : 1;
    static_assert(Base::template row_exec_count<BaseShape, Shared::kRows>() == Reg::kRows &&
                      Base::template col_exec_count<BaseShape, Shared::kCols>() == Reg::kCols,
                  "the register tile must hold exactly this wavefront's share of the shared tile");
    static constexpr int kLineBytes = Shared::kPitch * int(sizeof(DType));
    // rows between the two reads of an operand tile, and how many rows a lane group's index moves the first one
    static constexpr int kPartRows = kAccumulatorOrder ? 4 * (kWaveSize / G::kLaneMajor) : 4;
    static constexpr int kGroupRows = kAccumulatorOrder ? 4 : 8;
    static_assert(kPartRows % kPeriod == 0 && BaseShape::kRows % kPeriod == 0,
                  "the tile's row is an immediate of the read: the swizzle must repeat with the rows between the two reads "
                  "and with the tile height (tl::LdsSwizzleTr)");

    DEVICE SharedToRegTrPieces() {
        const int lane = lane_id();
        const int L = lane & 15;
        const int col_grp = ((lane >> 4) % (G::kLaneMajor / 16)) * 16;
        const int line = Base::template warp_row0<Shared::kRows>() + (lane / G::kLaneMajor) * kGroupRows + (L >> 2);
        const int col0 = Base::template warp_col0<Shared::kCols>();
        const Shared whole(nullptr);
#pragma unroll
        for (int j = 0; j < Reg::kCols; ++j) {
            const int col = col0 + j * BaseShape::kCols + col_grp + 4 * (L & 3);
            offset_[j] = static_cast<unsigned int>(whole.offset(line, col)) * static_cast<unsigned int>(sizeof(DType));
            asm volatile("" : "+v"(offset_[j]));
        }
    }

    /// Request operand tile (kI, kJ) of this wavefront's share of the view `src` shifted down by kLine0 lines (a
    /// multiple of 4, folded into the instruction's immediate together with the tile's own row); not waited for.
    template <int kI, int kJ, int kLine0 = 0>
    DEVICE void read(const Shared& src, Reg& dst) const {
        static_assert(kLine0 % 4 == 0 && kLine0 % kPeriod == 0);
        constexpr int kOff0 = (kLine0 + kI * BaseShape::kRows) * kLineBytes, kOff1 = kOff0 + kPartRows * kLineBytes;
        static_assert(kOff1 < 65536, "the immediate offset of an LDS read has 16 bits");
        f16x4 lo, hi;
        asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                     : "=&v"(lo), "=&v"(hi)
                     : "v"(offset_[kJ] + detail::shared_view_address(src)), "n"(kOff0), "n"(kOff1));
        const f16x8 r = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        __builtin_memcpy(dst(kI, kJ).mutable_data(), &r, sizeof(r));
    }

    /// Absolute addresses, as in SharedToRegPieces: bind() once to a view, read_bound<i, j, kBytes>() reads operand tile
    /// (i, j) of the view kBytes further on, shift<j>(bytes) moves the address kept for column j of operand tiles.
    DEVICE void bind(const Shared& src) {
        const unsigned int base = detail::shared_view_address(src);
#pragma unroll
        for (int j = 0; j < Reg::kCols; ++j) {
            offset_[j] += base;
            asm volatile("" : "+v"(offset_[j]));
        }
    }
    template <int kI, int kJ, int kBytes = 0>
    DEVICE void read_bound(Reg& dst) const {
        read_bound_to<kI, kJ, kBytes>(dst(kI, kJ));
    }
    template <int kI, int kJ, int kBytes = 0>
    DEVICE void read_bound_to(BaseTile& dst) const {
        static_assert(kBytes >= 0 && kBytes % (kPeriod * kLineBytes) == 0, "the immediate moves the view by whole periods of the swizzle");
        constexpr int kOff0 = kBytes + kI * BaseShape::kRows * kLineBytes, kOff1 = kOff0 + kPartRows * kLineBytes;
        static_assert(kOff1 < 65536, "the immediate offset of an LDS read has 16 bits");
        f16x4 lo, hi;
        asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                     : "=&v"(lo), "=&v"(hi)
                     : "v"(offset_[kJ]), "n"(kOff0), "n"(kOff1));
        const f16x8 r = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        __builtin_memcpy(dst.mutable_data(), &r, sizeof(r));
    }
    template <int kJ>
    DEVICE void shift(int bytes) {
        offset_[kJ] += static_cast<unsigned int>(bytes);
        asm volatile("" : "+v"(offset_[kJ]));
    }

  private:
    unsigned int offset_[Reg::kCols];
};

}  // namespace tiledcuda::cell::copy
