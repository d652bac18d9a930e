// Global memory -> LDS without a stop in registers: the CDNA4 counterpart of the cp.async path of the reference's
// GlobalToSharedLoader (include/cell/copy/global_to_shared.hpp:250-295, copy_atom.hpp:326-356).
// global_load_lds_dwordx4 makes each of the 64 lanes fetch 16 bytes and writes them to LDS at base + 16 * lane, i.e.
// one instruction fills 1 KiB of LDS contiguously. The XOR swizzle of the shared tile is therefore applied on the
// global side: a lane computes which logical piece of which line belongs at its physical position and reads that.
// The loads are issued as inline assembly, untracked by the compiler: with the builtin, the compiler treats a tile
// in flight as a pending LDS write and waits for ALL outstanding loads before the next LDS read it cannot prove
// disjoint, and before every __syncthreads(), so a ring of stages degenerates to one tile in flight. Completion is
// the caller's business, exactly as with cp.async: wait_group<N>() / wait_group_and_barrier<N>() (cell/sync.hpp)
// before the stage is read.
#pragma once

#include "cell/copy/constants.hpp"
#include "cell/copy/warp.hpp"
#include "types/mod.hpp"

namespace tiledcuda::cell::copy {

using namespace traits;
namespace tl = tile_layout;

namespace detail {

/// 16 bytes per lane from gptr (per lane) to LDS at lds_wave_base + 16 * lane (lds_wave_base wave-uniform).
DEVICE void global_to_lds_16B(const void* gptr, const void* lds_wave_base) {
    const unsigned int lds_addr =
        __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds_wave_base)));
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_addr)
                 : "m0", "memory");
}

}  // namespace detail

/// Copy a global tile into a shared tile of the same shape, 1 KiB per instruction, the instructions dealt in
/// contiguous runs to the wavefronts of WarpLayout. Requirements (checked at compile time): 2-byte elements; the
/// shared tile is a whole allocation (pitch == line length, origin (0, 0)) whose lines divide 1 KiB; the tile is a
/// whole number of 1 KiB pieces per wavefront. Same call shape as GlobalToSharedLoader.
template <typename Shared_, typename WarpLayout_>
struct GlobalToSharedDirectLoader {
    using Shared = Shared_;
    using DType = typename Shared::DType;
    using WarpLayout = WarpLayout_;

    static constexpr int kWaves = tl::get_numel<WarpLayout>;
    static constexpr int kLineBytes = Shared::kLineLen * int(sizeof(DType));
    static constexpr int kTileBytes = Shared::kLines * kLineBytes;
    static constexpr int kLinesPerLoad = 1024 / kLineBytes;
    static constexpr int kLoads = kTileBytes / 1024;          // instructions per tile
    static constexpr int kLoadsPerWave = kLoads / kWaves;
    static constexpr int kPiecesPerLine = kLineBytes / 16;    // 16-byte pieces
    static constexpr int kPieceElems = 16 / int(sizeof(DType));

    static_assert(sizeof(DType) == 2, "direct-to-LDS loads are set up for 2-byte elements");
    static_assert(Shared::kPitch == Shared::kLineLen, "the shared tile must be a whole allocation, not a sub-tile");
    static_assert(kLineBytes >= 16 && 1024 % kLineBytes == 0, "a line must be 16 ... 1024 bytes and divide 1 KiB");
    static_assert(kTileBytes % (1024 * kWaves) == 0, "every wavefront must get a whole number of 1 KiB pieces");

    template <typename Global>
    DEVICE void operator()(const Global& src, Shared& dst) {
        static_assert(Global::kRows == Shared::kRows && Global::kCols == Shared::kCols,
                      "Global and shared memory tiles must have the same shape.");
        static_assert(Global::kType == Shared::kType, "Global and shared memory tiles must have the same layout.");
        constexpr int kGlobalPitch = Shared::kIsRowMajor ? Global::kRowStride : Global::kColStride;
        const int lane = lane_id();
        const int wave = __builtin_amdgcn_readfirstlane(wave_id());
        const int line_in_load = lane / kPiecesPerLine;
        const int piece = lane % kPiecesPerLine;  // physical 16-byte piece of the line
        const DType* g = src.data();
        const DType* s = dst.data();
#pragma unroll
        for (int j = 0; j < kLoadsPerWave; ++j) {
            const int t = wave * kLoadsPerWave + j;
            const int line = t * kLinesPerLoad + line_in_load;
            // the XOR swizzle is an involution: the logical element that lives at physical position p of a line is
            // apply(line, p)
            const int elem = Shared::kSwizzled ? Shared::Swizzle::apply(line, piece * kPieceElems) : piece * kPieceElems;
            detail::global_to_lds_16B(g + size_t(line) * kGlobalPitch + elem, s + t * (1024 / sizeof(DType)));
        }
    }
};

/// One direct-to-LDS load instruction, described but not yet issued: every lane fetches 16 bytes from base + offset
/// (a wave-uniform 64-bit base, which the instruction takes from scalar registers, plus a 32-bit byte offset per
/// lane: no 64-bit address arithmetic per load) and the 1 KiB lands at lds_addr + 16 * lane.
struct DirectLoad {
    unsigned int offset;    // per lane, bytes
    const void* base;       // wave-uniform
    unsigned int lds_addr;  // wave-uniform LDS byte address
};

/// Issue it (untracked by the compiler, like GlobalToSharedDirectLoader's loads). A kernel with one wavefront per SIMD
/// hands the description to compute::gemm_scheduled instead, which issues it behind a matrix instruction.
DEVICE void issue(const DirectLoad& load) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(load.offset), "s"(load.base),
                 "s"(load.lds_addr)
                 : "m0", "memory");
}

/// The copy of GlobalToSharedDirectLoader a piece at a time: piece j is the j-th of the kPieces load instructions this
/// wavefront contributes to a tile. The per-lane offsets (swizzle included) are computed once, at construction, for
/// global tiles whose lines are kGlobalPitch elements apart; piece(j, src, dst) then only combines them with the
/// tile's origin `src` (wave-uniform) and the stage `dst`. For kernels that spread the loads of the next tile over the
/// matrix instructions of the current one instead of issuing them in a burst (the address unit of a CU takes one
/// vector-memory instruction per ~14 cycles, and a wavefront that waits there issues nothing else).
/// kGlobalPitch_ == 0: the pitch is a run-time value, given to the constructor (a tile cut out of an operand whose
/// leading dimension is a run-time size, e.g. a column-major V of an attention layer: pitch = number of keys).
template <typename Shared_, typename WarpLayout_, const int kGlobalPitch_>
struct GlobalToSharedDirectPieces {
    using Shared = Shared_;
    using DType = typename Shared::DType;
    using Loader = GlobalToSharedDirectLoader<Shared_, WarpLayout_>;
    static constexpr int kPieces = Loader::kLoadsPerWave;
    static constexpr int kGlobalPitch = kGlobalPitch_;
    static_assert((long)Shared::kLines * kGlobalPitch * (long)sizeof(DType) < (1l << 32),
                  "a tile's lines are addressed with 32-bit byte offsets from its origin");

    DEVICE GlobalToSharedDirectPieces() : GlobalToSharedDirectPieces(kGlobalPitch_) {
        static_assert(kGlobalPitch_ > 0, "a run-time pitch goes to the other constructor");
    }
    DEVICE explicit GlobalToSharedDirectPieces(int global_pitch) {
        const int lane = lane_id();
        wave_ = __builtin_amdgcn_readfirstlane(wave_id());
        const int line_in_load = lane / Loader::kPiecesPerLine;
        const int piece = lane % Loader::kPiecesPerLine;  // physical 16-byte piece of the line
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
            const int line = (wave_ * kPieces + j) * Loader::kLinesPerLoad + line_in_load;
            const int elem = Shared::kSwizzled ? Shared::Swizzle::apply(line, piece * Loader::kPieceElems)
                                               : piece * Loader::kPieceElems;
            offset_[j] = (static_cast<unsigned int>(line) * static_cast<unsigned int>(global_pitch) + elem) *
                         static_cast<unsigned int>(sizeof(DType));
        }
    }

    /// Piece j of the copy of the global tile whose first element is at `src` into `dst`.
    DEVICE DirectLoad piece(int j, const DType* src, const Shared& dst) const {
        using lds_cptr = __attribute__((address_space(3))) const void*;
        const unsigned int lds = static_cast<unsigned int>(reinterpret_cast<uintptr_t>((lds_cptr)(dst.data()))) +
                                 static_cast<unsigned int>(wave_ * kPieces + j) * 1024u;
        return DirectLoad{offset_[j], src, static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(lds))};
    }

  private:
    unsigned int offset_[kPieces];
    int wave_;
};

}  // namespace tiledcuda::cell::copy
