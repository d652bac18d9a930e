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

}  // namespace tiledcuda::cell::copy
