// Compile-time 2-D layouts and the LDS swizzle.
//
// MatrixLayout / RowMajor / ColMajor and the free-standing queries keep the names and
// meaning of the reference's include/types/layout.hpp:26-53,275-296. The shared-memory
// layout is new: the reference stores every 16x16 BaseTile contiguously and applies
// CuTe Swizzle<2,3,3> inside it (layout.hpp:58-206) to serve ldmatrix; here a shared tile
// is a plain pitched 2-D array whose 4-element chunks are XOR-permuted within each line so
// that the per-lane 64-bit (f16) / 128-bit (f32) LDS accesses of a wavefront fall on
// distinct banks (64 banks x 4 B on gfx950).
#pragma once

#include "cell/traits/base.hpp"
#include "config.hpp"

#include <cstddef>

namespace tiledcuda::cell {

namespace tile_layout {

enum class Layout {
    kRowMajor = 0,
    kColMajor = 1,
    kSwizzledRowMajor = 2,
    kSwizzledColMajor = 3
};

HOST_DEVICE constexpr const char* layout_type_to_str(Layout type) {
    switch (type) {
        case Layout::kRowMajor: return "RowMajor";
        case Layout::kColMajor: return "ColMajor";
        case Layout::kSwizzledRowMajor: return "SwizzledRowMajor";
        case Layout::kSwizzledColMajor: return "SwizzledColMajor";
    }
    return "Unknown";
}

template <const int kRows_, const int kCols_, const int kRowStride_, const int kColStride_>
struct MatrixLayout {
    static constexpr int kRows = kRows_;
    static constexpr int kCols = kCols_;

    static constexpr int kRowStride = kRowStride_;
    static constexpr int kColStride = kColStride_;

    static constexpr int kNumel = kRows * kCols;

    // A layout whose column stride is 1 counts as row-major (so ColMajor<1, 1> does too).
    static constexpr Layout kType = kColStride == 1 ? Layout::kRowMajor : Layout::kColMajor;

    HOST_DEVICE constexpr int operator()(int i, int j) const { return i * kRowStride + j * kColStride; }
};

// The last dimension is contiguous.
template <const int kRow, const int kCol, const int kStride = kCol>
using RowMajor = MatrixLayout<kRow, kCol, kStride, 1>;

// The first dimension is contiguous.
template <const int kRow, const int kCol, const int kStride = kRow>
using ColMajor = MatrixLayout<kRow, kCol, 1, kStride>;

template <typename Layout>
static constexpr size_t num_rows = Layout::kRows;

template <typename Layout>
static constexpr size_t num_cols = Layout::kCols;

template <typename Layout>
static constexpr size_t row_stride = Layout::kRowStride;

template <typename Layout>
static constexpr size_t col_stride = Layout::kColStride;

template <typename Layout>
static constexpr size_t get_numel = Layout::kNumel;

template <typename Layout_>
static constexpr Layout layout_type = Layout_::kType;

template <const int kShape1, const int kShape2, const int kStride1, const int kStride2>
HOST_DEVICE constexpr auto make_tile_layout() {
    return MatrixLayout<kShape1, kShape2, kStride1, kStride2>{};
}

namespace detail {
HOST_DEVICE constexpr int cmax(int a, int b) { return a > b ? a : b; }
HOST_DEVICE constexpr int cmin(int a, int b) { return a < b ? a : b; }
// largest power of two dividing x (x > 0)
HOST_DEVICE constexpr int pow2_divisor(int x) { return x & (-x); }
}  // namespace detail

/// XOR permutation of the 4-element chunks of one line (row of a row-major tile, column of a
/// column-major one) of a pitched LDS tile.
///
/// One wavefront access touches 16 consecutive lines at one or two chunk positions per
/// pass (a 64-bit access is served 32 lanes at a time, a 128-bit access 16 lanes at a time,
/// 256 B = all 64 banks per pass). Lines whose start addresses coincide modulo 256 B would
/// collide, so their chunk index is XOR-ed with a per-line value. The XOR leaves bit 0 of
/// the chunk index of 2-byte elements alone, so a 16-byte global->LDS store of 8 halves
/// stays contiguous.
template <const int kPitch, const int kElemBytes>
struct LdsSwizzle {
    static constexpr int kChunk = 4;
    static constexpr int kChunkBytes = kChunk * kElemBytes;
    static constexpr int kChunksPerLine = kPitch / kChunk;
    static constexpr int kWindowChunks = 256 / kChunkBytes;
    static constexpr int kShift = kWindowChunks >= 32 ? 1 : 0;
    static constexpr int kLinesPerWindow = detail::cmin(16, detail::cmax(1, kWindowChunks / kChunksPerLine));
    static constexpr int kNumSwz =
        detail::cmax(1, detail::cmin(16 / kLinesPerWindow, detail::pow2_divisor(kChunksPerLine) >> kShift));

    static_assert(kPitch % kChunk == 0, "the pitch of a shared tile must be a multiple of 4 elements");
    /// apply(line + kLinePeriod, elem) == apply(line, elem): a view that starts a multiple of this many lines into
    /// the tile sees the same permutation (so its line offset is purely additive).
    static constexpr int kLinePeriod = kLinesPerWindow * kNumSwz;

    /// Position, within its line, of logical element `elem` of line `line`.
    HOST_DEVICE static constexpr int apply(int line, int elem) {
        const int chunk = elem >> 2;
        const int s = ((line / kLinesPerWindow) & (kNumSwz - 1)) << kShift;
        return ((chunk ^ s) << 2) | (elem & 3);
    }
};

/// XOR permutation for tiles of 2-byte elements that are read ACROSS their lines with the transposing LDS read
/// (ds_read_b64_tr_b16: the B operand of a matrix instruction out of a row-major tile, e.g. V [keys, head_dim] of an
/// attention layer). One pass of such a read serves two 16-lane groups, each of which fetches 4 consecutive lines x 32
/// bytes. kLines = 4: the two groups sit on adjacent 32-byte units of the same 4 lines (operand tiles 32 wide). Lines of
/// 256 bytes all start on bank 0, so the 4 lines are spread with unit ^= 2 * (line % 4); lines of 128 bytes alternate
/// between the two halves of the banks, so only lines 2 apart collide: unit ^= line & 2. kLines = 8 (lines of 256
/// bytes): the two groups sit on the same 32-byte unit of 8 consecutive lines (operand tiles 16 wide, each lane group
/// 4 lines further down): unit ^= line % 8; with lines of 128 bytes, whose 4 units alternate between the halves of the
/// banks by themselves, unit ^= (line / 2) % 4. 32-byte units (and with them the 16-byte pieces of direct-to-LDS
/// loads) stay contiguous.
template <const int kPitch, const int kElemBytes, const int kLines = 4>
struct LdsSwizzleTr {
    static_assert(kElemBytes == 2 && (kPitch == 128 || kPitch == 64),
                  "written for lines of 128 or 256 bytes of 2-byte elements");
    static_assert(kLines == 4 || kLines == 8, "4 or 8 lines per pass");
    static constexpr int kUnit = 16;  // elements per 32-byte unit
    static constexpr int kLinePeriod = kLines;

    HOST_DEVICE static constexpr int apply(int line, int elem) {
        const int s = kLines == 8 ? (kPitch == 128 ? (line & 7) : ((line >> 1) & 3))
                                  : kPitch == 128 ? ((line & 3) << 1) : (line & 2);
        return (((elem / kUnit) ^ s) * kUnit) | (elem % kUnit);
    }
};

/// XOR permutation for tiles of 2-byte elements with 256-byte lines whose lines are read 16 at a time in DEALT order
/// (copy::SharedToRegPieces<..., kDealtLines = true>): one pass of a 16-byte-per-lane read touches lines
/// 8 q + 4 h + r (q, r = 0..3; h fixed), which the standard permutation (unit ^= line % 16) would send to only 8 different
/// places. Here the 16-byte unit is XORed with 4 q + r: bits 3, 4 and 0, 1 of the line.
template <const int kPitch, const int kElemBytes>
struct LdsSwizzleDealt {
    static_assert(kElemBytes == 2 && kPitch == 128, "written for lines of 256 bytes of 2-byte elements");
    static constexpr int kUnit = 8;  // elements per 16-byte unit
    static constexpr int kLinePeriod = 32;

    HOST_DEVICE static constexpr int apply(int line, int elem) {
        const int s = (((line >> 3) & 3) << 2) | (line & 3);
        return (((elem / kUnit) ^ s) * kUnit) | (elem % kUnit);
    }
};

}  // namespace tile_layout
}  // namespace tiledcuda::cell
