// Architecture constants of the tile library for gfx950 (CDNA4).
//
// Plays the role of the reference's include/cell/traits/base.hpp:16-39, re-derived for
// 64-lane wavefronts and MFMA:
//   * a BaseTile is still 16x16 elements (so tile-count arithmetic written against
//     BaseTileShape<T>::kTileSize keeps working), but it is spread over 64 lanes, 4
//     elements per lane, instead of 32 lanes x 8 elements;
//   * lane l of a row-major BaseTile owns row (l % 16), columns 4*(l / 16) .. +3
//     (contiguous, one 64-bit access for f16, one 128-bit access for f32);
//     a column-major BaseTile is the transpose: column (l % 16), rows 4*(l / 16) .. +3;
//   * that distribution is exactly the operand layout of v_mfma_f32_16x16x16_f16, and two
//     BaseTiles adjacent along K form one operand of v_mfma_f32_16x16x32_f16 (the
//     contraction index may be permuted freely as long as A and B use the same
//     permutation); with the operands swapped the f32 result comes out in the same
//     row-major BaseTile distribution, so an accumulator can be converted to f16 and fed
//     back as the A operand of the next gemm without any cross-lane traffic.
#pragma once

#include "config.hpp"

#include <type_traits>

namespace tiledcuda::cell::traits {

template <typename Element>
concept BaseType =
    std::is_same_v<Element, float> || std::is_same_v<Element, __half> || std::is_same_v<Element, _Float16>;

template <typename Element>
concept HalfType = std::is_same_v<Element, __half> || std::is_same_v<Element, _Float16>;

/// Widest vector access and how many elements it carries.
template <typename Element>
struct TraitsBase {
    static constexpr int kAccessInBits = 128;
    static constexpr int kElmentBits = 8 * sizeof(Element);
    static constexpr int kNumPerAccess = kAccessInBits / kElmentBits;
};

template <typename Element>
    requires BaseType<Element>
struct BaseTileShape {
    using DType = Element;

    static constexpr int kTileSize = 16;
    static constexpr int kRows = kTileSize;
    static constexpr int kCols = kTileSize;
    static constexpr int kNumel = kRows * kCols;

    static constexpr int kLanes = kWaveSize;                 // 64
    static constexpr int kNumelPerThread = kNumel / kLanes;  // 4
    static constexpr int kRegsPerThread = sizeof(DType) * kNumelPerThread / sizeof(uint32_t);

    // Lane distribution: 16 lanes along the major index, 4 lane groups along the minor one,
    // each lane holding kVec contiguous minor elements.
    static constexpr int kLaneMajor = 16;
    static constexpr int kLaneGroups = kLanes / kLaneMajor;  // 4
    static constexpr int kVec = kNumelPerThread;             // 4

    // Each row (row-major) / column (column-major) of a BaseTile lives in this many lanes,
    // so a row reduction yields one value per lane per BaseTile row.
    static constexpr int kRowsPerLane = 1;

    // MFMA instruction shape fed by BaseTiles (f16 operands): two K-adjacent tiles per issue.
    static constexpr int kM = 16;
    static constexpr int kN = 16;
    static constexpr int kK = 32;
};

/// Index of this lane along the major dimension of a BaseTile (row of a row-major tile).
DEVICE int lane_major() { return lane_id() & 15; }
/// First minor index owned by this lane (column of a row-major tile).
DEVICE int lane_minor() { return (lane_id() >> 4) << 2; }

}  // namespace tiledcuda::cell::traits
