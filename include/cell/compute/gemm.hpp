// Tile-level gemm(a, b, c): c(i, j) += sum_k a(i, k) * b(k, j) over 16x16 BaseTiles,
// f16 x f16 -> f32. Same entry point and operand types as the reference's
// include/cell/compute/gemm.hpp:18-88, where each 16x16x16 step is two
// mma.sync.m16n8k16; here two K-adjacent BaseTiles of A and of B form the operands of one
// v_mfma_f32_16x16x32_f16 (an odd trailing K tile uses v_mfma_f32_16x16x16_f16).
//
// The operands are passed to the instruction swapped (B's share as the first operand):
// the instruction then produces C^T in its native accumulator distribution, which is C in
// the row-major BaseTile distribution (lane l: row l % 16, columns 4 * (l / 16) .. +3).
//
// With MFMA-shaped operand tiles (types/mfma_tile.hpp) every (i, j, k) step is exactly one instruction:
//   A 16 x 32, B 32 x 16, C 16 x 16 BaseTile  ->  v_mfma_f32_16x16x32_f16
//   A 32 x 16, B 16 x 32, C 32 x 32           ->  v_mfma_f32_32x32x16_f16
// (operands swapped as above, so the accumulator holds runs of consecutive columns of a row of C).
#pragma once

#include <type_traits>
#include <utility>

#include "cell/traits/base.hpp"
#include "types/layout.hpp"
#include "types/mfma_tile.hpp"
#include "types/tile_shape.hpp"

namespace tiledcuda::cell::compute {
namespace tl = tile_layout;

namespace detail {

template <typename RegTileA, typename RegTileB, typename RegTileC>
struct Gemm {
    using InTypeA = typename RegTileA::DType::DType;
    using InTypeB = typename RegTileB::DType::DType;
    using OutType = typename RegTileC::DType::DType;

    using BaseShape = traits::BaseTileShape<InTypeA>;

    static_assert(traits::HalfType<InTypeA>, "This GEMM supports only half-precision input elements.");
    static_assert(std::is_same_v<OutType, float>, "The output type must be float.");
    static_assert(std::is_same_v<InTypeA, InTypeB>, "Mismatched data type for operand A and B.");
    static_assert(RegTileB::kRows == RegTileA::kCols, "Mismatched k-dimension for operand A and B.");
    static_assert(RegTileA::kType == tl::Layout::kRowMajor, "Operand A must be made of row-major BaseTiles.");
    static_assert(RegTileB::kType == tl::Layout::kColMajor, "Operand B must be made of column-major BaseTiles.");
    static_assert(RegTileC::kType == tl::Layout::kRowMajor, "The accumulator must be made of row-major BaseTiles.");

    static constexpr int kMs = RegTileA::kRows;
    static constexpr int kNs = RegTileB::kCols;
    static constexpr int kKs = RegTileA::kCols;
    static_assert(kMs && kNs && kKs, "Invalid tile shapes for GEMM.");
    static_assert(RegTileC::kRows == kMs && RegTileC::kCols == kNs, "Mismatched accumulator shape.");

    DEVICE void operator()(const RegTileA& a, const RegTileB& b, RegTileC& c) {
#pragma unroll
        for (int k = 0; k + 1 < kKs; k += 2) {
#pragma unroll
            for (int i = 0; i < kMs; ++i) {
#pragma unroll
                for (int j = 0; j < kNs; ++j)
                    mfma_k32(a(i, k).data(), a(i, k + 1).data(), b(k, j).data(), b(k + 1, j).data(),
                             c(i, j).mutable_data());
            }
        }
        if constexpr (kKs % 2 == 1) {
#pragma unroll
            for (int i = 0; i < kMs; ++i) {
#pragma unroll
                for (int j = 0; j < kNs; ++j)
                    mfma_k16(a(i, kKs - 1).data(), b(kKs - 1, j).data(), c(i, j).mutable_data());
            }
        }
    }

  private:
    DEVICE static f16x4 load4(const InTypeA* p) {
        f16x4 v;
        __builtin_memcpy(&v, p, sizeof(v));
        return v;
    }

    DEVICE static void mfma_k32(const InTypeA* a0, const InTypeA* a1, const InTypeB* b0, const InTypeB* b1,
                                OutType* c) {
        const f16x4 al = load4(a0), ah = load4(a1), bl = load4(b0), bh = load4(b1);
        const f16x8 av = __builtin_shufflevector(al, ah, 0, 1, 2, 3, 4, 5, 6, 7);
        const f16x8 bv = __builtin_shufflevector(bl, bh, 0, 1, 2, 3, 4, 5, 6, 7);
        f32x4 acc;
        __builtin_memcpy(&acc, c, sizeof(acc));
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bv, av, acc, 0, 0, 0);
        __builtin_memcpy(c, &acc, sizeof(acc));
    }

    DEVICE static void mfma_k16(const InTypeA* a, const InTypeB* b, OutType* c) {
        const f16x4 av = load4(a), bv = load4(b);
        f32x4 acc;
        __builtin_memcpy(&acc, c, sizeof(acc));
        acc = __builtin_amdgcn_mfma_f32_16x16x16f16(bv, av, acc, 0, 0, 0);
        __builtin_memcpy(c, &acc, sizeof(acc));
    }
};

template <typename T>
struct IsMfmaTile : std::false_type {};
template <typename E, const int kR, const int kC, const tl::Layout kT>
struct IsMfmaTile<MfmaTile<E, kR, kC, kT>> : std::true_type {};

/// gemm over MFMA-shaped operand tiles: one matrix instruction per (i, j, k).
template <typename RegTileA, typename RegTileB, typename RegTileC>
struct GemmMfmaTiles {
    using TileA = typename RegTileA::DType;
    using TileB = typename RegTileB::DType;
    using TileC = typename RegTileC::DType;
    using InType = typename TileA::DType;

    static_assert(traits::HalfType<InType> && std::is_same_v<InType, typename TileB::DType>,
                  "This GEMM supports only half-precision input elements of one type.");
    static_assert(std::is_same_v<typename TileC::DType, float>, "The output type must be float.");
    static_assert(TileA::kType == tl::Layout::kRowMajor && TileB::kType == tl::Layout::kColMajor,
                  "Operand A must be made of row-major tiles, operand B of column-major tiles.");
    static constexpr bool k16 = TileA::kTileRows == 16 && TileA::kTileCols == 32;
    static constexpr bool k32 = TileA::kTileRows == 32 && TileA::kTileCols == 16;
    static_assert(k16 || k32, "operand A must be a 16 x 32 or a 32 x 16 tile");
    static_assert(TileB::kTileRows == TileA::kTileCols && TileB::kTileCols == TileA::kTileRows,
                  "operand B must be the 32 x 16 / 16 x 32 counterpart of operand A");
    static_assert(traits::TileGeometry<TileC>::kRows == TileA::kTileRows &&
                      traits::TileGeometry<TileC>::kCols == TileB::kTileCols &&
                      traits::TileGeometry<TileC>::kRowMajor,
                  "the accumulator must be the row-major 16 x 16 BaseTile or the 32 x 32 MFMA tile");

    static constexpr int kMs = RegTileA::kRows, kNs = RegTileB::kCols, kKs = RegTileA::kCols;
    static_assert(RegTileB::kRows == kKs, "Mismatched k-dimension for operand A and B.");
    static_assert(RegTileC::kRows == kMs && RegTileC::kCols == kNs, "Mismatched accumulator shape.");

    DEVICE void operator()(const RegTileA& a, const RegTileB& b, RegTileC& c) {
#pragma unroll
        for (int k = 0; k < kKs; ++k) {
#pragma unroll
            for (int i = 0; i < kMs; ++i) {
#pragma unroll
                for (int j = 0; j < kNs; ++j) {
                    f16x8 av, bv;
                    __builtin_memcpy(&av, a(i, k).data(), sizeof(av));
                    __builtin_memcpy(&bv, b(k, j).data(), sizeof(bv));
                    if constexpr (k16) {
                        f32x4 acc;
                        __builtin_memcpy(&acc, c(i, j).data(), sizeof(acc));
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bv, av, acc, 0, 0, 0);
                        __builtin_memcpy(c(i, j).mutable_data(), &acc, sizeof(acc));
                    } else {
                        f32x16 acc;
                        __builtin_memcpy(&acc, c(i, j).data(), sizeof(acc));
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(bv, av, acc, 0, 0, 0);
                        __builtin_memcpy(c(i, j).mutable_data(), &acc, sizeof(acc));
                    }
                }
            }
        }
    }
};

}  // namespace detail

/// Which register file an accumulator or operand of a scheduled product is pinned in. A wavefront that runs alone on
/// its SIMD has 256 VGPRs and 256 AGPRs; the matrix instructions take their accumulator and either operand from both.
enum class RegFile { kVgpr = 0, kAgpr = 1 };

/// The matrix instructions of a tile product c += a b, one at a time, for kernels that place every instruction
/// themselves (one wavefront per SIMD: nothing else feeds the matrix pipe while that wavefront does something else,
/// so where its LDS reads, global loads and vector-ALU work sit relative to its matrix instructions decides the
/// kernel's speed). at<i, j, k>(a, b, c) issues c(i, j) += a(i, k) b(k, j) as inline assembly, with the accumulator
/// tile constrained to kAccFile and the A tile to kAFile (left alone, the compiler moves large accumulator sets through
/// VGPRs and spills); the statements are volatile, so they stay in the order written. Operand tiles: 16 x 32 / 32 x 16
/// (v_mfma_f32_16x16x32_f16, accumulator of 16 x 16 BaseTiles) or 32 x 16 / 16 x 32 (v_mfma_f32_32x32x16_f16,
/// 32 x 32 accumulator tiles) of f16; the sums are those of gemm(a, b, c) bit for bit.
/// The compiler does not know these statements are matrix instructions and inserts none of the wait states their
/// results need before other instructions read them: keep every such read at least two matrix instructions behind the
/// write, or call settle_accumulators(c) first; and compile the kernel so that c can stay where it is between the
/// calls (__launch_bounds__ of one wavefront per SIMD when the pinned tiles need more than 256 registers).
/// The same holds in the other direction: a vector-ALU write to a register (clearing an accumulator, converting an
/// operand) DIRECTLY in front of the matrix instruction that reads it is not waited for either - observed on gfx950: the
/// instruction took the register's previous contents as its C operand. Write such registers a few instructions ahead
/// (clear_pinned / pin_tiles at the point where the tile is set up, not in front of the product).
template <typename RegTileA, typename RegTileB, typename RegTileC, const RegFile kAccFile = RegFile::kAgpr,
          const RegFile kAFile = RegFile::kVgpr>
struct ScheduledGemm {
    using G = detail::GemmMfmaTiles<RegTileA, RegTileB, RegTileC>;
    static constexpr int kMs = G::kMs, kNs = G::kNs, kKs = G::kKs;
    static constexpr int kCount = kMs * kNs * kKs;
    using Acc = std::conditional_t<G::k16, f32x4, f32x16>;

#define TCU_SCHEDULED_MFMA(ACC, AOP)                                                                              \
    if constexpr (G::k16)                                                                                         \
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+" ACC(acc) : "v"(bv), AOP(av));               \
    else                                                                                                          \
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+" ACC(acc) : "v"(bv), AOP(av))
#define TCU_SCHEDULED_MFMA_LOAD(ACC, AOP)                                                                         \
    if constexpr (G::k16)                                                                                         \
        asm volatile("s_mov_b32 m0, %5\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %3, %4" \
                     : "+" ACC(acc)                                                                               \
                     : "v"(bv), AOP(av), "v"(load.offset), "s"(load.base), "s"(load.lds_addr)                    \
                     : "m0", "memory");                                                                           \
    else                                                                                                          \
        asm volatile("s_mov_b32 m0, %5\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %3, %4" \
                     : "+" ACC(acc)                                                                               \
                     : "v"(bv), AOP(av), "v"(load.offset), "s"(load.base), "s"(load.lds_addr)                    \
                     : "m0", "memory")
#define TCU_SCHEDULED_MFMA_FROM(ACC, AOP)                                                                         \
    if constexpr (G::k16)                                                                                         \
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %3" : "=&" ACC(acc) : "v"(bv), AOP(av), "v"(from));   \
    else                                                                                                          \
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&" ACC(acc) : "v"(bv), AOP(av), "v"(from))
#define TCU_SCHEDULED_DISPATCH(MACRO)                                                 \
    if constexpr (kAccFile == RegFile::kAgpr && kAFile == RegFile::kVgpr) {           \
        MACRO("a", "v");                                                              \
    } else if constexpr (kAccFile == RegFile::kAgpr && kAFile == RegFile::kAgpr) {    \
        MACRO("a", "a");                                                              \
    } else if constexpr (kAccFile == RegFile::kVgpr && kAFile == RegFile::kVgpr) {    \
        MACRO("v", "v");                                                              \
    } else {                                                                          \
        MACRO("v", "a");                                                              \
    }

    /// c(kI, kJ) += a(kI, kK) b(kK, kJ).
    template <int kI, int kJ, int kK>
    DEVICE static void at(const RegTileA& a, const RegTileB& b, RegTileC& c) {
        f16x8 av, bv;
        Acc acc;
        __builtin_memcpy(&av, a(kI, kK).data(), sizeof(av));
        __builtin_memcpy(&bv, b(kK, kJ).data(), sizeof(bv));
        __builtin_memcpy(&acc, c(kI, kJ).data(), sizeof(acc));
        TCU_SCHEDULED_DISPATCH(TCU_SCHEDULED_MFMA)
        __builtin_memcpy(c(kI, kJ).mutable_data(), &acc, sizeof(acc));
    }

    /// The same, followed in the same statement by a direct-to-LDS load (a copy::DirectLoad): m0 is written before the
    /// matrix instruction, which thereby is the wait state the load needs after that write.
    template <int kI, int kJ, int kK, typename Load>
    DEVICE static void at(const RegTileA& a, const RegTileB& b, RegTileC& c, const Load& load) {
        f16x8 av, bv;
        Acc acc;
        __builtin_memcpy(&av, a(kI, kK).data(), sizeof(av));
        __builtin_memcpy(&bv, b(kK, kJ).data(), sizeof(bv));
        __builtin_memcpy(&acc, c(kI, kJ).data(), sizeof(acc));
        TCU_SCHEDULED_DISPATCH(TCU_SCHEDULED_MFMA_LOAD)
        __builtin_memcpy(c(kI, kJ).mutable_data(), &acc, sizeof(acc));
    }

    /// c(kI, kJ) = a(kI, kK) b(kK, kJ) + init: the first instruction of a product whose sums start from another tile
    /// (held in VGPRs) instead of from c's old contents, e.g. scores accumulated from minus the row maximum.
    template <int kI, int kJ, int kK, typename TileInit>
    DEVICE static void at_from(const RegTileA& a, const RegTileB& b, RegTileC& c, const TileInit& init) {
        f16x8 av, bv;
        Acc acc, from;
        static_assert(sizeof(TileInit) == sizeof(Acc), "the initial tile must have the accumulator tile's shape");
        __builtin_memcpy(&av, a(kI, kK).data(), sizeof(av));
        __builtin_memcpy(&bv, b(kK, kJ).data(), sizeof(bv));
        __builtin_memcpy(&from, init.data(), sizeof(from));
        TCU_SCHEDULED_DISPATCH(TCU_SCHEDULED_MFMA_FROM)
        __builtin_memcpy(c(kI, kJ).mutable_data(), &acc, sizeof(acc));
    }
#undef TCU_SCHEDULED_DISPATCH
#undef TCU_SCHEDULED_MFMA_FROM
#undef TCU_SCHEDULED_MFMA_LOAD
#undef TCU_SCHEDULED_MFMA
};

/// The whole product c += a b through ScheduledGemm, in a fixed order, with a hook per instruction:
///   * the instructions go k-step by k-step, row of A tiles by row, the tiles of a row forwards in even rows and
///     backwards in odd ones, so that every instruction shares an operand with the one before it;
///   * before instruction number n = (k * kMs + i) * kNs + position-in-row the caller's hook is called with
///     std::integral_constant<int, n>: the place for the fragment reads of the next k-step (SharedToRegLoader::load_one)
///     - they are ordinary LDS reads, the compiler keeps them between the assembly statements they are written between;
///   * if the hook returns something (a copy::DirectLoad), that direct-to-LDS load is issued in the same assembly
///     statement as the instruction;
///   * if the hook has a member after(std::integral_constant<int, n>), it is called behind instruction n: the place
///     for small doses of vector-ALU work (one transcendental plus one or two plain instructions hide under a matrix
///     instruction of the same wavefront; larger groups cost their full issue time), e.g. a slice of a softmax.
/// Accumulators in AGPRs, operands in VGPRs. See ScheduledGemm for what the caller owes the accumulators
/// (settle_accumulators before any other read, __launch_bounds__ of one wavefront per SIMD).
template <typename RegTileA, typename RegTileB, typename RegTileC, typename Hook>
DEVICE void gemm_scheduled(const RegTileA& a, const RegTileB& b, RegTileC& c, Hook&& hook) {
    using S = ScheduledGemm<RegTileA, RegTileB, RegTileC>;
    constexpr int kMs = S::kMs, kNs = S::kNs;
    [&]<int... kIs>(std::integer_sequence<int, kIs...>) {
        (
            [&] {
                constexpr int n = kIs;
                constexpr int k = n / (kMs * kNs), i = n / kNs % kMs, pos = n % kNs;
                constexpr int j = (i & 1) ? kNs - 1 - pos : pos;
                using N = std::integral_constant<int, n>;
                using HookResult = decltype(hook(N{}));
                if constexpr (std::is_void_v<HookResult>) {
                    hook(N{});
                    S::template at<i, j, k>(a, b, c);
                } else {
                    const HookResult load = hook(N{});
                    S::template at<i, j, k>(a, b, c, load);
                }
                if constexpr (requires { hook.after(N{}); }) hook.after(N{});
            }(),
            ...);
    }(std::make_integer_sequence<int, S::kCount>{});
}

/// Pin every tile of a register tile in the given register file as of here (an empty statement the compiler must
/// satisfy): operand tiles that a ScheduledGemm takes from AGPRs, or values that must not be rematerialised later.
template <const RegFile kFile, typename Reg>
DEVICE void pin_tiles(Reg& t) {
    [&]<int... kIs>(std::integer_sequence<int, kIs...>) {
        (
            [&] {
                using Tile = typename Reg::DType;
                using Vec = std::conditional_t<sizeof(Tile) == 16, u32x4, u32x16>;
                static_assert(sizeof(Tile) == sizeof(Vec), "tiles of 4 or 16 registers per lane");
                auto& tile = t(kIs / Reg::kCols, kIs % Reg::kCols);
                Vec v;
                __builtin_memcpy(&v, tile.data(), sizeof(v));
                if constexpr (kFile == RegFile::kAgpr) asm volatile("" : "+a"(v));
                else asm volatile("" : "+v"(v));
                __builtin_memcpy(tile.mutable_data(), &v, sizeof(v));
            }(),
            ...);
    }(std::make_integer_sequence<int, Reg::kRows * Reg::kCols>{});
}

/// Clear an accumulator tile and place it in AGPRs, where gemm_scheduled keeps it (the statements also keep the
/// compiler from sinking the clears to the first use, where nothing would hide them).
template <typename RegTileC>
DEVICE void clear_pinned(RegTileC& c) {
    [&]<int... kIs>(std::integer_sequence<int, kIs...>) {
        (
            [&] {
                using Acc = std::conditional_t<sizeof(typename RegTileC::DType) == sizeof(f32x4), f32x4, f32x16>;
                Acc acc;
#pragma unroll
                for (int e = 0; e < int(sizeof(Acc) / sizeof(float)); ++e) acc[e] = 0.f;
                asm volatile("" : "+a"(acc));
                __builtin_memcpy(c(kIs / RegTileC::kCols, kIs % RegTileC::kCols).mutable_data(), &acc, sizeof(acc));
            }(),
            ...);
    }(std::make_integer_sequence<int, RegTileC::kRows * RegTileC::kCols>{});
}

/// After the last gemm_scheduled on c and before anything else reads c: one wait that covers the longest requirement
/// of a matrix instruction's result (19 issue slots), then every tile passes through a statement of its own (volatile
/// statements keep their order, so each of those comes after the wait).
template <typename RegTileC>
DEVICE void settle_accumulators(RegTileC& c) {
    asm volatile("s_nop 15\n\ts_nop 3");
    [&]<int... kIs>(std::integer_sequence<int, kIs...>) {
        (
            [&] {
                auto& tile = c(kIs / RegTileC::kCols, kIs % RegTileC::kCols);
                using Acc = std::conditional_t<sizeof(typename RegTileC::DType) == sizeof(f32x4), f32x4, f32x16>;
                Acc acc;
                __builtin_memcpy(&acc, tile.data(), sizeof(acc));
                asm volatile("" : "+a"(acc));
                __builtin_memcpy(tile.mutable_data(), &acc, sizeof(acc));
            }(),
            ...);
    }(std::make_integer_sequence<int, RegTileC::kRows * RegTileC::kCols>{});
}

template <typename RegTileA, typename RegTileB, typename RegTileC>
DEVICE void gemm(const RegTileA& a, const RegTileB& b, RegTileC& c) {
    if constexpr (detail::IsMfmaTile<typename RegTileA::DType>::value) {
        detail::GemmMfmaTiles<RegTileA, RegTileB, RegTileC> gemm;
        gemm(a, b, c);
    } else {
        detail::Gemm<RegTileA, RegTileB, RegTileC> gemm;
        gemm(a, b, c);
    }
}

}  // namespace tiledcuda::cell::compute
