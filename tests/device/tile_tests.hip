// Device-side unit tests of the tile primitives, exported through a small C table so that
// pytest can drive them (one process, torch-owned device buffers).
//
// The cases restate the reference's C++ unit tests with the same shapes and warp layouts:
//   g2s round trip          tests/cpp/cell/test_g2s_load.cu:118-144
//   swizzled vs plain load  tests/cpp/cell/test_swizzled_copy.cu:399-450 (strengthened: the
//                           register tiles are written back and must equal the source)
//   store round trip        tests/cpp/cell/test_swizzled_copy.cu:452-499
//   g2r / r2g               tests/cpp/cell/test_g2r_copy.cu (which only prints)
//   tile gemm               tests/cpp/cell/test_gemm.cu:306-351
//   reduce / broadcast      tests/cpp/cell/test_reduce.cu, test_broadcast.cu (which only print)
//   softmax                 tests/cpp/cell/test_softmax.cu:117-163
// The CDNA4 data path of the library has the same kinds of cases: direct-to-LDS loads into a ring stage must
// reproduce the source, MFMA-shaped operand tiles read with ds_read_b128 and with the transposing read must
// reproduce the source (swizzled and plain), and gemm() on those tiles must match the oracle for both instruction
// shapes, including a B operand stored row-major and transposed on the way to registers.
// Every kernel is launched with one workgroup; the host side checks results against the
// CPU oracle or against the identity.
#include "cell/mod.hpp"
#include "types/mod.hpp"
#include "util/static_for.hpp"

#include <string>
#include <utility>
#include <vector>

using namespace tiledcuda;
using namespace tiledcuda::cell;
using namespace tiledcuda::cell::copy;
namespace tl = tiledcuda::cell::tile_layout;

namespace {

template <bool kRowMajor, int kRows, int kCols>
using LayoutOf = std::conditional_t<kRowMajor, tl::RowMajor<kRows, kCols>, tl::ColMajor<kRows, kCols>>;

// ------------------------------------------------------------------ global -> shared -> global
template <typename Element, bool kRowMajor, int kRows, int kCols, typename WarpLayout, bool kSwizzled, bool kStream = false>
__global__ void __launch_bounds__(512) k_g2s_roundtrip(const Element* src, Element* dst) {
    extern __shared__ __align__(16) unsigned char buf[];
    auto* smem = reinterpret_cast<Element*>(buf);
    using Layout = LayoutOf<kRowMajor, kRows, kCols>;
    using Global = GlobalTile<Element, Layout>;
    using Shared = SharedTile<Element, Layout, kSwizzled>;

    Global g_src(src);
    Global g_dst(dst);
    Shared s(smem);
    GlobalToSharedLoader<Shared, WarpLayout> loader;
    std::conditional_t<kStream, SharedToGlobalStreamStorer<Shared, WarpLayout>, SharedToGlobalStorer<Shared, WarpLayout>> storer;
    loader(g_src, s);
    __copy_async();
    __syncthreads();
    storer(s, g_dst);
}

// ------------------------------------------------------------------ global -> shared -> (iterator) -> reg -> global
// Operand-A style: row-major tile, chunks along the columns, RowReuseCont; every wavefront
// row's register tile is written back (wavefront columns hold copies, so only column 0 writes).
template <typename Element, int kRows, int kCols, int kChunk, typename WarpLayout, bool kSwizzled>
__global__ void __launch_bounds__(512) k_s2r_row_major(const Element* src, Element* dst) {
    extern __shared__ __align__(16) unsigned char buf[];
    auto* smem = reinterpret_cast<Element*>(buf);
    using Global = GlobalTile<Element, tl::RowMajor<kRows, kCols>>;
    using Shared = SharedTile<Element, tl::RowMajor<kRows, kCols>, kSwizzled>;
    using SIter = STileIterator<Shared, TileShape<kRows, kChunk>>;
    constexpr int kWR = tl::num_rows<WarpLayout>;
    constexpr int kMs = kRows / kWR / 16, kKs = kChunk / 16;
    using Reg = RegTile<BaseTileRowMajor<Element>, tl::RowMajor<kMs, kKs>>;

    Global g_src(src);
    Shared s(smem);
    GlobalToSharedLoader<Shared, WarpLayout> g2s;
    g2s(g_src, s);
    __copy_async();
    __syncthreads();

    SIter iter(smem);
    SharedToRegLoader<Reg, WarpLayout, WarpReuse::kRowReuseCont> s2r;
    using Base = warp::CopyBase<WarpLayout, WarpReuse::kRowReuseCont>;
    for (int k = 0; k < SIter::sc1; ++k) {
        Reg r;
        s2r(iter(k), r);
        if (Base::warp_col_id() == 0) {
            // write this wavefront-row's block back, BaseTile by BaseTile (wavefronts of one row hold copies)
            Element* block = dst + Base::warp_row_id() * (kRows / kWR) * kCols + k * kChunk;
#pragma unroll
            for (int i = 0; i < kMs; ++i)
#pragma unroll
                for (int j = 0; j < kKs; ++j)
                    copy::detail::move_base_tile<Element, const typename Reg::DType, kCols, 1, false>(
                        block + i * 16 * kCols + j * 16, r(i, j));
        }
    }
}

// Operand-B style: column-major tile, chunks along the rows, ColReuseCont.
template <typename Element, int kRows, int kCols, int kChunk, typename WarpLayout, bool kSwizzled>
__global__ void __launch_bounds__(512) k_s2r_col_major(const Element* src, Element* dst) {
    extern __shared__ __align__(16) unsigned char buf[];
    auto* smem = reinterpret_cast<Element*>(buf);
    using Global = GlobalTile<Element, tl::ColMajor<kRows, kCols>>;
    using Shared = SharedTile<Element, tl::ColMajor<kRows, kCols>, kSwizzled>;
    using SIter = STileIterator<Shared, TileShape<kChunk, kCols>>;
    constexpr int kWC = tl::num_cols<WarpLayout>;
    constexpr int kKs = kChunk / 16, kNs = kCols / kWC / 16;
    using Reg = RegTile<BaseTileColMajor<Element>, tl::ColMajor<kKs, kNs>>;

    Global g_src(src);
    Shared s(smem);
    GlobalToSharedLoader<Shared, WarpLayout> g2s;
    g2s(g_src, s);
    __copy_async();
    __syncthreads();

    SIter iter(smem);
    SharedToRegLoader<Reg, WarpLayout, WarpReuse::kColReuseCont> s2r;
    using Base = warp::CopyBase<WarpLayout, WarpReuse::kColReuseCont>;
    for (int k = 0; k < SIter::sc0; ++k) {
        Reg r;
        s2r(iter(k), r);
        if (Base::warp_row_id() == 0) {
            Element* block = dst + k * kChunk + Base::warp_col_id() * (kCols / kWC) * kRows;
#pragma unroll
            for (int i = 0; i < kKs; ++i)
#pragma unroll
                for (int j = 0; j < kNs; ++j)
                    copy::detail::move_base_tile<Element, const typename Reg::DType, 1, kRows, false>(
                        block + i * 16 + j * 16 * kRows, r(i, j));
        }
    }
}

// ------------------------------------------------------------------ global -> reg -> shared -> global
template <typename Element, bool kRowMajor, int kRows, int kCols, typename WarpLayout, bool kSwizzled>
__global__ void __launch_bounds__(512) k_store_roundtrip(const Element* src, Element* dst) {
    extern __shared__ __align__(16) unsigned char buf[];
    auto* smem = reinterpret_cast<Element*>(buf);
    using Layout = LayoutOf<kRowMajor, kRows, kCols>;
    using Global = GlobalTile<Element, Layout>;
    using Shared = SharedTile<Element, Layout, kSwizzled>;
    constexpr int kRs = kRows / tl::num_rows<WarpLayout> / 16, kCs = kCols / tl::num_cols<WarpLayout> / 16;
    using Base = std::conditional_t<kRowMajor, BaseTileRowMajor<Element>, BaseTileColMajor<Element>>;
    using Reg = RegTile<Base, LayoutOf<kRowMajor, kRs, kCs>>;

    Global g_src(src);
    Global g_dst(dst);
    Shared s(smem);
    Reg r;
    GlobalToRegLoader<Reg, WarpLayout, WarpReuse::kCont> g2r;
    RegToSharedStorer<Reg, WarpLayout> r2s;
    SharedToGlobalStorer<Shared, WarpLayout> s2g;
    g2r(g_src, r);
    r2s(r, s);
    __syncthreads();
    s2g(s, g_dst);
}

// ------------------------------------------------------------------ global -> reg -> global
template <typename Element, bool kGlobalRowMajor, bool kRegRowMajor, int kRows, int kCols, typename WarpLayout>
__global__ void __launch_bounds__(512) k_g2r_roundtrip(const Element* src, Element* dst) {
    using Layout = LayoutOf<kGlobalRowMajor, kRows, kCols>;
    using Global = GlobalTile<Element, Layout>;
    constexpr int kRs = kRows / tl::num_rows<WarpLayout> / 16, kCs = kCols / tl::num_cols<WarpLayout> / 16;
    using Base = std::conditional_t<kRegRowMajor, BaseTileRowMajor<Element>, BaseTileColMajor<Element>>;
    using Reg = RegTile<Base, LayoutOf<kRegRowMajor, kRs, kCs>>;
    Global g_src(src);
    Global g_dst(dst);
    Reg r;
    GlobalToRegLoader<Reg, WarpLayout, WarpReuse::kCont> g2r;
    RegToGlobalStorer<Global, Reg, WarpLayout> r2g;
    g2r(g_src, r);
    r2g(r, g_dst);
}

// ------------------------------------------------------------------ tile gemm through LDS
// C[kM, kN] f32 = A[kM, kK] (row-major) · B[kK, kN] (column-major), one workgroup.
template <int kM, int kN, int kK, typename WarpLayout, int kChunkK, bool kSwizzled>
__global__ void __launch_bounds__(512) k_tile_gemm(const __half* dA, const __half* dB, float* dC) {
    extern __shared__ __align__(16) unsigned char buf[];
    auto* sA_ptr = reinterpret_cast<__half*>(buf);
    auto* sB_ptr = sA_ptr + kM * kK;
    constexpr int kWR = tl::num_rows<WarpLayout>, kWC = tl::num_cols<WarpLayout>;

    using GlobalA = GlobalTile<__half, tl::RowMajor<kM, kK>>;
    using SharedA = SharedTile<__half, tl::RowMajor<kM, kK>, kSwizzled>;
    using SIterA = STileIterator<SharedA, TileShape<kM, kChunkK>>;
    using RegA = RegTile<BaseTileRowMajor<__half>, tl::RowMajor<kM / kWR / 16, kChunkK / 16>>;

    using GlobalB = GlobalTile<__half, tl::ColMajor<kK, kN>>;
    using SharedB = SharedTile<__half, tl::ColMajor<kK, kN>, kSwizzled>;
    using SIterB = STileIterator<SharedB, TileShape<kChunkK, kN>>;
    using RegB = RegTile<BaseTileColMajor<__half>, tl::ColMajor<kChunkK / 16, kN / kWC / 16>>;

    using GlobalC = GlobalTile<float, tl::RowMajor<kM, kN>>;
    using RegC = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kM / kWR / 16, kN / kWC / 16>>;

    GlobalA gA(dA);
    GlobalB gB(dB);
    SharedA sA(sA_ptr);
    SharedB sB(sB_ptr);
    GlobalToSharedLoader<SharedA, WarpLayout> g2s_a;
    GlobalToSharedLoader<SharedB, WarpLayout> g2s_b;
    g2s_a(gA, sA);
    g2s_b(gB, sB);
    __copy_async();
    __syncthreads();

    SIterA sAs(sA_ptr);
    SIterB sBs(sB_ptr);
    SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont> s2r_a;
    SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont> s2r_b;
    RegA rA;
    RegB rB;
    RegC acc;
    for (int k = 0; k < SIterA::sc1; ++k) {
        s2r_a(sAs(k), rA);
        s2r_b(sBs(k), rB);
        compute::gemm(rA, rB, acc);
    }
    GlobalC gC(dC);
    RegToGlobalStorer<GlobalC, RegC, WarpLayout> r2g;
    r2g(acc, gC);
}

// ------------------------------------------------------------------ CDNA4 data path
// global -> (direct-to-LDS, stage kStage of a ring of 3) -> global
template <bool kRowMajor, int kRows, int kCols, typename WarpLayout, bool kSwizzled, bool kPieces = false>
__global__ void __launch_bounds__(512) k_direct_ring_roundtrip(const __half* src, __half* dst) {
    extern __shared__ __align__(1024) unsigned char buf[];
    using Layout = LayoutOf<kRowMajor, kRows, kCols>;
    using Global = GlobalTile<__half, Layout>;
    using Shared = SharedTile<__half, Layout, kSwizzled>;
    using Ring = SharedRing<Shared, 3>;
    Ring ring(reinterpret_cast<__half*>(buf));
    Global g_src(src);
    Global g_dst(dst);
    GlobalToSharedDirectLoader<Shared, WarpLayout> loader;
    SharedToGlobalStorer<Shared, WarpLayout> storer;
    auto stage = ring[Ring::next(0)];
    if constexpr (kPieces) {
        // the same copy, a load instruction at a time
        using Pieces = GlobalToSharedDirectPieces<Shared, WarpLayout, kRowMajor ? Global::kRowStride : Global::kColStride>;
        Pieces pieces;
        for (int j = Pieces::kPieces - 1; j >= 0; --j) issue(pieces.piece(j, g_src.data(), stage));
    } else {
        loader(g_src, stage);
    }
    wait_group_and_barrier<0>();
    storer(stage, g_dst);
}

// shared -> MFMA-shaped operand tiles -> global. kTileMajor x kTileMinor: 16 x 32 or 32 x 16 (major = rows of a
// row-major operand, columns of a column-major one).
template <bool kRowMajor, int kRows, int kCols, int kChunk, typename WarpLayout, bool kSwizzled, int kTileMajor>
__global__ void __launch_bounds__(512) k_s2r_mfma_tiles(const __half* src, __half* dst) {
    extern __shared__ __align__(1024) unsigned char buf[];
    auto* smem = reinterpret_cast<__half*>(buf);
    constexpr int kTileMinor = 512 / kTileMajor;
    using Layout = LayoutOf<kRowMajor, kRows, kCols>;
    using Global = GlobalTile<__half, Layout>;
    using Shared = SharedTile<__half, Layout, kSwizzled>;
    Global g_src(src);
    Shared s(smem);
    GlobalToSharedLoader<Shared, WarpLayout> g2s;
    g2s(g_src, s);
    __copy_async();
    __syncthreads();
    if constexpr (kRowMajor) {
        using SIter = STileIterator<Shared, TileShape<kRows, kChunk>>;
        constexpr int kWR = tl::num_rows<WarpLayout>;
        using Tile = MfmaTile<__half, kTileMajor, kTileMinor, tl::Layout::kRowMajor>;
        using Reg = RegTile<Tile, tl::RowMajor<kRows / kWR / kTileMajor, kChunk / kTileMinor>>;
        SharedToRegLoader<Reg, WarpLayout, WarpReuse::kRowReuseCont> s2r;
        using Base = warp::CopyBase<WarpLayout, WarpReuse::kRowReuseCont>;
        SIter iter(smem);
        for (int k = 0; k < SIter::sc1; ++k) {
            Reg r;
            s2r(iter(k), r);
            if (Base::warp_col_id() == 0) {
                __half* block = dst + Base::warp_row_id() * (kRows / kWR) * kCols + k * kChunk;
#pragma unroll
                for (int i = 0; i < Reg::kRows; ++i)
#pragma unroll
                    for (int j = 0; j < Reg::kCols; ++j)
                        copy::detail::move_tile<__half, const Tile, kCols, 1, false>(
                            block + i * kTileMajor * kCols + j * kTileMinor, r(i, j));
            }
        }
    } else {
        using SIter = STileIterator<Shared, TileShape<kChunk, kCols>>;
        constexpr int kWC = tl::num_cols<WarpLayout>;
        using Tile = MfmaTile<__half, kTileMinor, kTileMajor, tl::Layout::kColMajor>;
        using Reg = RegTile<Tile, tl::ColMajor<kChunk / kTileMinor, kCols / kWC / kTileMajor>>;
        SharedToRegLoader<Reg, WarpLayout, WarpReuse::kColReuseCont> s2r;
        using Base = warp::CopyBase<WarpLayout, WarpReuse::kColReuseCont>;
        SIter iter(smem);
        for (int k = 0; k < SIter::sc0; ++k) {
            Reg r;
            s2r(iter(k), r);
            if (Base::warp_row_id() == 0) {
                __half* block = dst + k * kChunk + Base::warp_col_id() * (kCols / kWC) * kRows;
#pragma unroll
                for (int i = 0; i < Reg::kRows; ++i)
#pragma unroll
                    for (int j = 0; j < Reg::kCols; ++j)
                        copy::detail::move_tile<__half, const Tile, 1, kRows, false>(
                            block + i * kTileMinor + j * kTileMajor * kRows, r(i, j));
            }
        }
    }
}

// row-major shared [kRows (contraction index), kCols] -> column-major operand tiles through the transposing read ->
// global (row-major again: every element must come back to its place)
template <int kRows, int kCols, int kChunk, typename WarpLayout, bool kSwizzled, int kTileCols>
__global__ void __launch_bounds__(512) k_s2r_transposed(const __half* src, __half* dst) {
    extern __shared__ __align__(1024) unsigned char buf[];
    auto* smem = reinterpret_cast<__half*>(buf);
    constexpr int kTileRows = 512 / kTileCols;  // 32 x 16 or 16 x 32
    using Global = GlobalTile<__half, tl::RowMajor<kRows, kCols>>;
    using Shared = SharedTile<__half, tl::RowMajor<kRows, kCols>, kSwizzled>;
    using SIter = STileIterator<Shared, TileShape<kChunk, kCols>>;
    constexpr int kWC = tl::num_cols<WarpLayout>;
    using Tile = MfmaTile<__half, kTileRows, kTileCols, tl::Layout::kColMajor>;
    using Reg = RegTile<Tile, tl::ColMajor<kChunk / kTileRows, kCols / kWC / kTileCols>>;
    Global g_src(src);
    Shared s(smem);
    GlobalToSharedLoader<Shared, WarpLayout> g2s;
    g2s(g_src, s);
    __copy_async();
    __syncthreads();
    SharedToRegLoaderTr<Reg, WarpLayout, WarpReuse::kColReuseCont> s2r;
    using Base = warp::CopyBase<WarpLayout, WarpReuse::kColReuseCont>;
    SIter iter(smem);
    for (int k = 0; k < SIter::sc0; ++k) {
        Reg r;
        s2r(iter(k), r);
        if (Base::warp_row_id() == 0) {
            __half* block = dst + k * kChunk * kCols + Base::warp_col_id() * (kCols / kWC);
#pragma unroll
            for (int i = 0; i < Reg::kRows; ++i)
#pragma unroll
                for (int j = 0; j < Reg::kCols; ++j)
                    copy::detail::move_tile<__half, const Tile, kCols, 1, false>(
                        block + i * kTileRows * kCols + j * kTileCols, r(i, j));
        }
    }
}

// C = A · B through direct-to-LDS loads and MFMA-shaped tiles, one workgroup. kShape32: v_mfma_f32_32x32x16_f16,
// else v_mfma_f32_16x16x32_f16. kBRowMajor: B is stored row-major [kK, kN] and transposed by the loader.
// (the scheduled form is compiled for one wavefront per SIMD: its accumulators must have room to stay in AGPRs)
template <int kM, int kN, int kK, typename WarpLayout, bool kShape32, bool kBRowMajor, bool kScheduled = false>
__global__ void __launch_bounds__(kScheduled ? 256 : 512) k_tile_gemm_mfma(const __half* dA, const __half* dB, float* dC) {
    extern __shared__ __align__(1024) unsigned char buf[];
    auto* sA_ptr = reinterpret_cast<__half*>(buf);
    auto* sB_ptr = sA_ptr + kM * kK;
    constexpr int kWR = tl::num_rows<WarpLayout>, kWC = tl::num_cols<WarpLayout>;
    using Shape = traits::MfmaTileShape<__half, kShape32 ? traits::MfmaShape::k32x32x16 : traits::MfmaShape::k16x16x32>;
    constexpr int kChunkK = 64 / Shape::kK * Shape::kK;  // 64

    using GlobalA = GlobalTile<__half, tl::RowMajor<kM, kK>>;
    using SharedA = SharedTile<__half, tl::RowMajor<kM, kK>, true>;
    using SIterA = STileIterator<SharedA, TileShape<kM, kChunkK>>;
    using RegA = RegTile<typename Shape::TileA, tl::RowMajor<kM / kWR / Shape::kM, kChunkK / Shape::kK>>;

    using LayoutB = std::conditional_t<kBRowMajor, tl::RowMajor<kK, kN>, tl::ColMajor<kK, kN>>;
    using GlobalB = GlobalTile<__half, LayoutB>;
    using SharedB = SharedTile<__half, LayoutB, true>;
    using SIterB = STileIterator<SharedB, TileShape<kChunkK, kN>>;
    using RegB = RegTile<typename Shape::TileB, tl::ColMajor<kChunkK / Shape::kK, kN / kWC / Shape::kN>>;

    using GlobalC = GlobalTile<float, tl::RowMajor<kM, kN>>;
    using RegC = RegTile<typename Shape::TileC, tl::RowMajor<kM / kWR / Shape::kM, kN / kWC / Shape::kN>>;

    GlobalA gA(dA);
    GlobalB gB(dB);
    SharedA sA(sA_ptr);
    SharedB sB(sB_ptr);
    GlobalToSharedDirectLoader<SharedA, WarpLayout> g2s_a;
    GlobalToSharedDirectLoader<SharedB, WarpLayout> g2s_b;
    g2s_a(gA, sA);
    g2s_b(gB, sB);
    wait_group_and_barrier<0>();

    SIterA sAs(sA_ptr);
    SIterB sBs(sB_ptr);
    SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont> s2r_a;
    std::conditional_t<kBRowMajor, SharedToRegLoaderTr<RegB, WarpLayout, WarpReuse::kColReuseCont>,
                       SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>>
        s2r_b;
    RegA rA;
    RegB rB;
    RegC acc;
    if constexpr (kScheduled) {
        // the one-wavefront-per-SIMD form: accumulators pinned in AGPRs, the fragments of chunk k + 1 read one at a
        // time from the hook of the matrix instructions of chunk k (the first instructions of a chunk get them)
        static_assert(!kShape32 && !kBRowMajor);
        RegA rA2[2];
        RegB rB2[2];
        constexpr int kFragsA = RegA::kRows * RegA::kCols, kFragsB = RegB::kRows * RegB::kCols;
        constexpr int kMfmas = RegA::kRows * RegB::kCols * RegA::kCols;
        static_assert(kFragsA + kFragsB <= kMfmas);
        auto read_fragment = [&](int k, int which, int r) {
            if (r < kFragsA) s2r_a.load_one(sAs(k), rA2[which], r / RegA::kCols, r % RegA::kCols);
            else s2r_b.load_one(sBs(k), rB2[which], (r - kFragsA) / RegB::kCols, (r - kFragsA) % RegB::kCols);
        };
        compute::clear_pinned(acc);
        for (int r = 0; r < kFragsA + kFragsB; ++r) read_fragment(0, 0, r);
        [&]<int... kChunks>(std::integer_sequence<int, kChunks...>) {
            (compute::gemm_scheduled(rA2[kChunks & 1], rB2[kChunks & 1], acc,
                                     [&](auto n_c) {
                                         constexpr int n = decltype(n_c)::value;
                                         if constexpr (kChunks + 1 < SIterA::sc1 && n < kFragsA + kFragsB)
                                             read_fragment(kChunks + 1, (kChunks + 1) & 1, n);
                                     }),
             ...);
        }(std::make_integer_sequence<int, SIterA::sc1>{});
        compute::settle_accumulators(acc);
    } else {
        for (int k = 0; k < SIterA::sc1; ++k) {
            s2r_a(sAs(k), rA);
            s2r_b(sBs(k), rB);
            compute::gemm(rA, rB, acc);
        }
    }
    GlobalC gC(dC);
    RegToGlobalStorer<GlobalC, RegC, WarpLayout> r2g;
    r2g(acc, gC);
}

/// A gemm_scheduled hook that does nothing before an instruction and counts the calls behind them.
struct CountingHook {
    int issued = 0;
    template <typename N>
    DEVICE void operator()(N) {}
    template <typename N>
    DEVICE void after(N) {
        ++issued;
    }
};

// C = A · B with the fragment-at-a-time readers of a one-wavefront-per-SIMD kernel: A through SharedToRegPieces (one
// untracked ds_read_b128 per operand tile), B stored ROW-major [kK, kN] in a tile with the transposing-read swizzle
// (tl::LdsSwizzleTr) through SharedToRegTrPieces (standard contraction order), both waited for with
// wait_shared_reads; the matrix instructions through gemm_scheduled on v_mfma_f32_32x32x16_f16 tiles (accumulators
// pinned in AGPRs), whose after() hook runs behind every instruction (here it counts them into C's padding check).
template <int kM, int kN, int kK, typename WarpLayout>
__global__ void __launch_bounds__(256) k_tile_gemm_pieces(const __half* dA, const __half* dB, float* dC) {
    extern __shared__ __align__(1024) unsigned char buf[];
    auto* sA_ptr = reinterpret_cast<__half*>(buf);
    auto* sB_ptr = sA_ptr + kM * kK;
    constexpr int kWR = tl::num_rows<WarpLayout>, kWC = tl::num_cols<WarpLayout>;
    using Shape = traits::MfmaTileShape<__half, traits::MfmaShape::k32x32x16>;
    using GlobalA = GlobalTile<__half, tl::RowMajor<kM, kK>>;
    using SharedA = SharedTile<__half, tl::RowMajor<kM, kK>, true>;
    using RegA = RegTile<typename Shape::TileA, tl::RowMajor<kM / kWR / 32, kK / 16>>;
    using GlobalB = GlobalTile<__half, tl::RowMajor<kK, kN>>;
    using SharedB = SharedTile<__half, tl::RowMajor<kK, kN>, true, tl::LdsSwizzleTr<kN, 2>>;
    using RegB = RegTile<typename Shape::TileB, tl::ColMajor<kK / 16, kN / kWC / 32>>;
    using GlobalC = GlobalTile<float, tl::RowMajor<kM, kN>>;
    using RegC = RegTile<typename Shape::TileC, tl::RowMajor<kM / kWR / 32, kN / kWC / 32>>;

    GlobalA gA(dA);
    GlobalB gB(dB);
    SharedA sA(sA_ptr);
    SharedB sB(sB_ptr);
    GlobalToSharedDirectLoader<SharedA, WarpLayout> g2s_a;
    GlobalToSharedDirectLoader<SharedB, WarpLayout> g2s_b;
    g2s_a(gA, sA);
    g2s_b(gB, sB);
    wait_group_and_barrier<0>();

    SharedToRegPieces<RegA, SharedA, WarpLayout, WarpReuse::kRowReuseCont> read_a;
    SharedToRegTrPieces<RegB, SharedB, WarpLayout, WarpReuse::kColReuseCont> read_b;
    RegA rA;
    RegB rB;
    RegC acc;
    compute::clear_pinned(acc);
    static_for<RegA::kRows>([&](auto i_c) {
        static_for<RegA::kCols>([&](auto k_c) { read_a.template read<decltype(i_c)::value, decltype(k_c)::value>(sA, rA); });
    });
    static_for<RegB::kRows>([&](auto k_c) {
        static_for<RegB::kCols>([&](auto j_c) { read_b.template read<decltype(k_c)::value, decltype(j_c)::value>(sB, rB); });
    });
    wait_shared_reads<0>();
    CountingHook hook;
    compute::gemm_scheduled(rA, rB, acc, hook);
    compute::settle_accumulators(acc);
    if (hook.issued != RegA::kRows * RegA::kCols * RegB::kCols) return;  // C stays NaN: the case fails
    GlobalC gC(dC);
    RegToGlobalStorer<GlobalC, RegC, WarpLayout> r2g;
    r2g(acc, gC);
}

// The same chain on v_mfma_f32_16x16x32_f16: two 16 x 16 score accumulators side by side, converted, are the 16 x 32 A
// operand of the second product when V is fetched in their contraction order (SharedToRegTrPieces<..., true> on 32 x 16
// operand tiles, a shared tile with the 8-line form of LdsSwizzleTr). The fragment readers run in their bound form:
// bind() once, read_bound() / read_bound_to() with immediates, shift() to another allocation and back.
template <int kM, int kN, int kK, int kP, typename WarpLayout>
__global__ void __launch_bounds__(256) k_tile_b2b_accumulator_order_k32(const __half* dA, const __half* dBV, float* dD) {
    extern __shared__ __align__(1024) unsigned char buf[];
    auto* sA_ptr = reinterpret_cast<__half*>(buf) + 2048;  // (4 KiB in front: the bound views below start there)
    auto* sB_ptr = sA_ptr + kM * kK;
    auto* sV_ptr = sB_ptr + kN * kK;
    constexpr int kWR = tl::num_rows<WarpLayout>;
    static_assert(tl::num_cols<WarpLayout> == 1 && kM == 16 * kWR && kN % 32 == 0 && kK % 32 == 0 && kP == 128);
    using Shape = traits::MfmaTileShape<__half, traits::MfmaShape::k16x16x32>;
    using SharedA = SharedTile<__half, tl::RowMajor<kM, kK>, true>;
    using SharedB = SharedTile<__half, tl::ColMajor<kK, kN>, true>;
    using SharedV = SharedTile<__half, tl::RowMajor<kN, kP>, true, tl::LdsSwizzleTr<kP, 2, 8>>;
    using RegA = RegTile<typename Shape::TileA, tl::RowMajor<1, kK / 32>>;
    using RegB = RegTile<typename Shape::TileB, tl::ColMajor<kK / 32, kN / 16>>;
    using RegS = RegTile<typename Shape::TileC, tl::RowMajor<1, kN / 16>>;
    using RegP = RegTile<typename Shape::TileA, tl::RowMajor<1, kN / 32>>;
    using RegV = RegTile<typename Shape::TileB, tl::ColMajor<kN / 32, kP / 16>>;
    using RegD = RegTile<typename Shape::TileC, tl::RowMajor<1, kP / 16>>;
    using GlobalD = GlobalTile<float, tl::RowMajor<kM, kP>>;

    GlobalTile<__half, tl::RowMajor<kM, kK>> gA(dA);
    GlobalTile<__half, tl::ColMajor<kK, kN>> gB(dBV);
    GlobalTile<__half, tl::RowMajor<kN, kP>> gV(dBV + kN * kK);
    SharedA sA(sA_ptr);
    SharedB sB(sB_ptr);
    SharedV sV(sV_ptr);
    GlobalToSharedDirectLoader<SharedA, WarpLayout>{}(gA, sA);
    GlobalToSharedDirectLoader<SharedB, WarpLayout>{}(gB, sB);
    GlobalToSharedDirectLoader<SharedV, WarpLayout>{}(gV, sV);
    wait_group_and_barrier<0>();

    RegA rA;
    RegB rB;
    RegV rV;
    RegS rS;
    compute::pin_tiles<compute::RegFile::kVgpr>(rS);
    SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>{}(sA, rA);
    SharedToRegPieces<RegB, SharedB, WarpLayout, WarpReuse::kColReuseCont> read_b;
    SharedToRegTrPieces<RegV, SharedV, WarpLayout, WarpReuse::kColReuseCont, true> read_v;
    // bound to a view 4 KiB in front of the tile, every read with the immediate that brings it back; one fragment's
    // address moved away and back with shift()
    read_b.bind(SharedB(sB_ptr - 2048));
    read_v.bind(SharedV(sV_ptr - 2048));
    read_b.template shift<0, 0>(8192);
    read_v.template shift<0>(-4096);
    read_b.template shift<0, 0>(-8192);
    read_v.template shift<0>(4096);
    static_for<RegB::kRows * RegB::kCols>([&](auto n_c) {
        constexpr int n = decltype(n_c)::value;
        read_b.template read_bound<n / RegB::kCols, n % RegB::kCols, 4096>(rB);
    });
    static_for<RegV::kRows * RegV::kCols>([&](auto n_c) {
        constexpr int n = decltype(n_c)::value;
        read_v.template read_bound_to<n / RegV::kCols, n % RegV::kCols, 4096>(rV(n / RegV::kCols, n % RegV::kCols));
    });
    wait_shared_reads<0>();

    using First = compute::ScheduledGemm<RegA, RegB, RegS, compute::RegFile::kVgpr, compute::RegFile::kVgpr>;
    static_for<RegB::kCols>([&](auto j_c) {
        static_for<RegA::kCols>([&](auto k_c) { First::template at<0, decltype(j_c)::value, decltype(k_c)::value>(rA, rB, rS); });
    });
    asm volatile("s_nop 15\n\ts_nop 3");
    compute::pin_tiles<compute::RegFile::kVgpr>(rS);
    // accumulator tiles 2 j and 2 j + 1  ->  A operand tile j: elements 0..3 and 4..7
    RegP rP;
    static_for<RegP::kCols>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; e += 2)
                compute::convert_pair_here(rS(0, 2 * j + h)(0, e), rS(0, 2 * j + h)(0, e + 1), rP(0, j).mutable_data() + 4 * h + e);
    });
    RegD rD;
    compute::clear_pinned(rD);
    using Second = compute::ScheduledGemm<RegP, RegV, RegD>;
    static_for<RegV::kRows>([&](auto k_c) {
        static_for<RegV::kCols>([&](auto j_c) { Second::template at<0, decltype(j_c)::value, decltype(k_c)::value>(rP, rV, rD); });
    });
    compute::settle_accumulators(rD);
    GlobalD gD(dD);
    RegToGlobalStorer<GlobalD, RegD, WarpLayout> r2g;
    r2g(rD, gD);
}

// D = f16(A · B) · V on wavefronts that own 32 rows each: the 32 x 32 accumulator tiles of the first product, converted
// to f16 in place, ARE the A operand of the second one, because V (row-major [kN, kP], transposing-read swizzle) is
// fetched in the accumulator's own contraction order (SharedToRegTrPieces<..., kAccumulatorOrder = true>); every
// matrix instruction placed with ScheduledGemm::at. b = B column-major (stored [kN, kK]) followed by V.
template <int kM, int kN, int kK, int kP, typename WarpLayout>
__global__ void __launch_bounds__(256) k_tile_b2b_accumulator_order(const __half* dA, const __half* dBV, float* dD) {
    extern __shared__ __align__(1024) unsigned char buf[];
    auto* sA_ptr = reinterpret_cast<__half*>(buf);
    auto* sB_ptr = sA_ptr + kM * kK;
    auto* sV_ptr = sB_ptr + kN * kK;
    constexpr int kWR = tl::num_rows<WarpLayout>;
    static_assert(tl::num_cols<WarpLayout> == 1 && kM == 32 * kWR);
    using Shape = traits::MfmaTileShape<__half, traits::MfmaShape::k32x32x16>;
    using SharedA = SharedTile<__half, tl::RowMajor<kM, kK>, true>;
    using SharedB = SharedTile<__half, tl::ColMajor<kK, kN>, true>;
    using SharedV = SharedTile<__half, tl::RowMajor<kN, kP>, true, tl::LdsSwizzleTr<kP, 2>>;
    using RegA = RegTile<typename Shape::TileA, tl::RowMajor<1, kK / 16>>;
    using RegB = RegTile<typename Shape::TileB, tl::ColMajor<kK / 16, kN / 32>>;
    using RegS = RegTile<typename Shape::TileC, tl::RowMajor<1, kN / 32>>;
    using RegP = RegTile<typename Shape::TileA, tl::RowMajor<1, kN / 16>>;
    using RegV = RegTile<typename Shape::TileB, tl::ColMajor<kN / 16, kP / 32>>;
    using RegD = RegTile<typename Shape::TileC, tl::RowMajor<1, kP / 32>>;
    using GlobalD = GlobalTile<float, tl::RowMajor<kM, kP>>;

    GlobalTile<__half, tl::RowMajor<kM, kK>> gA(dA);
    GlobalTile<__half, tl::ColMajor<kK, kN>> gB(dBV);
    GlobalTile<__half, tl::RowMajor<kN, kP>> gV(dBV + kN * kK);
    SharedA sA(sA_ptr);
    SharedB sB(sB_ptr);
    SharedV sV(sV_ptr);
    GlobalToSharedDirectLoader<SharedA, WarpLayout>{}(gA, sA);
    GlobalToSharedDirectLoader<SharedB, WarpLayout>{}(gB, sB);
    GlobalToSharedDirectLoader<SharedV, WarpLayout>{}(gV, sV);
    wait_group_and_barrier<0>();

    RegA rA;
    RegB rB;
    RegV rV;
    // the accumulators of the first product are cleared (vector-ALU writes) HERE, well ahead of its first matrix
    // instruction: see ScheduledGemm on vector-ALU writes directly in front of an instruction that reads them
    RegS rS;
    compute::pin_tiles<compute::RegFile::kVgpr>(rS);
    SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>{}(sA, rA);
    SharedToRegPieces<RegB, SharedB, WarpLayout, WarpReuse::kColReuseCont> read_b;
    SharedToRegTrPieces<RegV, SharedV, WarpLayout, WarpReuse::kColReuseCont, true> read_v;
    static_for<RegB::kRows * RegB::kCols>([&](auto n_c) {
        constexpr int n = decltype(n_c)::value;
        read_b.template read<n / RegB::kCols, n % RegB::kCols>(sB, rB);
    });
    static_for<RegV::kRows * RegV::kCols>([&](auto n_c) {
        constexpr int n = decltype(n_c)::value;
        read_v.template read<n / RegV::kCols, n % RegV::kCols>(sV, rV);
    });
    wait_shared_reads<0>();

    // first product, accumulators in VGPRs (they are read by the vector ALU next)
    using First = compute::ScheduledGemm<RegA, RegB, RegS, compute::RegFile::kVgpr, compute::RegFile::kVgpr>;
    static_for<RegB::kCols>([&](auto j_c) {
        static_for<RegA::kCols>([&](auto k_c) { First::template at<0, decltype(j_c)::value, decltype(k_c)::value>(rA, rB, rS); });
    });
    asm volatile("s_nop 15\n\ts_nop 3");
    compute::pin_tiles<compute::RegFile::kVgpr>(rS);
    // accumulator tile j, elements 8 s2 + e  ->  A operand tile 2 j + s2, element e
    RegP rP;
    static_for<RegS::kCols>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
#pragma unroll
        for (int e = 0; e < 16; e += 2)
            compute::convert_pair_here(rS(0, j)(e), rS(0, j)(e + 1), rP(0, 2 * j + e / 8).mutable_data() + e % 8);
    });
    RegD rD;
    compute::clear_pinned(rD);
    using Second = compute::ScheduledGemm<RegP, RegV, RegD>;
    static_for<RegV::kRows>([&](auto k_c) {
        static_for<RegV::kCols>([&](auto j_c) { Second::template at<0, decltype(j_c)::value, decltype(k_c)::value>(rP, rV, rD); });
    });
    compute::settle_accumulators(rD);
    GlobalD gD(dD);
    RegToGlobalStorer<GlobalD, RegD, WarpLayout> r2g;
    r2g(rD, gD);
}

// ------------------------------------------------------------------ reduce / broadcast / softmax
// src [kRows, kCols] f32 row-major, one wavefront per 16... rows split over kW wavefronts.
// out_vec[kRows]: op 0 = row sum, 1 = row max; out_tile: op 2 = broadcast of row sums,
// 3 = tile minus row max (fused), 4 = softmax.
template <typename Element, int kRows, int kCols, int kW, int kOp>
__global__ void __launch_bounds__(512) k_row_ops(const Element* src, Element* out_vec, Element* out_tile) {
    using WarpLayout = tl::RowMajor<kW, 1>;
    using Global = GlobalTile<Element, tl::RowMajor<kRows, kCols>>;
    constexpr int kRs = kRows / kW / 16, kCs = kCols / 16;
    using Reg = RegTile<BaseTileRowMajor<Element>, tl::RowMajor<kRs, kCs>>;
    using Vec = RegTile<Element, tl::RowMajor<kRs, 1>>;
    Global g_src(src);
    Reg r;
    Vec v;
    GlobalToRegLoader<Reg, WarpLayout, WarpReuse::kCont> g2r;
    g2r(g_src, r);

    if constexpr (kOp == 0) {
        compute::SumReduce<Reg, tl::Layout::kRowMajor> op;
        op(r, v);
    } else if constexpr (kOp == 1) {
        compute::MaxReduce<Reg, tl::Layout::kRowMajor> op;
        op(r, v);
    } else if constexpr (kOp == 2) {
        compute::SumReduce<Reg, tl::Layout::kRowMajor> op;
        op(r, v);
        compute::Broadcast<Vec, Reg, tl::Layout::kRowMajor> bc;
        bc(v, r);
    } else if constexpr (kOp == 3) {
        compute::MaxReduce<Reg, tl::Layout::kRowMajor> op;
        op(r, v);
        compute::BroadcastSub<Vec, Reg, tl::Layout::kRowMajor> bs;
        bs(v, r);
    } else if constexpr (kOp == 4) {
        compute::Softmax<Reg, tl::Layout::kRowMajor> sm;
        sm(r, v);
    } else if constexpr (kOp == 5) {
        compute::SumReduce<Reg, tl::Layout::kRowMajor> op;
        op(r, v);
        compute::BroadcastAdd<Vec, Reg, tl::Layout::kRowMajor> b;
        b(v, r);
    } else if constexpr (kOp == 6) {
        compute::MaxReduce<Reg, tl::Layout::kRowMajor> op;
        op(r, v);
        compute::BroadcastMul<Vec, Reg, tl::Layout::kRowMajor> b;
        b(v, r);
    } else {
        compute::SumReduce<Reg, tl::Layout::kRowMajor> op;
        op(r, v);
        compute::BroadcastDiv<Vec, Reg, tl::Layout::kRowMajor> b;
        b(v, r);
    }
    // every lane of a row group holds the row value; lanes 0..15 of each wavefront write it
    const int lane = lane_id();
    if (lane < 16) {
#pragma unroll
        for (int i = 0; i < kRs; ++i) out_vec[wave_id() * (kRows / kW) + i * 16 + lane] = v(i, 0);
    }
    Global g_out(out_tile);
    RegToGlobalStorer<Global, Reg, WarpLayout> r2g;
    r2g(r, g_out);
}

// column-wise reductions on column-major tiles: src [kRows, kCols] column-major, kW wavefronts along the columns
template <typename Element, int kRows, int kCols, int kW, int kOp>
__global__ void __launch_bounds__(512) k_col_ops(const Element* src, Element* out_vec, Element* out_tile) {
    using WarpLayout = tl::RowMajor<1, kW>;
    using Global = GlobalTile<Element, tl::ColMajor<kRows, kCols>>;
    constexpr int kRs = kRows / 16, kCs = kCols / kW / 16;
    using Reg = RegTile<BaseTileColMajor<Element>, tl::ColMajor<kRs, kCs>>;
    using Vec = RegTile<Element, tl::RowMajor<1, kCs>>;
    Global g_src(src);
    Reg r;
    Vec v;
    GlobalToRegLoader<Reg, WarpLayout, WarpReuse::kCont> g2r;
    g2r(g_src, r);
    if constexpr (kOp == 0) {
        compute::SumReduce<Reg, tl::Layout::kColMajor> op;
        op(r, v);
    } else if constexpr (kOp == 1) {
        compute::MaxReduce<Reg, tl::Layout::kColMajor> op;
        op(r, v);
    } else if constexpr (kOp == 2) {
        compute::MaxReduce<Reg, tl::Layout::kColMajor> op;
        op(r, v);
        compute::BroadcastSub<Vec, Reg, tl::Layout::kColMajor> bs;
        bs(v, r);
    } else if constexpr (kOp == 3) {
        compute::SumReduce<Reg, tl::Layout::kColMajor> op;
        op(r, v);
        compute::Broadcast<Vec, Reg, tl::Layout::kColMajor> bc;
        bc(v, r);
    } else if constexpr (kOp == 4) {
        compute::Softmax<Reg, tl::Layout::kColMajor> sm;
        sm(r, v);
    } else {
        compute::MaxReduce<Reg, tl::Layout::kColMajor> op;
        op(r, v);
        compute::BroadcastMul<Vec, Reg, tl::Layout::kColMajor> b;
        b(v, r);
    }
    const int lane = lane_id();
    if (lane < 16) {
#pragma unroll
        for (int j = 0; j < kCs; ++j) out_vec[wave_id() * (kCols / kW) + j * 16 + lane] = v(0, j);
    }
    Global g_out(out_tile);
    RegToGlobalStorer<Global, Reg, WarpLayout> r2g;
    r2g(r, g_out);
}

// element-wise maps: out = op(a) or op(a, b) on [kRows, kCols] tiles in either orientation, kW wavefronts.
// kOp: 0 exp, 1 log, 2 relu, 3 add, 4 sub, 5 mul, 6 div, 7 max, 8 min, 9 convert f32 -> f16 (out is __half)
template <typename Element, bool kRowMajor, int kRows, int kCols, int kW, int kOp>
__global__ void __launch_bounds__(512) k_elementwise(const Element* a, const Element* b, void* out) {
    using WarpLayout = std::conditional_t<kRowMajor, tl::RowMajor<kW, 1>, tl::RowMajor<1, kW>>;
    using GLayout = std::conditional_t<kRowMajor, tl::RowMajor<kRows, kCols>, tl::ColMajor<kRows, kCols>>;
    constexpr int kRs = kRowMajor ? kRows / kW / 16 : kRows / 16;
    constexpr int kCs = kRowMajor ? kCols / 16 : kCols / kW / 16;
    using RLayout = std::conditional_t<kRowMajor, tl::RowMajor<kRs, kCs>, tl::ColMajor<kRs, kCs>>;
    using Base = std::conditional_t<kRowMajor, BaseTileRowMajor<Element>, BaseTileColMajor<Element>>;
    using Reg = RegTile<Base, RLayout>;
    using Global = GlobalTile<Element, GLayout>;
    Global ga(a), gb(b);
    Reg ra, rb, rc;
    GlobalToRegLoader<Reg, WarpLayout, WarpReuse::kCont> g2r;
    g2r(ga, ra);
    g2r(gb, rb);
    if constexpr (kOp == 9) {
        using HBase = std::conditional_t<kRowMajor, BaseTileRowMajor<__half>, BaseTileColMajor<__half>>;
        using HReg = RegTile<HBase, RLayout>;
        using HGlobal = GlobalTile<__half, GLayout>;
        HReg rh;
        compute::RegTileConvert<Reg, HReg> cvt;
        cvt(ra, rh);
        HGlobal go(static_cast<__half*>(out));
        RegToGlobalStorer<HGlobal, HReg, WarpLayout> r2g;
        r2g(rh, go);
    } else {
        if constexpr (kOp == 0) { compute::RegTileExp<Reg> op; op(ra, rc); }
        if constexpr (kOp == 1) { compute::RegTileLog<Reg> op; op(ra, rc); }
        if constexpr (kOp == 2) { compute::RegTileRelu<Reg> op; op(ra, rc); }
        if constexpr (kOp == 3) { compute::RegTileAdd<Reg> op; op(ra, rb, rc); }
        if constexpr (kOp == 4) { compute::RegTileSub<Reg> op; op(ra, rb, rc); }
        if constexpr (kOp == 5) { compute::RegTileMul<Reg> op; op(ra, rb, rc); }
        if constexpr (kOp == 6) { compute::RegTileDiv<Reg> op; op(ra, rb, rc); }
        if constexpr (kOp == 7) { compute::RegTileMax<Reg> op; op(ra, rb, rc); }
        if constexpr (kOp == 8) { compute::RegTileMin<Reg> op; op(ra, rb, rc); }
        Global go(static_cast<Element*>(out));
        RegToGlobalStorer<Global, Reg, WarpLayout> r2g;
        r2g(rc, go);
    }
}

// ------------------------------------------------------------------ registry
struct Case {
    std::string kind;   // which family
    std::string name;   // human-readable id
    int dims[8];        // family-specific: rows, cols, (k), elem bytes, row_major, ...
    int threads;
    int lds_bytes;
    void (*launch)(const void* a, const void* b, void* c, void* d, int threads, int lds, hipStream_t s);
};

std::vector<Case>& registry() {
    static std::vector<Case> r;
    return r;
}

template <auto Kernel, typename E>
void launch2(const void* a, const void*, void* c, void*, int threads, int lds, hipStream_t s) {
    hipLaunchKernelGGL(Kernel, dim3(1), dim3(threads), lds, s, static_cast<const E*>(a), static_cast<E*>(c));
}
template <auto Kernel>
void launch_gemm(const void* a, const void* b, void* c, void*, int threads, int lds, hipStream_t s) {
    hipLaunchKernelGGL(Kernel, dim3(1), dim3(threads), lds, s, static_cast<const __half*>(a),
                       static_cast<const __half*>(b), static_cast<float*>(c));
}
template <auto Kernel, typename E>
void launch_ops(const void* a, const void*, void* c, void* d, int threads, int lds, hipStream_t s) {
    hipLaunchKernelGGL(Kernel, dim3(1), dim3(threads), lds, s, static_cast<const E*>(a), static_cast<E*>(c),
                       static_cast<E*>(d));
}

template <int kM, int kN, int kK, int kWR, int kWC>
void reg_gemm_pieces() {
    using W = tl::RowMajor<kWR, kWC>;
    registry().push_back({"tile_gemm",
                          "pieces_scheduled_mfma32x32x16_" + std::to_string(kM) + "x" + std::to_string(kN) + "x" +
                              std::to_string(kK) + "_w" + std::to_string(kWR) + "x" + std::to_string(kWC) + "_b_row_major",
                          {kM, kN, kK, 2, 1, 0, 0, 0},
                          kWR * kWC * 64,
                          (kM + kN) * kK * 2,
                          &launch_gemm<k_tile_gemm_pieces<kM, kN, kK, W>>});
}

template <int kM, int kN, int kK, int kP, int kWR>
void reg_b2b_acc_order_k32() {
    using W = tl::RowMajor<kWR, 1>;
    registry().push_back({"tile_b2b",
                          "accumulator_order_16x16x32_" + std::to_string(kM) + "x" + std::to_string(kN) + "x" + std::to_string(kK) +
                              "x" + std::to_string(kP) + "_w" + std::to_string(kWR) + "x1",
                          {kM, kN, kK, kP, 0, 0, 0, 0},
                          kWR * 64,
                          (kM * kK + kN * kK + kN * kP) * 2 + 4096,
                          &launch_gemm<k_tile_b2b_accumulator_order_k32<kM, kN, kK, kP, W>>});
}

template <int kM, int kN, int kK, int kP, int kWR>
void reg_b2b_acc_order() {
    using W = tl::RowMajor<kWR, 1>;
    registry().push_back({"tile_b2b",
                          "accumulator_order_" + std::to_string(kM) + "x" + std::to_string(kN) + "x" + std::to_string(kK) +
                              "x" + std::to_string(kP) + "_w" + std::to_string(kWR) + "x1",
                          {kM, kN, kK, kP, 0, 0, 0, 0},
                          kWR * 64,
                          (kM * kK + kN * kK + kN * kP) * 2,
                          &launch_gemm<k_tile_b2b_accumulator_order<kM, kN, kK, kP, W>>});
}

template <typename E>
constexpr const char* ename() {
    return sizeof(E) == 2 ? "f16" : "f32";
}

template <typename E, bool kRowMajor, int kRows, int kCols, int kWR, int kWC, bool kSwz, bool kStream = false>
void reg_g2s() {
    using W = tl::RowMajor<kWR, kWC>;
    registry().push_back({"g2s_roundtrip",
                          std::string(ename<E>()) + (kRowMajor ? "_row_" : "_col_") + std::to_string(kRows) + "x" +
                              std::to_string(kCols) + "_w" + std::to_string(kWR) + "x" + std::to_string(kWC) +
                              (kSwz ? "_swz" : "_plain") + (kStream ? "_stream_storer" : ""),
                          {kRows, kCols, 0, int(sizeof(E)), kRowMajor, 0, 0, 0},
                          kWR * kWC * 64,
                          int(kRows * kCols * sizeof(E)),
                          &launch2<k_g2s_roundtrip<E, kRowMajor, kRows, kCols, W, kSwz, kStream>, E>});
}

template <typename E, bool kRowMajor, int kRows, int kCols, int kChunk, int kWR, int kWC, bool kSwz>
void reg_s2r() {
    using W = tl::RowMajor<kWR, kWC>;
    Case c{"s2r_identity",
           std::string(ename<E>()) + (kRowMajor ? "_row_" : "_col_") + std::to_string(kRows) + "x" +
               std::to_string(kCols) + "_c" + std::to_string(kChunk) + "_w" + std::to_string(kWR) + "x" +
               std::to_string(kWC) + (kSwz ? "_swz" : "_plain"),
           {kRows, kCols, kChunk, int(sizeof(E)), kRowMajor, 0, 0, 0},
           kWR * kWC * 64,
           int(kRows * kCols * sizeof(E)),
           nullptr};
    if constexpr (kRowMajor)
        c.launch = &launch2<k_s2r_row_major<E, kRows, kCols, kChunk, W, kSwz>, E>;
    else
        c.launch = &launch2<k_s2r_col_major<E, kRows, kCols, kChunk, W, kSwz>, E>;
    registry().push_back(c);
}

template <typename E, bool kRowMajor, int kRows, int kCols, int kWR, int kWC, bool kSwz>
void reg_store() {
    using W = tl::RowMajor<kWR, kWC>;
    registry().push_back({"store_roundtrip",
                          std::string(ename<E>()) + (kRowMajor ? "_row_" : "_col_") + std::to_string(kRows) + "x" +
                              std::to_string(kCols) + "_w" + std::to_string(kWR) + "x" + std::to_string(kWC) +
                              (kSwz ? "_swz" : "_plain"),
                          {kRows, kCols, 0, int(sizeof(E)), kRowMajor, 0, 0, 0},
                          kWR * kWC * 64,
                          int(kRows * kCols * sizeof(E)),
                          &launch2<k_store_roundtrip<E, kRowMajor, kRows, kCols, W, kSwz>, E>});
}

template <typename E, bool kGRow, bool kRRow, int kRows, int kCols, int kWR, int kWC>
void reg_g2r() {
    using W = tl::RowMajor<kWR, kWC>;
    registry().push_back({"g2r_roundtrip",
                          std::string(ename<E>()) + (kGRow ? "_grow" : "_gcol") + (kRRow ? "_rrow_" : "_rcol_") +
                              std::to_string(kRows) + "x" + std::to_string(kCols) + "_w" + std::to_string(kWR) + "x" +
                              std::to_string(kWC),
                          {kRows, kCols, 0, int(sizeof(E)), kGRow, kRRow, 0, 0},
                          kWR * kWC * 64,
                          0,
                          &launch2<k_g2r_roundtrip<E, kGRow, kRRow, kRows, kCols, W>, E>});
}

template <int kM, int kN, int kK, int kWR, int kWC, int kChunkK, bool kSwz = true>
void reg_gemm() {
    using W = tl::RowMajor<kWR, kWC>;
    registry().push_back({"tile_gemm",
                          std::to_string(kM) + "x" + std::to_string(kN) + "x" + std::to_string(kK) + "_w" +
                              std::to_string(kWR) + "x" + std::to_string(kWC) + "_c" + std::to_string(kChunkK) +
                              (kSwz ? "_swz" : "_plain"),
                          {kM, kN, kK, kChunkK, 0, 0, 0, 0},
                          kWR * kWC * 64,
                          int((kM * kK + kK * kN) * sizeof(__half)),
                          &launch_gemm<k_tile_gemm<kM, kN, kK, W, kChunkK, kSwz>>});
}

template <bool kRowMajor, int kRows, int kCols, int kWR, int kWC, bool kSwz, bool kPieces = false>
void reg_direct() {
    using W = tl::RowMajor<kWR, kWC>;
    registry().push_back({"g2s_roundtrip",
                          std::string(kPieces ? "f16_direct_pieces" : "f16_direct_ring") + (kRowMajor ? "_row_" : "_col_") + std::to_string(kRows) + "x" +
                              std::to_string(kCols) + "_w" + std::to_string(kWR) + "x" + std::to_string(kWC) +
                              (kSwz ? "_swz" : "_plain"),
                          {kRows, kCols, 0, 2, kRowMajor, 0, 0, 0},
                          kWR * kWC * 64,
                          int(3 * kRows * kCols * sizeof(__half)),
                          &launch2<k_direct_ring_roundtrip<kRowMajor, kRows, kCols, W, kSwz, kPieces>, __half>});
}

template <bool kRowMajor, int kRows, int kCols, int kChunk, int kWR, int kWC, bool kSwz, int kTileMajor>
void reg_s2r_mfma() {
    using W = tl::RowMajor<kWR, kWC>;
    registry().push_back({"s2r_identity",
                          std::string("f16_mfma") + std::to_string(kTileMajor) + "x" + std::to_string(512 / kTileMajor) +
                              (kRowMajor ? "_row_" : "_col_") + std::to_string(kRows) + "x" + std::to_string(kCols) +
                              "_c" + std::to_string(kChunk) + "_w" + std::to_string(kWR) + "x" + std::to_string(kWC) +
                              (kSwz ? "_swz" : "_plain"),
                          {kRows, kCols, kChunk, 2, kRowMajor, 0, 0, 0},
                          kWR * kWC * 64,
                          int(kRows * kCols * sizeof(__half)),
                          &launch2<k_s2r_mfma_tiles<kRowMajor, kRows, kCols, kChunk, W, kSwz, kTileMajor>, __half>});
}

template <int kRows, int kCols, int kChunk, int kWR, int kWC, bool kSwz, int kTileCols>
void reg_s2r_tr() {
    using W = tl::RowMajor<kWR, kWC>;
    registry().push_back({"s2r_identity",
                          std::string("f16_transposed") + std::to_string(512 / kTileCols) + "x" + std::to_string(kTileCols) +
                              "_row_" + std::to_string(kRows) + "x" + std::to_string(kCols) + "_c" +
                              std::to_string(kChunk) + "_w" + std::to_string(kWR) + "x" + std::to_string(kWC) +
                              (kSwz ? "_swz" : "_plain"),
                          {kRows, kCols, kChunk, 2, 1, 0, 0, 0},
                          kWR * kWC * 64,
                          int(kRows * kCols * sizeof(__half)),
                          &launch2<k_s2r_transposed<kRows, kCols, kChunk, W, kSwz, kTileCols>, __half>});
}

template <int kM, int kN, int kK, int kWR, int kWC, bool kShape32, bool kBRowMajor, bool kScheduled = false>
void reg_gemm_mfma() {
    using W = tl::RowMajor<kWR, kWC>;
    registry().push_back({"tile_gemm",
                          std::string(kScheduled ? "scheduled_" : "") + std::string(kShape32 ? "mfma32x32x16_" : "mfma16x16x32_") + std::to_string(kM) + "x" +
                              std::to_string(kN) + "x" + std::to_string(kK) + "_w" + std::to_string(kWR) + "x" +
                              std::to_string(kWC) + (kBRowMajor ? "_b_row_major" : ""),
                          {kM, kN, kK, 64, kBRowMajor, 0, 0, 0},
                          kWR * kWC * 64,
                          int((kM * kK + kK * kN) * sizeof(__half)),
                          &launch_gemm<k_tile_gemm_mfma<kM, kN, kK, W, kShape32, kBRowMajor, kScheduled>>});
}

template <typename E, int kRows, int kCols, int kW, int kOp>
void reg_row_op() {
    static const char* names[] = {"sum", "max", "bcast_sum", "sub_max", "softmax", "add_sum", "mul_max", "div_sum"};
    registry().push_back({"row_ops",
                          std::string(ename<E>()) + "_" + names[kOp] + "_" + std::to_string(kRows) + "x" +
                              std::to_string(kCols) + "_w" + std::to_string(kW),
                          {kRows, kCols, kOp, int(sizeof(E)), 1, 0, 0, 0},
                          kW * 64,
                          0,
                          &launch_ops<k_row_ops<E, kRows, kCols, kW, kOp>, E>});
}

template <typename E, int kRows, int kCols, int kW, int kOp>
void reg_col_op() {
    static const char* names[] = {"sum", "max", "sub_max", "bcast_sum", "softmax", "mul_max"};
    registry().push_back({"col_ops",
                          std::string(ename<E>()) + "_" + names[kOp] + "_" + std::to_string(kRows) + "x" +
                              std::to_string(kCols) + "_w" + std::to_string(kW),
                          {kRows, kCols, kOp, int(sizeof(E)), 0, 0, 0, 0},
                          kW * 64,
                          0,
                          &launch_ops<k_col_ops<E, kRows, kCols, kW, kOp>, E>});
}

template <auto Kernel, typename E>
void launch_elementwise(const void* a, const void* b, void* c, void*, int threads, int lds, hipStream_t s) {
    hipLaunchKernelGGL(Kernel, dim3(1), dim3(threads), lds, s, static_cast<const E*>(a), static_cast<const E*>(b), c);
}

template <typename E, bool kRowMajor, int kRows, int kCols, int kW, int kOp>
void reg_elementwise() {
    static const char* names[] = {"exp", "log", "relu", "add", "sub", "mul", "div", "max", "min", "convert_f16"};
    registry().push_back({"elementwise",
                          std::string(ename<E>()) + "_" + names[kOp] + (kRowMajor ? "_row_" : "_col_") +
                              std::to_string(kRows) + "x" + std::to_string(kCols) + "_w" + std::to_string(kW),
                          {kRows, kCols, kOp, int(sizeof(E)), kRowMajor, 0, 0, 0},
                          kW * 64,
                          0,
                          &launch_elementwise<k_elementwise<E, kRowMajor, kRows, kCols, kW, kOp>, E>});
}

template <typename E, bool kSwz>
void reg_g2s_family() {
    // shapes and warp layouts of the reference's test_g2s_load.cu:118-144
    reg_g2s<E, true, 16, 16, 1, 1, kSwz>();
    reg_g2s<E, true, 16, 64, 1, 4, kSwz>();
    reg_g2s<E, true, 64, 16, 4, 1, kSwz>();
    reg_g2s<E, true, 32, 32, 2, 2, kSwz>();
    reg_g2s<E, true, 64, 64, 2, 2, kSwz>();
    reg_g2s<E, true, 96, 128, 2, 4, kSwz>();
    reg_g2s<E, true, 96, 128, 2, 4, kSwz, true>();  // ... leaving through SharedToGlobalStreamStorer
    reg_g2s<E, false, 128, 96, 2, 2, kSwz, true>();
    reg_g2s<E, true, 192, 32, 2, 2, kSwz>();
    reg_g2s<E, false, 16, 16, 1, 1, kSwz>();
    reg_g2s<E, false, 64, 16, 4, 1, kSwz>();
    reg_g2s<E, false, 16, 64, 1, 4, kSwz>();
    reg_g2s<E, false, 64, 64, 2, 2, kSwz>();
    reg_g2s<E, false, 128, 96, 2, 2, kSwz>();
}

void build_registry() {
    if (!registry().empty()) return;
    reg_g2s_family<__half, false>();
    reg_g2s_family<__half, true>();
    reg_g2s_family<float, false>();
    reg_g2s_family<float, true>();

    // swizzled and plain loads must both reproduce the source (test_swizzled_copy.cu:399-450 shapes)
    reg_s2r<__half, true, 16, 16, 16, 1, 1, false>();
    reg_s2r<__half, true, 16, 16, 16, 1, 1, true>();
    reg_s2r<__half, true, 16, 32, 16, 1, 1, true>();
    reg_s2r<__half, true, 16, 32, 32, 1, 1, true>();
    reg_s2r<__half, true, 32, 64, 16, 1, 1, true>();
    reg_s2r<__half, true, 32, 64, 32, 2, 1, true>();
    reg_s2r<__half, true, 64, 64, 64, 2, 2, true>();
    reg_s2r<__half, true, 64, 64, 32, 2, 2, false>();
    reg_s2r<__half, true, 64, 128, 32, 2, 2, true>();
    reg_s2r<__half, true, 64, 128, 128, 4, 1, true>();
    reg_s2r<__half, true, 128, 128, 64, 2, 4, true>();
    reg_s2r<__half, true, 64, 256, 32, 2, 2, true>();
    reg_s2r<__half, true, 32, 48, 16, 2, 1, true>();
    reg_s2r<float, true, 32, 64, 32, 2, 1, true>();
    reg_s2r<__half, false, 16, 16, 16, 1, 1, true>();
    reg_s2r<__half, false, 32, 16, 16, 1, 1, true>();
    reg_s2r<__half, false, 64, 32, 32, 1, 2, true>();
    reg_s2r<__half, false, 64, 64, 64, 2, 2, true>();
    reg_s2r<__half, false, 64, 64, 32, 2, 2, false>();
    reg_s2r<__half, false, 128, 64, 32, 2, 2, true>();
    reg_s2r<__half, false, 128, 128, 64, 4, 2, true>();
    reg_s2r<__half, false, 32, 256, 32, 2, 2, true>();

    // store round trips (test_swizzled_copy.cu:452-499)
    reg_store<float, true, 16, 16, 1, 1, true>();
    reg_store<float, true, 64, 64, 2, 2, true>();
    reg_store<float, true, 64, 256, 2, 2, true>();
    reg_store<float, true, 64, 64, 2, 2, false>();
    reg_store<__half, true, 16, 16, 1, 1, false>();
    reg_store<__half, true, 64, 128, 2, 2, false>();
    reg_store<__half, true, 64, 128, 2, 2, true>();
    reg_store<float, false, 64, 64, 2, 2, true>();
    reg_store<__half, false, 64, 32, 2, 1, true>();

    // global <-> register, all four orientation combinations
    reg_g2r<__half, true, true, 16, 16, 1, 1>();
    reg_g2r<__half, true, true, 64, 64, 2, 2>();
    reg_g2r<__half, false, false, 64, 64, 2, 2>();
    reg_g2r<__half, true, false, 32, 32, 1, 1>();
    reg_g2r<__half, false, true, 32, 32, 2, 1>();
    reg_g2r<float, true, true, 64, 32, 2, 2>();
    reg_g2r<float, false, false, 32, 64, 1, 2>();

    // tile gemm: the (M, N, K, warps, chunkK) combinations of the reference's test_gemm.cu:312-350
    reg_gemm<16, 16, 16, 1, 1, 16>();
    reg_gemm<16, 16, 32, 1, 1, 16>();
    reg_gemm<16, 16, 32, 1, 1, 32>();
    reg_gemm<32, 32, 32, 1, 1, 16>();
    reg_gemm<32, 32, 32, 1, 1, 32>();
    reg_gemm<32, 32, 64, 1, 1, 32>();
    reg_gemm<64, 64, 64, 1, 1, 16>();
    reg_gemm<64, 64, 64, 1, 1, 64>();
    reg_gemm<128, 64, 64, 1, 1, 32>();
    reg_gemm<96, 48, 80, 1, 1, 16>();
    reg_gemm<96, 48, 80, 1, 1, 80>();
    reg_gemm<32, 64, 128, 2, 1, 32>();
    reg_gemm<64, 32, 128, 1, 2, 64>();
    reg_gemm<32, 32, 64, 2, 2, 32>();
    reg_gemm<64, 64, 64, 2, 2, 32>();
    reg_gemm<64, 64, 64, 2, 2, 64>();
    reg_gemm<64, 32, 128, 4, 1, 64>();
    reg_gemm<32, 64, 128, 1, 4, 64>();
    reg_gemm<128, 128, 128, 2, 2, 64>();
    reg_gemm<64, 128, 128, 2, 4, 32>();
    reg_gemm<64, 128, 128, 2, 4, 128>();
    reg_gemm<64, 64, 64, 2, 2, 32, false>();
    reg_gemm<32, 32, 48, 1, 1, 48>();

    // the CDNA4 data path: direct-to-LDS loads into a ring stage (lines of 64, 128, 256 and 512 bytes)
    reg_direct<true, 64, 64, 2, 2, true>();
    reg_direct<true, 64, 64, 2, 2, false>();
    reg_direct<true, 256, 64, 4, 2, true>();
    reg_direct<true, 128, 32, 2, 1, true>();
    reg_direct<true, 32, 128, 1, 2, true>();
    reg_direct<true, 16, 256, 1, 1, true>();
    reg_direct<false, 64, 128, 2, 2, true>();
    reg_direct<false, 64, 256, 4, 2, true>();
    reg_direct<false, 128, 64, 1, 4, false>();
    // the same copies dealt a piece at a time (GlobalToSharedDirectPieces + issue)
    reg_direct<true, 64, 64, 2, 2, true, true>();
    reg_direct<true, 256, 64, 2, 2, true, true>();
    reg_direct<true, 16, 256, 1, 1, false, true>();
    reg_direct<false, 64, 256, 2, 2, true, true>();
    reg_direct<false, 128, 64, 1, 4, false, true>();
    // MFMA-shaped operand tiles out of LDS (ds_read_b128): both instruction shapes, both operands
    reg_s2r_mfma<true, 64, 64, 64, 2, 2, true, 16>();
    reg_s2r_mfma<true, 64, 64, 32, 2, 2, false, 16>();
    reg_s2r_mfma<true, 128, 128, 64, 4, 1, true, 16>();
    reg_s2r_mfma<true, 256, 64, 32, 4, 2, true, 16>();
    reg_s2r_mfma<true, 64, 64, 16, 2, 2, true, 32>();
    reg_s2r_mfma<true, 128, 128, 64, 2, 2, true, 32>();
    reg_s2r_mfma<false, 64, 64, 64, 2, 2, true, 16>();
    reg_s2r_mfma<false, 64, 256, 32, 4, 2, true, 16>();
    reg_s2r_mfma<false, 128, 64, 32, 2, 2, false, 16>();
    reg_s2r_mfma<false, 64, 128, 16, 2, 2, true, 32>();
    // column-major operand tiles out of a row-major shared tile (ds_read_b64_tr_b16)
    reg_s2r_tr<64, 64, 32, 2, 2, true, 16>();
    reg_s2r_tr<64, 64, 32, 2, 2, false, 16>();
    reg_s2r_tr<128, 128, 64, 2, 4, true, 16>();
    reg_s2r_tr<64, 128, 16, 2, 2, true, 32>();
    reg_s2r_tr<128, 64, 32, 1, 1, true, 32>();
    // gemm() on MFMA-shaped tiles, operands brought in by the direct loader
    reg_gemm_mfma<64, 64, 64, 2, 2, false, false>();
    reg_gemm_mfma<128, 128, 128, 2, 2, false, false>();
    reg_gemm_mfma<64, 128, 128, 2, 4, false, false>();
    reg_gemm_mfma<128, 64, 64, 4, 1, false, false>();
    reg_gemm_mfma<64, 64, 64, 2, 2, true, false>();
    reg_gemm_mfma<128, 128, 128, 2, 2, true, false>();
    reg_gemm_mfma<128, 64, 128, 4, 1, true, false>();
    reg_gemm_mfma<64, 64, 64, 2, 2, false, true>();
    reg_gemm_mfma<128, 128, 64, 2, 2, false, true>();
    reg_gemm_mfma<64, 64, 128, 2, 2, true, true>();
    // gemm_scheduled(): AGPR-pinned accumulators, fragment reads placed by the hook (1, 2 and 4 chunks of K)
    reg_gemm_mfma<64, 64, 64, 2, 2, false, false, true>();
    reg_gemm_mfma<128, 128, 128, 2, 2, false, false, true>();
    reg_gemm_mfma<256, 256, 64, 2, 2, false, false, true>();
    reg_gemm_mfma<128, 64, 256, 1, 1, false, false, true>();

    // reductions, broadcasts, softmax (test_reduce.cu / test_broadcast.cu / test_softmax.cu shapes)
    reg_row_op<float, 16, 16, 1, 0>();
    reg_row_op<float, 16, 16, 1, 1>();
    reg_row_op<float, 32, 64, 1, 0>();
    reg_row_op<float, 32, 64, 2, 1>();
    reg_row_op<float, 64, 128, 4, 0>();
    reg_row_op<__half, 32, 32, 1, 0>();
    reg_row_op<__half, 32, 32, 1, 1>();
    reg_row_op<float, 32, 64, 1, 2>();
    reg_row_op<float, 32, 64, 2, 3>();
    reg_row_op<float, 16, 16, 1, 4>();
    reg_row_op<float, 32, 32, 1, 4>();
    reg_row_op<float, 64, 16, 4, 4>();
    reg_row_op<__half, 32, 32, 1, 4>();
    reg_col_op<float, 16, 16, 1, 0>();
    reg_col_op<float, 64, 32, 2, 1>();
    reg_col_op<float, 64, 32, 1, 2>();
    reg_col_op<__half, 32, 32, 1, 0>();
    reg_row_op<float, 32, 64, 2, 5>();
    reg_row_op<float, 32, 32, 1, 6>();
    reg_row_op<float, 64, 32, 4, 7>();
    reg_row_op<__half, 32, 32, 1, 7>();
    reg_col_op<float, 32, 64, 2, 3>();
    reg_col_op<float, 16, 16, 1, 4>();
    reg_col_op<float, 64, 32, 2, 4>();
    reg_col_op<__half, 32, 32, 1, 4>();
    reg_col_op<float, 32, 32, 1, 5>();

    // element-wise maps (reference: map.hpp:84-133, math_functor.hpp): every functor, both orientations
    reg_elementwise<float, true, 32, 32, 1, 0>();
    reg_elementwise<float, true, 32, 32, 1, 1>();
    reg_elementwise<float, true, 32, 64, 2, 2>();
    reg_elementwise<float, true, 64, 32, 4, 3>();
    reg_elementwise<float, true, 32, 32, 1, 4>();
    reg_elementwise<float, true, 32, 32, 1, 5>();
    reg_elementwise<float, true, 32, 32, 1, 6>();
    reg_elementwise<float, true, 32, 32, 2, 7>();
    reg_elementwise<float, true, 32, 32, 2, 8>();
    reg_elementwise<float, true, 32, 64, 2, 9>();
    reg_elementwise<float, false, 32, 64, 2, 0>();
    reg_elementwise<float, false, 64, 32, 1, 6>();
    reg_elementwise<float, false, 32, 32, 1, 8>();
    reg_elementwise<float, false, 32, 32, 1, 9>();
    reg_elementwise<__half, true, 32, 32, 1, 0>();
    reg_elementwise<__half, true, 32, 32, 1, 1>();
    reg_elementwise<__half, true, 32, 32, 1, 2>();
    reg_elementwise<__half, true, 32, 64, 2, 3>();
    reg_elementwise<__half, true, 32, 32, 1, 5>();
    reg_elementwise<__half, true, 32, 32, 1, 6>();
    reg_elementwise<__half, false, 32, 32, 1, 7>();
    reg_elementwise<__half, false, 32, 32, 1, 8>();

    // (new cases go last: the host side seeds its inputs with the case number)
    // fragment-at-a-time readers + gemm_scheduled on 32x32x16 tiles with an after() hook; B row-major
    reg_gemm_pieces<64, 64, 64, 2, 2>();
    reg_gemm_pieces<128, 128, 64, 2, 2>();
    reg_gemm_pieces<128, 64, 128, 4, 1>();
    reg_gemm_pieces<32, 128, 32, 1, 1>();
    // two chained products with the accumulator of the first as the A operand of the second
    reg_b2b_acc_order<32, 64, 64, 64, 1>();
    reg_b2b_acc_order<64, 128, 32, 64, 2>();
    reg_b2b_acc_order<128, 64, 128, 64, 4>();
    reg_b2b_acc_order_k32<16, 32, 32, 128, 1>();
    reg_b2b_acc_order_k32<32, 64, 128, 128, 2>();
    reg_b2b_acc_order_k32<64, 128, 64, 128, 4>();
}

thread_local std::string g_err;

// prints (device printf) a 32 x 48 f16 ramp held as 2 x 3 row-major BaseTiles, a 32 x 32 f32 MFMA accumulator tile and
// the row maxima of the first, each in matrix order
__global__ void __launch_bounds__(64) k_print_tiles(const __half* src) {
    using Global = GlobalTile<__half, tl::RowMajor<32, 48>>;
    using Reg = RegTile<BaseTileRowMajor<__half>, tl::RowMajor<2, 3>>;
    Global g(src);
    Reg r;
    GlobalToRegLoader<Reg, tl::RowMajor<1, 1>, WarpReuse::kCont> g2r;
    g2r(g, r);
    RegTilePrinter<Reg> print;
    print(r, threadIdx.x);

    using Vec = RegTile<__half, tl::RowMajor<2, 1>>;
    Vec v;
    compute::MaxReduce<Reg, tl::Layout::kRowMajor> row_max;
    row_max(r, v);
    RegVecPrinter<Vec> print_vec;
    print_vec(v, threadIdx.x);

    using Acc = RegTile<MfmaTileC32x32<float>, tl::RowMajor<1, 1>>;
    Acc acc;
    // element (row, col) = row + col / 100: this lane holds row lane % 32, columns 8 q + 4 (lane / 32) + e
    for (int q = 0; q < 4; ++q)
        for (int e = 0; e < 4; ++e)
            acc(0, 0)(4 * q + e) = float(threadIdx.x % 32) + float(8 * q + 4 * (threadIdx.x / 32) + e) * 0.01f;
    RegTilePrinter<Acc> print_acc;
    print_acc(acc, threadIdx.x);
}

}  // namespace

extern "C" {

int tt_num_cases(void) {
    build_registry();
    return static_cast<int>(registry().size());
}

/// kind / name are NUL-terminated strings owned by the library; dims has 8 ints.
int tt_case_info(int id, const char** kind, const char** name, int* dims, int* threads, int* lds_bytes) {
    build_registry();
    if (id < 0 || id >= (int)registry().size()) return -1;
    const Case& c = registry()[id];
    *kind = c.kind.c_str();
    *name = c.name.c_str();
    for (int i = 0; i < 8; ++i) dims[i] = c.dims[i];
    *threads = c.threads;
    *lds_bytes = c.lds_bytes;
    return 0;
}

/// Run case `id` on `stream`. Buffers are device pointers; their meaning depends on the family:
///   copies:    a = src, c = dst
///   tile_gemm: a = A, b = B, c = C
///   row/col ops: a = src, c = per-line vector, d = tile output
///   elementwise: a, b = operands, c = result
int tt_run_case(int id, const void* a, const void* b, void* c, void* d, void* stream) {
    build_registry();
    if (id < 0 || id >= (int)registry().size()) return -1;
    const Case& cs = registry()[id];
    cs.launch(a, b, c, d, cs.threads, cs.lds_bytes, static_cast<hipStream_t>(stream));
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        g_err = hipGetErrorString(e);
        return -3;
    }
    return 0;
}

/// Launches the tile printer demonstration (one wavefront; output goes to the process's stdout at the next
/// synchronisation). src: 32 x 48 f16, row-major.
int tt_print_tiles(const void* src, void* stream) {
    hipLaunchKernelGGL(k_print_tiles, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), static_cast<const __half*>(src));
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        g_err = hipGetErrorString(e);
        return -3;
    }
    return 0;
}

const char* tt_last_error(void) { return g_err.c_str(); }

}  // extern "C"
