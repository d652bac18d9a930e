// GEMM kernels composed from the tile primitives.
//   * GemmTraits / simple_gemm: global -> register -> MFMA; the kernel of the reference's
//     README and examples/cpp/01_gemm/01_gemm_global_reg/gemm.hpp:13-92.
//   * KeGemmTraits / gemm: global -> LDS -> register -> MFMA, C staged through LDS; the
//     kernel of examples/cpp/01_gemm/02_gemm_all_mem/gemm.hpp:15-155. A barrier is added
//     at the end of each k-step: the reference overwrites the shared tiles of the next
//     step while other warps may still be reading them.
//   * PipelinedGemmTileTraits / gemm_tile_pipelined: the same all-memory kernel on the CDNA4 data path, still
//     composed from tile-library functors only: direct-to-LDS loads into a two-stage SharedRing
//     (GlobalToSharedDirectLoader), one ds_read_b128 per 16 x 32 / 32 x 16 operand tile (SharedToRegLoader on
//     MfmaTile operands), one v_mfma_f32_16x16x32_f16 per gemm() step, register double-buffering of the operand
//     tiles, XCD-aware tile order. It performs the arithmetic of kernels/gemm_pipelined.hpp in the same order
//     (results identical bit for bit).
// A is row-major [M, K], B is column-major [K, N] (stored [N, K]), C is row-major [M, N].
#pragma once

#include "cell/mod.hpp"
#include "kernels/gemm_pipelined.hpp"  // detail::xcd_tile_coords
#include "types/mod.hpp"

namespace tiledcuda::kernels {

using namespace tiledcuda::cell;
using namespace tiledcuda::cell::copy;
namespace tl = tile_layout;

template <const int kM, const int kN, const int kK>
using GemmShape = TileShape<kM, kN, kK>;

template <typename InType, typename AccType, typename WholeShape, const int kTM, const int kTN, typename WarpLayout,
          const int kChunkK_ = 64>
struct GemmTraits {
    using BaseShape = traits::BaseTileShape<InType>;
    static constexpr int kChunkK = kChunkK_;

    static constexpr int kThreads = tl::get_numel<WarpLayout> * kWaveSize;
    static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
    static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;

    static constexpr int kM = dim_size<0, WholeShape>;
    static constexpr int kN = dim_size<1, WholeShape>;
    static constexpr int kK = dim_size<2, WholeShape>;

    // operand A
    using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK, kK>>;
    using IteratorA = GTileIterator<GlobalA, TileShape<kTM, kChunkK>>;

    static constexpr int kAMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kAKs = kChunkK / BaseShape::kTileSize;
    using RegA = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAMs, kAKs>>;
    using ALoader = GlobalToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

    // operand B
    using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kTN, kK>>;
    using IteratorB = GTileIterator<GlobalB, TileShape<kChunkK, kTN>>;

    static constexpr int kBKs = kChunkK / BaseShape::kTileSize;
    static constexpr int kBNs = kTN / kWarpPerCol / BaseShape::kTileSize;
    using RegB = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kBKs, kBNs>>;
    using BLoader = GlobalToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

    // output C
    using GlobalC = GlobalTile<AccType, tl::RowMajor<kTM, kTN, kN>>;

    static constexpr int kCMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kCNs = kTN / kWarpPerCol / BaseShape::kTileSize;
    using RegC = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kCMs, kCNs>>;
    using CStorer = RegToGlobalStorer<GlobalC, RegC, WarpLayout>;
};

template <typename InType, typename AccType,                    //
          const int kM, const int kN, const int kK,             //
          const int kTM, const int kTN,                         //
          typename IteratorA, typename RegA, typename ALoader,  //
          typename IteratorB, typename RegB, typename BLoader,  //
          typename GlobalC, typename RegC, typename CStorer>
__global__ void __launch_bounds__(512) simple_gemm(const InType* dA, const InType* dB, AccType* dC) {
    const int offset_a = blockIdx.x * kTM * kK;
    const int offset_b = blockIdx.y * kTN * kK;
    const int offset_c = blockIdx.x * kTM * kN + blockIdx.y * kTN;

    IteratorA gAs(dA + offset_a);
    RegA rA;
    ALoader loader_a;

    IteratorB gBs(dB + offset_b);
    RegB rB;
    BLoader loader_b;

    RegC acc;
    GlobalC gC(dC + offset_c);
    CStorer storer_c;

    for (int k = 0; k < IteratorA::sc1; ++k) {
        loader_a(gAs(k), rA);
        loader_b(gBs(k), rB);
        compute::gemm(rA, rB, acc);
    }

    storer_c(acc, gC);
}

template <typename InType, typename AccType, typename WholeShape, typename CtaTileShape, const int kRK,
          typename WarpLayout>
struct KeGemmTraits {
    using BaseShape = traits::BaseTileShape<InType>;

    static constexpr int kThreads = tl::get_numel<WarpLayout> * kWaveSize;
    static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
    static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;

    static constexpr int kM = dim_size<0, WholeShape>;
    static constexpr int kN = dim_size<1, WholeShape>;
    static constexpr int kK = dim_size<2, WholeShape>;

    static constexpr int kTM = dim_size<0, CtaTileShape>;
    static constexpr int kTN = dim_size<1, CtaTileShape>;
    static constexpr int kTK = dim_size<2, CtaTileShape>;

    static const bool kSwizzled = true;

    // operand A
    using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK, kK>>;
    using GIteratorA = GTileIterator<GlobalA, TileShape<kTM, kTK>>;
    using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, kSwizzled>;
    using SIteratorA = STileIterator<SharedA, TileShape<kTM, kRK>>;

    static constexpr int kAMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kAKs = kRK / BaseShape::kTileSize;
    using RegA = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAMs, kAKs>>;

    using G2SLoaderA = GlobalToSharedLoader<SharedA, WarpLayout>;
    using S2RLoaderA = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

    // operand B
    using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kTN, kK>>;
    using GIteratorB = GTileIterator<GlobalB, TileShape<kTK, kTN>>;
    using SharedB = SharedTile<InType, tl::ColMajor<kTK, kTN>, kSwizzled>;
    using SIteratorB = STileIterator<SharedB, TileShape<kRK, kTN>>;

    static_assert(GIteratorA::sc1 == GIteratorB::sc0, "mismatched K dimension!");
    static_assert(SIteratorA::sc1 == SIteratorB::sc0, "mismatched K dimension!");

    static constexpr int kBKs = kRK / BaseShape::kTileSize;
    static constexpr int kBNs = kTN / kWarpPerCol / BaseShape::kTileSize;
    using RegB = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kBKs, kBNs>>;

    using G2SLoaderB = GlobalToSharedLoader<SharedB, WarpLayout>;
    using S2RLoaderB = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

    // output C
    using GlobalC = GlobalTile<AccType, tl::RowMajor<kTM, kTN, kN>>;
    using SharedC = SharedTile<AccType, tl::RowMajor<kTM, kTN>, kSwizzled>;

    static constexpr int kCMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kCNs = kTN / kWarpPerCol / BaseShape::kTileSize;
    using RegC = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kCMs, kCNs>>;

    using R2SStorerC = RegToSharedStorer<RegC, WarpLayout>;
    using S2GStorerC = SharedToGlobalStorer<SharedC, WarpLayout>;

    static constexpr int kShmInput = (kTM + kTN) * kTK * sizeof(InType);
    static constexpr int kShmOutput = kTM * kTN * sizeof(AccType);
    static constexpr int kShmBytes = kShmInput > kShmOutput ? kShmInput : kShmOutput;
};

template <typename InType, typename AccType,                  //
          const int kM, const int kN, const int kK,           //
          const int kTM, const int kTN, const int kTK,        //
          typename GIteratorA, typename SIteratorA,           //
          typename SharedA, typename RegA,                    //
          typename G2SLoaderA, typename S2RLoaderA,           //
          typename GIteratorB, typename SIteratorB,           //
          typename SharedB, typename RegB,                    //
          typename G2SLoaderB, typename S2RLoaderB,           //
          typename GlobalC, typename SharedC, typename RegC,  //
          typename R2SStorerC, typename S2GStorerC>
__global__ void __launch_bounds__(512) gemm(const InType* dA, const InType* dB, AccType* dC) {
    const int offset_a = blockIdx.x * kTM * kK;
    const int offset_b = blockIdx.y * kTN * kK;
    const int offset_c = blockIdx.x * kTM * kN + blockIdx.y * kTN;

    extern __shared__ __align__(16) unsigned char buf[];
    InType* sA_ptr = reinterpret_cast<InType*>(buf);
    InType* sB_ptr = sA_ptr + SIteratorA::Tile::kNumel;
    AccType* sC_ptr = reinterpret_cast<AccType*>(buf);

    GIteratorA gAs(dA + offset_a);
    SIteratorA sAs(sA_ptr);

    GIteratorB gBs(dB + offset_b);
    SIteratorB sBs(sB_ptr);

    SharedA sA(sA_ptr);
    RegA rA;

    SharedB sB(sB_ptr);
    RegB rB;

    RegC acc;
    SharedC sC(sC_ptr);
    GlobalC gC(dC + offset_c);

    G2SLoaderA g2s_a;
    S2RLoaderA s2r_a;

    G2SLoaderB g2s_b;
    S2RLoaderB s2r_b;

    R2SStorerC r2s_c;
    S2GStorerC s2g_c;

    for (int k1 = 0; k1 < GIteratorA::sc1; ++k1) {
        g2s_a(gAs(k1), sA);
        g2s_b(gBs(k1), sB);
        __copy_async();
        __syncthreads();

#pragma unroll
        for (int k2 = 0; k2 < SIteratorA::sc1; ++k2) {
            s2r_a(sAs(k2), rA);
            s2r_b(sBs(k2), rB);

            compute::gemm(rA, rB, acc);
        }
        __syncthreads();  // everyone is done reading sA / sB before the next step overwrites them
    }
    r2s_c(acc, sC);
    __syncthreads();
    s2g_c(sC, gC);
}

template <typename InType, typename OutType, typename WholeShape, const int kTM_, const int kTN_, typename WarpLayout>
struct PipelinedGemmTileTraits {
    static constexpr int kThreads = tl::get_numel<WarpLayout> * kWaveSize;
    static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
    static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;

    static constexpr int kM = dim_size<0, WholeShape>;
    static constexpr int kN = dim_size<1, WholeShape>;
    static constexpr int kK = dim_size<2, WholeShape>;
    static constexpr int kTM = kTM_, kTN = kTN_;
    static constexpr int kTK = 64;  // one LDS stage: lines of 128 bytes
    static constexpr int kRK = 32;  // one MFMA k-step
    static constexpr int kStages = 2;
    static_assert(kM % kTM == 0 && kN % kTN == 0 && kK % kTK == 0);

    using Shape = traits::MfmaTileShape<InType, traits::MfmaShape::k16x16x32>;

    // operand A
    using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK, kK>>;
    using GIteratorA = GTileIterator<GlobalA, TileShape<kTM, kTK>>;
    using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, true>;
    using RingA = SharedRing<SharedA, kStages>;
    using SIteratorA = STileIterator<SharedA, TileShape<kTM, kRK>>;
    using RegA = RegTile<typename Shape::TileA, tl::RowMajor<kTM / kWarpPerRow / Shape::kM, 1>>;
    using G2SLoaderA = GlobalToSharedDirectLoader<SharedA, WarpLayout>;
    using S2RLoaderA = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

    // operand B
    using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kTN, kK>>;
    using GIteratorB = GTileIterator<GlobalB, TileShape<kTK, kTN>>;
    using SharedB = SharedTile<InType, tl::ColMajor<kTK, kTN>, true>;
    using RingB = SharedRing<SharedB, kStages>;
    using SIteratorB = STileIterator<SharedB, TileShape<kRK, kTN>>;
    using RegB = RegTile<typename Shape::TileB, tl::ColMajor<1, kTN / kWarpPerCol / Shape::kN>>;
    using G2SLoaderB = GlobalToSharedDirectLoader<SharedB, WarpLayout>;
    using S2RLoaderB = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

    // output C
    static constexpr int kCMs = kTM / kWarpPerRow / 16, kCNs = kTN / kWarpPerCol / 16;
    using RegAcc = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kCMs, kCNs>>;
    using RegC = RegTile<BaseTileRowMajor<OutType>, tl::RowMajor<kCMs, kCNs>>;
    using SharedC = SharedTile<OutType, tl::RowMajor<kTM, kTN>, true>;
    using GlobalC = GlobalTile<OutType, tl::RowMajor<kTM, kTN, kN>>;
    using R2SStorerC = RegToSharedStorer<RegC, WarpLayout>;
    using S2GStorerC = SharedToGlobalStorer<SharedC, WarpLayout>;

    static constexpr int kShmInput = RingA::kBytes + RingB::kBytes;
    // an f32 result goes from registers straight to global memory; only f16 is staged through LDS
    static constexpr int kShmOutput = sizeof(OutType) == 2 ? kTM * kTN * int(sizeof(OutType)) : 0;
    static constexpr int kShmBytes = kShmInput > kShmOutput ? kShmInput : kShmOutput;
    static_assert(kShmBytes <= kMaxLdsBytes);
};

/// grid = (kM / kTM) * (kN / kTN) workgroups (1-D), block = Traits::kThreads, dynamic LDS = Traits::kShmBytes.
template <typename InType, typename OutType, typename Traits>
__global__ void __launch_bounds__(Traits::kThreads) gemm_tile_pipelined(const InType* dA, const InType* dB, OutType* dC) {
    constexpr int kM = Traits::kM, kN = Traits::kN, kK = Traits::kK, kTM = Traits::kTM, kTN = Traits::kTN;
    int tile_m, tile_n;
    detail::xcd_tile_coords(blockIdx.x, kM / kTM, kN / kTN, tile_m, tile_n);

    extern __shared__ __align__(1024) unsigned char buf[];
    auto* sA_ptr = reinterpret_cast<InType*>(buf);
    auto* sB_ptr = reinterpret_cast<InType*>(buf + Traits::RingA::kBytes);

    typename Traits::GIteratorA gAs(dA + size_t(tile_m) * kTM * kK);
    typename Traits::GIteratorB gBs(dB + size_t(tile_n) * kTN * kK);
    typename Traits::RingA ringA(sA_ptr);
    typename Traits::RingB ringB(sB_ptr);

    typename Traits::G2SLoaderA g2s_a;
    typename Traits::G2SLoaderB g2s_b;
    typename Traits::S2RLoaderA s2r_a;
    typename Traits::S2RLoaderB s2r_b;

    typename Traits::RegA rA[2];  // operand tiles of the k-step being multiplied and of the next one
    typename Traits::RegB rB[2];
    typename Traits::RegAcc acc;

    auto load_stage = [&](int k1, int stage) {
        auto sA = ringA[stage];
        auto sB = ringB[stage];
        g2s_a(gAs(k1), sA);
        g2s_b(gBs(k1), sB);
    };
    auto load_frags = [&](int stage, int k2, int which) {
        typename Traits::SIteratorA sAs(ringA.stage_data(stage));
        typename Traits::SIteratorB sBs(ringB.stage_data(stage));
        s2r_a(sAs(k2), rA[which]);
        s2r_b(sBs(k2), rB[which]);
    };

    constexpr int kTiles = Traits::GIteratorA::sc1;
    load_stage(0, 0);
    wait_group_and_barrier<0>();
    load_frags(0, 0, 0);

    int stage = 0;
    for (int k1 = 0; k1 < kTiles; ++k1) {
        const int next = Traits::RingA::next(stage);
        // tile k1 + 1 goes to the other stage, which everyone left at the hand-over of the previous iteration
        if (k1 + 1 < kTiles) load_stage(k1 + 1, next);
        // the copies are issued here, ahead of this iteration's matrix work (the compiler is otherwise free to sink
        // them below the MFMAs, right in front of the wait that needs them)
        commit_copy_group();
        load_frags(stage, 1, 1);
        compute::gemm(rA[0], rB[0], acc);
        commit_copy_group();
        if (k1 + 1 < kTiles) {
            // this wavefront's copies have landed and its reads of `stage` have returned; then everyone's
            wait_group_and_barrier<0>();
            load_frags(next, 0, 0);
        }
        compute::gemm(rA[1], rB[1], acc);
        stage = next;
    }

    typename Traits::GlobalC gC(dC + size_t(tile_m) * kTM * kN + size_t(tile_n) * kTN);
    if constexpr (std::is_same_v<OutType, float>) {
        RegToGlobalStorer<typename Traits::GlobalC, typename Traits::RegAcc, typename Traits::R2SStorerC::WarpLayout> r2g;
        r2g(acc, gC);
    } else {
        typename Traits::RegC out;
        compute::RegTileConvert<typename Traits::RegAcc, typename Traits::RegC> convert;
        convert(acc, out);
        __syncthreads();  // everyone is done with the operand stages: the space is reused for C
        typename Traits::SharedC sC(reinterpret_cast<OutType*>(buf));
        typename Traits::R2SStorerC r2s_c;
        typename Traits::S2GStorerC s2g_c;
        r2s_c(out, sC);
        __syncthreads();
        s2g_c(sC, gC);
    }
}

/// The one-wavefront-per-SIMD GEMM (kernels/gemm_w128.hpp, the kernel the large shapes run on) written with
/// tile-library functors only: 256 x 256 x 64 workgroup tile, 2 x 2 wavefronts of 128 x 128, two LDS stages.
template <typename InType, typename OutType, typename WholeShape>
struct ScheduledGemmTileTraits {
    using WarpLayout = tl::RowMajor<2, 2>;
    static constexpr int kThreads = 4 * kWaveSize;
    static constexpr int kM = dim_size<0, WholeShape>;
    static constexpr int kN = dim_size<1, WholeShape>;
    static constexpr int kK = dim_size<2, WholeShape>;
    static constexpr int kTM = 256, kTN = 256, kTK = 64, kRK = 32, kStages = 2;
    static_assert(kM % kTM == 0 && kN % kTN == 0 && kK % kTK == 0);

    using Shape = traits::MfmaTileShape<InType, traits::MfmaShape::k16x16x32>;
    static constexpr int kMs = kTM / 2 / Shape::kM, kNs = kTN / 2 / Shape::kN;  // 8 x 8 MFMA tiles per wavefront

    using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK, kK>>;
    using GIteratorA = GTileIterator<GlobalA, TileShape<kTM, kTK>>;
    using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, true>;
    using RingA = SharedRing<SharedA, kStages>;
    using SIteratorA = STileIterator<SharedA, TileShape<kTM, kRK>>;
    using RegA = RegTile<typename Shape::TileA, tl::RowMajor<kMs, 1>>;
    using PiecesA = GlobalToSharedDirectPieces<SharedA, WarpLayout, kK>;
    using S2RLoaderA = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

    using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kTN, kK>>;
    using GIteratorB = GTileIterator<GlobalB, TileShape<kTK, kTN>>;
    using SharedB = SharedTile<InType, tl::ColMajor<kTK, kTN>, true>;
    using RingB = SharedRing<SharedB, kStages>;
    using SIteratorB = STileIterator<SharedB, TileShape<kRK, kTN>>;
    using RegB = RegTile<typename Shape::TileB, tl::ColMajor<1, kNs>>;
    using PiecesB = GlobalToSharedDirectPieces<SharedB, WarpLayout, kK>;
    using S2RLoaderB = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

    using RegAcc = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kMs, kNs>>;
    using RegC = RegTile<BaseTileRowMajor<OutType>, tl::RowMajor<kMs, kNs>>;
    using SharedC = SharedTile<OutType, tl::RowMajor<kTM, kTN>, true>;
    using GlobalC = GlobalTile<OutType, tl::RowMajor<kTM, kTN, kN>>;
    using R2SStorerC = RegToSharedStorer<RegC, WarpLayout>;
    using S2GStorerC = SharedToGlobalStreamStorer<SharedC, WarpLayout>;  // whole rows, never read again: streamed out

    static constexpr int kShmInput = RingA::kBytes + RingB::kBytes;
    static constexpr int kShmOutput = sizeof(OutType) == 2 ? kTM * kTN * int(sizeof(OutType)) : 0;
    static constexpr int kShmBytes = kShmInput > kShmOutput ? kShmInput : kShmOutput;
    static_assert(kShmBytes <= kMaxLdsBytes);
    static_assert(PiecesA::kPieces == 8 && PiecesB::kPieces == 8 && kMs == 8 && kNs == 8,
                  "the schedule below deals 16 loads and 16 fragment reads over 64 matrix instructions");
};

/// grid = (kM / 256) * (kN / 256) workgroups (1-D), block = 256, dynamic LDS = Traits::kShmBytes.
/// A tile of K is two gemm_scheduled calls of 64 matrix instructions (k-steps 0 and 1). The hook of the first reads
/// the 16 operand fragments of k-step 1, one per two instructions; then one LDS-only barrier (tile k1 + 1 has landed,
/// everyone has left tile k1's stage); the hook of the second reads the fragments of tile k1 + 1 / k-step 0 and hands
/// gemm_scheduled this wavefront's 16 loads of tile k1 + 2, one per four instructions, into the stage just vacated.
/// The schedule, the operand order and therefore the sums are those of gemm_w128 (bit-identical results).
template <typename InType, typename OutType, typename Traits>
__global__ void __launch_bounds__(Traits::kThreads) gemm_tile_w128(const InType* dA, const InType* dB, OutType* dC) {
    constexpr int kM = Traits::kM, kN = Traits::kN, kK = Traits::kK, kTM = Traits::kTM, kTN = Traits::kTN;
    int tile_m, tile_n;
    detail::xcd_tile_coords(blockIdx.x, kM / kTM, kN / kTN, tile_m, tile_n);

    extern __shared__ __align__(1024) unsigned char buf[];
    typename Traits::GIteratorA gAs(dA + size_t(tile_m) * kTM * kK);
    typename Traits::GIteratorB gBs(dB + size_t(tile_n) * kTN * kK);
    typename Traits::RingA ringA(reinterpret_cast<InType*>(buf));
    typename Traits::RingB ringB(reinterpret_cast<InType*>(buf + Traits::RingA::kBytes));

    typename Traits::PiecesA pieces_a;
    typename Traits::PiecesB pieces_b;
    typename Traits::S2RLoaderA s2r_a;
    typename Traits::S2RLoaderB s2r_b;

    typename Traits::RegA rA[2];  // operand tiles of k-step 0 / k-step 1
    typename Traits::RegB rB[2];
    typename Traits::RegAcc acc;

    // load q of this wavefront for tile k1 (q < 8: a piece of A, else of B)
    auto load = [&](int k1, int stage, int q) -> DirectLoad {
        return q < 8 ? pieces_a.piece(q, gAs(k1).data(), ringA[stage]) : pieces_b.piece(q - 8, gBs(k1).data(), ringB[stage]);
    };
    // fragment r of k-step k2 of the tile in `stage`, in the order the next 64 instructions need them: row 0 of A and
    // all of B first
    auto read_fragment = [&](int stage, int k2, int which, int r) {
        typename Traits::SIteratorA sAs(ringA.stage_data(stage));
        typename Traits::SIteratorB sBs(ringB.stage_data(stage));
        if (r == 0) s2r_a.load_one(sAs(k2), rA[which], 0, 0);
        else if (r <= 8) s2r_b.load_one(sBs(k2), rB[which], 0, r - 1);
        else s2r_a.load_one(sAs(k2), rA[which], r - 8, 0);
    };

    constexpr int kTiles = Traits::GIteratorA::sc1;
#pragma unroll
    for (int q = 0; q < 16; ++q) issue(load(0, 0, q));
    if constexpr (kTiles > 1) {
#pragma unroll
        for (int q = 0; q < 16; ++q) issue(load(1, 1, q));
    }
    compute::clear_pinned(acc);  // while the first tiles are on their way
    if constexpr (kTiles > 1) wait_group_and_barrier<16>();  // tile 0 has landed, for everyone
    else wait_group_and_barrier<0>();
#pragma unroll
    for (int r = 0; r < 16; ++r) read_fragment(0, 0, 0, r);

    // kMore: there is a tile k1 + 1; kMore2: there is a tile k1 + 2
    // (stage: k1 % 2 - a constant in the loop unrolled by two, so that the addresses there are immediates)
    auto tile = [&](int k1, auto more_c, auto more2_c, auto stage_v) __attribute__((always_inline)) {
        constexpr bool kMore = decltype(more_c)::value, kMore2 = decltype(more2_c)::value;
        const int stage = stage_v;
        compute::gemm_scheduled(rA[0], rB[0], acc, [&](auto n_c) {
            constexpr int n = decltype(n_c)::value;
            if constexpr (n % 2 == 0 && n / 2 < 16) read_fragment(stage, 1, 1, n / 2);
        });
        wait_group_and_barrier<0>();
        compute::gemm_scheduled(rA[1], rB[1], acc, [&](auto n_c) {
            constexpr int n = decltype(n_c)::value;
            if constexpr (kMore && n % 2 == 0 && n / 2 < 16) read_fragment(stage ^ 1, 0, 0, n / 2);
            if constexpr (kMore2 && n % 4 == 1) return load(k1 + 2, stage, n / 4);
        });
    };
    {
        int k1 = 0;
        for (; k1 + 3 < kTiles; k1 += 2) {
            tile(k1, std::true_type{}, std::true_type{}, std::integral_constant<int, 0>{});
            tile(k1 + 1, std::true_type{}, std::true_type{}, std::integral_constant<int, 1>{});
        }
        for (; k1 + 2 < kTiles; ++k1) tile(k1, std::true_type{}, std::true_type{}, k1 & 1);
        if (k1 + 1 < kTiles) {
            tile(k1, std::true_type{}, std::false_type{}, k1 & 1);
            ++k1;
        }
        tile(k1, std::false_type{}, std::false_type{}, k1 & 1);
    }
    compute::settle_accumulators(acc);

    typename Traits::GlobalC gC(dC + size_t(tile_m) * kTM * kN + size_t(tile_n) * kTN);
    if constexpr (std::is_same_v<OutType, float>) {
        RegToGlobalStorer<typename Traits::GlobalC, typename Traits::RegAcc, typename Traits::WarpLayout> r2g;
        r2g(acc, gC);
    } else {
        typename Traits::RegC out;
        compute::RegTileConvert<typename Traits::RegAcc, typename Traits::RegC> convert;
        convert(acc, out);
        __syncthreads();  // everyone is done with the operand stages: the space is reused for C
        typename Traits::SharedC sC(reinterpret_cast<OutType*>(buf));
        typename Traits::R2SStorerC r2s_c;
        typename Traits::S2GStorerC s2g_c;
        r2s_c(out, sC);
        __syncthreads();
        s2g_c(sC, gC);
    }
}

}  // namespace tiledcuda::kernels
