// Back-to-back GEMM D = (A·B)·C with the [kTM x kTN] intermediate kept in registers.
// Follows the structure of the reference's examples/cpp/02_fused_two_gemms/fused_gemm.hpp:12-181
// (FusedGemmTraits / KeFusedGemm): A, D row-major; B, C column-major; the f32 accumulator of
// the first product is rounded to f16 and used as the A operand of the second one.
// Differences: M and the batch count are run-time values (every stride depends only on
// N, K, P), D may be f16 or f32, and A is read from global memory once, before the n-loop
// (the reference re-reads it on every iteration, fused_gemm.hpp:156).
#pragma once

#include "cell/mod.hpp"
#include "types/mod.hpp"

namespace tiledcuda::kernels {

using namespace tiledcuda::cell;
using namespace tiledcuda::cell::copy;
namespace tl = tile_layout;

template <const int kM, const int kN, const int kK, const int kP>
using FusedGemmShape = TileShape<kM, kN, kK, kP>;

/// WholeShape carries N, K, P (M is a run-time argument of the kernel; its entry in the
/// shape is only used for documentation).
template <typename InType, typename AccType, typename OutType, typename WholeShape, typename CtaTileShape,
          typename WarpLayout_ = tl::RowMajor<2, 1>>
struct FusedGemmTraits {
    using BaseShape = traits::BaseTileShape<InType>;
    using WarpLayout = WarpLayout_;

    static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
    static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;
    static_assert(kWarpPerCol == 1, "WarpPerCol must be 1");

    static constexpr int kThreads = tl::get_numel<WarpLayout> * kWaveSize;

    static constexpr int kN = dim_size<1, WholeShape>;
    static constexpr int kK = dim_size<2, WholeShape>;
    static constexpr int kP = dim_size<3, WholeShape>;

    static constexpr int kTM = dim_size<0, CtaTileShape>;
    static constexpr int kTN = dim_size<1, CtaTileShape>;
    static constexpr int kTK = dim_size<2, CtaTileShape>;
    static constexpr int kTP = dim_size<3, CtaTileShape>;
    static_assert(kTK == kK, "The current implementation requires kTK == K.");
    static_assert(kTP == kP, "The current implementation requires kTP == P.");

    // operand A [M, K] row-major
    using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK, kK>>;
    using GIteratorA = GTileIterator<GlobalA, TileShape<kTM, kTK>>;
    using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, true>;

    static constexpr int kAMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kAKs = kTK / BaseShape::kTileSize;
    using RegA = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAMs, kAKs>>;
    using SharedALoader = GlobalToSharedLoader<SharedA, WarpLayout>;
    using RegALoader = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

    // operand B [K, N] column-major
    using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kN, kK>>;
    using GIteratorB = GTileIterator<GlobalB, TileShape<kTK, kTN>>;
    using SharedB = SharedTile<InType, tl::ColMajor<kTK, kTN>, true>;

    static constexpr int kBKs = kTK / BaseShape::kTileSize;
    static constexpr int kBNs = kTN / kWarpPerCol / BaseShape::kTileSize;
    using RegB = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kBKs, kBNs>>;
    using SharedBLoader = GlobalToSharedLoader<SharedB, WarpLayout>;
    using RegBLoader = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

    // operand C [N, P] column-major
    using GlobalC = GlobalTile<InType, tl::ColMajor<kN, kTP, kN>>;
    using GIteratorC = GTileIterator<GlobalC, TileShape<kTN, kTP>>;
    using SharedC = SharedTile<InType, tl::ColMajor<kTN, kTP>, true>;

    static constexpr int kCNs = kTN / BaseShape::kTileSize;
    static constexpr int kCPs = kTP / kWarpPerCol / BaseShape::kTileSize;
    using RegC = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kCNs, kCPs>>;
    using SharedCLoader = GlobalToSharedLoader<SharedC, WarpLayout>;
    using RegCLoader = SharedToRegLoader<RegC, WarpLayout, WarpReuse::kColReuseCont>;

    // output D [M, P] row-major
    using GlobalD = GlobalTile<OutType, tl::RowMajor<kTM, kTP, kP>>;

    static constexpr int kDMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kDPs = kTP / kWarpPerCol / BaseShape::kTileSize;
    using RegD = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kDMs, kDPs>>;
    using RegDCast = RegTile<BaseTileRowMajor<OutType>, tl::RowMajor<kDMs, kDPs>>;
    using DStorer = RegToGlobalStorer<GlobalD, RegDCast, WarpLayout>;
    using ConvertD = compute::RegTileConvert<RegD, RegDCast>;

    static constexpr int kAccMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kAccNs = kTN / kWarpPerCol / BaseShape::kTileSize;
    using RegAcc = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kAccMs, kAccNs>>;
    using RegAccCast = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAccMs, kAccNs>>;
    using ConvertAcc = compute::RegTileConvert<RegAcc, RegAccCast>;

    static constexpr int kShmBytes = (kTM * kTK + kTK * kTN + kTN * kTP) * sizeof(InType);
};

/// grid = (M / kTM, 1, batch), block = Traits::kThreads, dynamic LDS = Traits::kShmBytes.
template <typename InType, typename OutType, typename Traits>
__global__ void __launch_bounds__(Traits::kThreads) KeFusedGemm(const InType* dA, const InType* dB, const InType* dC,
                                                                OutType* dD, int kM) {
    constexpr int kN = Traits::kN, kK = Traits::kK, kP = Traits::kP;
    constexpr int kTM = Traits::kTM;

    const InType* A = dA + blockIdx.z * (size_t(kM) * kK) + blockIdx.x * (kTM * kK);
    const InType* B = dB + blockIdx.z * (kK * kN);
    const InType* gC_ptr = dC + blockIdx.z * (kN * kP);
    OutType* gD_ptr = dD + blockIdx.z * (size_t(kM) * kP) + blockIdx.x * (kTM * kP);

    extern __shared__ __align__(16) unsigned char shared_buf[];
    auto* shm = reinterpret_cast<InType*>(shared_buf);
    InType* sA_ptr = shm;
    InType* sB_ptr = shm + Traits::SharedA::kNumel;
    InType* sC_ptr = sB_ptr + Traits::SharedB::kNumel;

    typename Traits::GIteratorA gAs(A);
    typename Traits::SharedA sA(sA_ptr);
    typename Traits::RegA rA;
    typename Traits::SharedALoader load_sa;
    typename Traits::RegALoader load_ra;

    typename Traits::GIteratorB gBs(B);
    typename Traits::SharedB sB(sB_ptr);
    typename Traits::RegB rB;
    typename Traits::SharedBLoader load_sb;
    typename Traits::RegBLoader load_rb;

    typename Traits::GIteratorC gCs(gC_ptr);
    typename Traits::SharedC sC(sC_ptr);
    typename Traits::RegC rC;
    typename Traits::SharedCLoader load_sc;
    typename Traits::RegCLoader load_rc;

    typename Traits::RegD rD;
    typename Traits::RegAcc acc;
    typename Traits::RegAccCast acc_half;
    typename Traits::ConvertAcc cast_acc;

    // A is needed by every n-iteration: stage it once and keep it in registers.
    load_sa(gAs(0), sA);
    __copy_async();
    __syncthreads();
    load_ra(sA, rA);

    for (int n = 0; n < Traits::GIteratorC::sc0; ++n) {
        load_sb(gBs(0, n), sB);
        load_sc(gCs(n), sC);
        __copy_async();
        __syncthreads();

        load_rb(sB, rB);
        load_rc(sC, rC);
        __syncthreads();

        compute::gemm(rA, rB, acc);
        cast_acc(acc, acc_half);
        compute::gemm(acc_half, rC, rD);
        acc.clear();
    }

    typename Traits::RegDCast rD_out;
    typename Traits::ConvertD cast_d;
    cast_d(rD, rD_out);

    typename Traits::GlobalD gD(gD_ptr);
    typename Traits::DStorer storer_d;
    storer_d(rD_out, gD);
}

/// The LDS-resident back-to-back GEMM (kernels/b2b_gemm_fwd.hpp, what K = P = 128 runs on) written with tile-library
/// types and functors only. Against KeFusedGemm above: every operand goes global -> LDS directly
/// (GlobalToSharedDirectLoader), all of a block's loads in flight at once and handed over with
/// wait_group_and_barrier<N>(); the products run on v_mfma_f32_16x16x32_f16 operand tiles (one ds_read_b128 per tile);
/// the 8 wavefronts split the first product by n and the second by p, so the f16-rounded intermediate crosses
/// wavefronts through a shared tile (RegToSharedStorer / SharedToRegLoader) instead of staying in one wavefront's
/// registers - which is what lets 32 rows keep a whole CU busy. N is walked in blocks of 256 through the same shared
/// tiles: B is refilled under the second product of the current block, C under the first product of the next.
/// The sums are those of b2b_gemm_resident in the same order: bit-identical results.
/// kK_, kP_: the inner sizes (whole, resident); kTN_: columns of B / rows of C per block; kWaves_: wavefronts, each of
/// which owns kTN / kWaves values of n in the first product and kP / kWaves values of p in the second (multiples of
/// 16). The defaults are the K = P = 128 configuration; <N, 64, 64, 128, 4> serves K = P = 64.
template <typename InType, typename OutType, const int kN_, const int kK_ = 128, const int kP_ = 128, const int kTN_ = 256,
          const int kWaves_ = 8>
struct ResidentFusedGemmTraits {
    static constexpr int kN = kN_, kK = kK_, kP = kP_;
    static constexpr int kTM = 32, kTN = kTN_;
    static_assert(kN % kTN == 0 && kK % 32 == 0 && kTN % 32 == 0);
    static constexpr int kWaves = kWaves_, kThreads = kWaves * kWaveSize;
    static_assert(kTN % (16 * kWaves) == 0 && kP % (16 * kWaves) == 0, "every wavefront owns whole 16-wide tiles of n and of p");
    using WarpLayout = tl::RowMajor<1, kWaves>;
    using Shape = traits::MfmaTileShape<InType, traits::MfmaShape::k16x16x32>;

    using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK>>;
    using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kTN>>;       // 256 columns of B: 256 rows of the stored [N, K]
    using GlobalC = GlobalTile<InType, tl::ColMajor<kTN, kP, kN>>;   // 256 rows of C: columns of the stored [P, N]
    using GlobalD = GlobalTile<OutType, tl::RowMajor<kTM, kP>>;
    using SharedA = SharedTile<InType, tl::RowMajor<kTM, kK>, true>;
    using SharedB = SharedTile<InType, tl::ColMajor<kK, kTN>, true>;
    using SharedC = SharedTile<InType, tl::ColMajor<kTN, kP>, true>;
    using SharedS = SharedTile<InType, tl::RowMajor<kTM, kTN>, true>;  // the intermediate of one block
    // a 2-byte output tile is gathered in LDS behind the operands and leaves as whole rows (SharedToGlobalStreamStorer);
    // a 4-byte one would not fit beside them and goes from registers to memory
    static constexpr bool kStageD = sizeof(OutType) == 2;
    using SharedD = SharedTile<OutType, tl::RowMajor<kTM, kP>, true>;
    static constexpr int kShmOperands =
        (SharedA::kNumel + SharedB::kNumel + SharedC::kNumel + SharedS::kNumel) * int(sizeof(InType));  // 152 KiB by default
    static constexpr int kShmBytes = kShmOperands + (kStageD ? SharedD::kNumel * int(sizeof(OutType)) : 0);  // 160 KiB
    static_assert(kShmBytes <= kMaxLdsBytes);

    using LoadA = GlobalToSharedDirectLoader<SharedA, WarpLayout>;
    using LoadB = GlobalToSharedDirectLoader<SharedB, WarpLayout>;
    using LoadC = GlobalToSharedDirectLoader<SharedC, WarpLayout>;
    static constexpr int kLoadsC = LoadC::kLoadsPerWave;  // the youngest loads of a block: still in flight at its first hand-over

    // first product: a wavefront owns 32 values of n
    using RegA = RegTile<typename Shape::TileA, tl::RowMajor<kTM / 16, kK / 32>>;
    using RegB = RegTile<typename Shape::TileB, tl::ColMajor<kK / 32, kTN / kWaves / 16>>;
    using RegAcc = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kTM / 16, kTN / kWaves / 16>>;
    using RegAccCast = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kTM / 16, kTN / kWaves / 16>>;
    using ReadA = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;
    using ReadB = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;
    using ConvertAcc = compute::RegTileConvert<RegAcc, RegAccCast>;
    using StoreS = RegToSharedStorer<RegAccCast, WarpLayout>;
    // second product: a wavefront owns 16 values of p
    using RegS = RegTile<typename Shape::TileA, tl::RowMajor<kTM / 16, kTN / 32>>;
    using RegC = RegTile<typename Shape::TileB, tl::ColMajor<kTN / 32, kP / kWaves / 16>>;
    using RegD = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kTM / 16, kP / kWaves / 16>>;
    using RegDCast = RegTile<BaseTileRowMajor<OutType>, tl::RowMajor<kTM / 16, kP / kWaves / 16>>;
    using ReadS = SharedToRegLoader<RegS, WarpLayout, WarpReuse::kRowReuseCont>;
    using ReadC = SharedToRegLoader<RegC, WarpLayout, WarpReuse::kColReuseCont>;
    using ConvertD = compute::RegTileConvert<RegD, RegDCast>;
    using StoreD = RegToGlobalStorer<GlobalD, RegDCast, WarpLayout>;
    using StageD = RegToSharedStorer<RegDCast, WarpLayout>;
    using StreamD = SharedToGlobalStreamStorer<SharedD, WarpLayout>;
};

/// grid = (M / 32, batch), block = 512, dynamic LDS = Traits::kShmBytes.
template <typename InType, typename OutType, typename Traits>
__global__ void __launch_bounds__(Traits::kThreads)
    b2b_gemm_tile_resident(const InType* dA, const InType* dB, const InType* dC, OutType* dD, int kM) {
    constexpr int kN = Traits::kN, kK = Traits::kK, kP = Traits::kP, kTM = Traits::kTM, kTN = Traits::kTN;
    constexpr int kBlocks = kN / kTN;
    const size_t batch = blockIdx.y;
    const InType* A = dA + (batch * kM + size_t(blockIdx.x) * kTM) * kK;
    const InType* B = dB + batch * size_t(kN) * kK;
    const InType* C = dC + batch * size_t(kP) * kN;
    OutType* D = dD + (batch * kM + size_t(blockIdx.x) * kTM) * kP;

    extern __shared__ __align__(1024) unsigned char shared_buf[];
    auto* shm = reinterpret_cast<InType*>(shared_buf);
    typename Traits::SharedA sA(shm);
    typename Traits::SharedB sB(shm + Traits::SharedA::kNumel);
    typename Traits::SharedC sC(shm + Traits::SharedA::kNumel + Traits::SharedB::kNumel);
    typename Traits::SharedS sS(shm + Traits::SharedA::kNumel + Traits::SharedB::kNumel + Traits::SharedC::kNumel);

    typename Traits::LoadA load_a;
    typename Traits::LoadB load_b;
    typename Traits::LoadC load_c;
    auto block_b = [&](int nb) { return typename Traits::GlobalB(B + size_t(nb) * kTN * kK); };
    auto block_c = [&](int nb) { return typename Traits::GlobalC(C + size_t(nb) * kTN); };

    // everything of the first block in flight at once: one memory round trip when N is a single block
    load_a(typename Traits::GlobalA(A), sA);
    load_b(block_b(0), sB);
    load_c(block_c(0), sC);

    typename Traits::ReadA read_a;
    typename Traits::ReadB read_b;
    typename Traits::ReadS read_s;
    typename Traits::ReadC read_c;
    typename Traits::ConvertAcc cast_acc;
    typename Traits::StoreS store_s;

    typename Traits::RegA rA;
    typename Traits::RegB rB;
    typename Traits::RegS rS;
    typename Traits::RegC rC;
    typename Traits::RegAcc acc;
    typename Traits::RegAccCast acc_half;
    typename Traits::RegD rD;

    for (int nb = 0; nb < kBlocks; ++nb) {
        // A and this block of B have landed (the younger loads, of C, may still be on their way), for everyone; and
        // everyone is done with the previous block's C and intermediate
        wait_group_and_barrier<Traits::kLoadsC>();
        if (nb == 0) read_a(sA, rA);
        read_b(sB, rB);
        acc.clear();
        compute::gemm(rA, rB, acc);
        cast_acc(acc, acc_half);  // the intermediate is rounded to f16: part of the operation's specification
        store_s(acc_half, sS);
        wait_group_and_barrier<0>();  // C has landed, the intermediate is written, B is free; for everyone
        if (nb + 1 < kBlocks) load_b(block_b(nb + 1), sB);  // under the second product
        read_s(sS, rS);
        read_c(sC, rC);
        compute::gemm(rS, rC, rD);
        if (nb + 1 < kBlocks) {
            // everyone's reads of C and of the intermediate have returned: C is refilled under the next first product
            __syncthreads();
            load_c(block_c(nb + 1), sC);
        }
    }

    typename Traits::RegDCast rD_out;
    typename Traits::ConvertD cast_d;
    cast_d(rD, rD_out);
    typename Traits::GlobalD gD(D);
    if constexpr (Traits::kStageD) {
        typename Traits::SharedD sD(reinterpret_cast<OutType*>(shared_buf + Traits::kShmOperands));
        typename Traits::StageD stage_d;
        typename Traits::StreamD stream_d;
        stage_d(rD_out, sD);
        __syncthreads();
        stream_d(sD, gD);
    } else {
        typename Traits::StoreD store_d;
        store_d(rD_out, gD);
    }
}

}  // namespace tiledcuda::kernels
