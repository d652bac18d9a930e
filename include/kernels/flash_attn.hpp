// FlashAttention forward, O = softmax(scale · Q·K)·V, composed from the tile primitives.
// Follows the structure of the reference's src/kernels/flash_attn.cu:18-312
// (FlashAttentionTraits / flash_attention: one workgroup per kTM query rows, wavefronts
// stacked along the rows, K/V streamed in kTN-long blocks through LDS, online softmax).
//
// Numerics differ from the reference on purpose: the running row maximum and row sum and
// the output accumulator are f32 (the reference keeps them in f16, flash_attn.cu:109,193-211),
// the maximum starts at -inf (the reference starts at 0 because every RegTile is
// zero-filled), the softmax scale is applied, and the output is rescaled lazily and
// normalised once at the end (FlashAttention-2) instead of every block (:290-297).
// Q is read from global memory once (the reference re-reads it per block, :241).
// Two kernels: flash_attention keeps the reference's single-stage structure (register-staged copies between two
// barriers per block); flash_attention_pipelined is the same composition with the K/V blocks double-buffered through
// direct-to-LDS loads (2.3 x faster at B4 H16 S2048 D128 with 128-row tiles).
//
// Layouts: Q row-major [M, K]; K column-major [K, N] (= [N, K] row-major, "keys as rows");
// V column-major [N, P] (the reference boundary) or row-major [N, P] (kVRowMajor);
// O row-major [M, P]. M, N and the batch count are run-time values when V is row-major;
// with a column-major V the leading dimension of V is N, so N is a template parameter.
#pragma once

#include "cell/mod.hpp"
#include "types/mod.hpp"

namespace tiledcuda::kernels {

using namespace tiledcuda::cell;
using namespace tiledcuda::cell::copy;
namespace tl = tile_layout;

template <const int kM, const int kN, const int kK, const int kP>
using FlashAttentionShape = TileShape<kM, kN, kK, kP>;

template <typename InType, typename AccType, typename OutType, typename WholeShape, typename CtaTileShape,
          const bool kVRowMajor_ = false, typename WarpLayout_ = tl::RowMajor<4, 1>>
struct FlashAttentionTraits {
    using BaseShape = traits::BaseTileShape<InType>;
    using WarpLayout = WarpLayout_;
    static constexpr bool kVRowMajor = kVRowMajor_;

    static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
    static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;
    static_assert(kWarpPerCol == 1, "WarpPerCol must be 1");

    static constexpr int kThreads = tl::get_numel<WarpLayout> * kWaveSize;

    static constexpr int kN = dim_size<1, WholeShape>;  // leading dimension of a column-major V
    static constexpr int kK = dim_size<2, WholeShape>;
    static constexpr int kP = dim_size<3, WholeShape>;

    static constexpr int kTM = dim_size<0, CtaTileShape>;
    static constexpr int kTN = dim_size<1, CtaTileShape>;
    static constexpr int kTK = dim_size<2, CtaTileShape>;
    static constexpr int kTP = dim_size<3, CtaTileShape>;
    static_assert(kK == kTK, "The current implementation requires kTK == K.");
    static_assert(kP == kTP, "The current implementation requires kTP == P.");

    // Q
    using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK>>;
    using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, true>;
    static constexpr int kAMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kAKs = kTK / BaseShape::kTileSize;
    using RegA = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAMs, kAKs>>;
    using SharedALoader = GlobalToSharedLoader<SharedA, WarpLayout>;
    using RegALoader = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

    // K block [kTK, kTN], column-major with leading dimension kK
    using GlobalB = GlobalTile<InType, tl::ColMajor<kTK, kTN, kK>>;
    using SharedB = SharedTile<InType, tl::ColMajor<kTK, kTN>, true>;
    static constexpr int kBKs = kTK / BaseShape::kTileSize;
    static constexpr int kBNs = kTN / kWarpPerCol / BaseShape::kTileSize;
    using RegB = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kBKs, kBNs>>;
    using SharedBLoader = GlobalToSharedLoader<SharedB, WarpLayout>;
    using RegBLoader = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

    // V block [kTN, kTP]
    using GlobalC = std::conditional_t<kVRowMajor, GlobalTile<InType, tl::RowMajor<kTN, kTP, kP>>,
                                       GlobalTile<InType, tl::ColMajor<kTN, kTP, kN>>>;
    using SharedC = std::conditional_t<kVRowMajor, SharedTile<InType, tl::RowMajor<kTN, kTP>, true>,
                                       SharedTile<InType, tl::ColMajor<kTN, kTP>, true>>;
    static constexpr int kCNs = kTN / BaseShape::kTileSize;
    static constexpr int kCPs = kTP / kWarpPerCol / BaseShape::kTileSize;
    using RegC = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kCNs, kCPs>>;
    using SharedCLoader = GlobalToSharedLoader<SharedC, WarpLayout>;
    using RegCLoader = SharedToRegLoader<RegC, WarpLayout, WarpReuse::kColReuseCont>;

    // O
    using GlobalD = GlobalTile<OutType, tl::RowMajor<kTM, kTP>>;
    static constexpr int kDMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kDPs = kTP / kWarpPerCol / BaseShape::kTileSize;
    using RegD = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kDMs, kDPs>>;
    using RegDCast = RegTile<BaseTileRowMajor<OutType>, tl::RowMajor<kDMs, kDPs>>;
    using DStorer = RegToGlobalStorer<GlobalD, RegDCast, WarpLayout>;

    // attention block
    static constexpr int kAccMs = kTM / kWarpPerRow / BaseShape::kTileSize;
    static constexpr int kAccNs = kTN / kWarpPerCol / BaseShape::kTileSize;
    using RegAcc = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kAccMs, kAccNs>>;
    using RegAccCast = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAccMs, kAccNs>>;

    using ConvertHalf = compute::RegTileConvert<RegAcc, RegAccCast>;
    using ConvertO = compute::RegTileConvert<RegD, RegDCast>;

    // one f32 statistic per BaseTile row per lane
    using RegVec = RegTile<AccType, tl::RowMajor<kAccMs, 1>>;

    using CopyVec = copy::BaseTileCopy<RegVec>;
    using RowMax = compute::MaxReduce<RegAcc, tl::Layout::kRowMajor>;
    using RowSum = compute::SumReduce<RegAcc, tl::Layout::kRowMajor>;

    using BroadcastSub = compute::BroadcastSub<RegVec, RegAcc, tl::Layout::kRowMajor>;
    using BroadcastMul = compute::BroadcastMul<RegVec, RegD, tl::Layout::kRowMajor>;
    using BroadcastDiv = compute::BroadcastDiv<RegVec, RegD, tl::Layout::kRowMajor>;

    using BlockExp = compute::RegTileExp<RegAcc>;

    using VecMax = compute::BaseTileMax<RegVec>;
    using VecAdd = compute::BaseTileAdd<RegVec>;
    using VecSub = compute::BaseTileSub<RegVec>;
    using VecMul = compute::BaseTileMul<RegVec>;
    using VecExp = compute::BaseTileExp<RegVec>;

    static constexpr int kShmBytes = (kTM * kTK + kTK * kTN + kTN * kTP) * sizeof(InType);

    // the same kernel on the direct-to-LDS path (flash_attention_pipelined): K and V blocks in two-stage rings
    using DirectALoader = GlobalToSharedDirectLoader<SharedA, WarpLayout>;
    using DirectBLoader = GlobalToSharedDirectLoader<SharedB, WarpLayout>;
    using DirectCLoader = GlobalToSharedDirectLoader<SharedC, WarpLayout>;
    using RingB = SharedRing<SharedB, 2>;
    using RingC = SharedRing<SharedC, 2>;
    // Q is only in LDS until it has been read into registers: it shares the rings' bytes
    static constexpr int kRingBytes = RingB::kBytes + RingC::kBytes;
    static constexpr int kShmBytesPipelined = kRingBytes > int(SharedA::kNumel * sizeof(InType))
                                                  ? kRingBytes : int(SharedA::kNumel * sizeof(InType));
};

/// grid = (M / kTM, 1, batch), block = Traits::kThreads, dynamic LDS = Traits::kShmBytes.
/// kM, kN: query rows and keys per batch item.
template <typename InType, typename OutType, typename Traits>
__global__ void __launch_bounds__(Traits::kThreads)
    flash_attention(const InType* dQ, const InType* dK, const InType* dV, OutType* dO, int kM, int kN, float scale) {
    constexpr int kK = Traits::kK, kP = Traits::kP;
    constexpr int kTM = Traits::kTM, kTN = Traits::kTN;
    using AccType = float;

    const InType* Q = dQ + blockIdx.z * (size_t(kM) * kK) + blockIdx.x * (kTM * kK);
    const InType* K = dK + blockIdx.z * (size_t(kN) * kK);
    const InType* V = dV + blockIdx.z * (size_t(kN) * kP);
    OutType* gO_ptr = dO + blockIdx.z * (size_t(kM) * kP) + blockIdx.x * (kTM * kP);

    extern __shared__ __align__(16) unsigned char shared_buf[];
    auto* shm = reinterpret_cast<InType*>(shared_buf);
    InType* sQ_ptr = shm;
    InType* sK_ptr = shm + Traits::SharedA::kNumel;
    InType* sV_ptr = sK_ptr + Traits::SharedB::kNumel;

    typename Traits::SharedA sQ(sQ_ptr);
    typename Traits::RegA rQ;
    typename Traits::SharedALoader load_sq;
    typename Traits::RegALoader load_rq;

    typename Traits::SharedB sK(sK_ptr);
    typename Traits::RegB rK;
    typename Traits::SharedBLoader load_sk;
    typename Traits::RegBLoader load_rk;

    typename Traits::SharedC sV(sV_ptr);
    typename Traits::RegC rV;
    typename Traits::SharedCLoader load_sv;
    typename Traits::RegCLoader load_rv;

    typename Traits::RegD rO;           // unnormalised output, f32
    typename Traits::RegAcc attn_block;  // scores, then probabilities, f32
    typename Traits::RegAccCast attn_half;

    typename Traits::RegVec run_max, run_sum, cur_max, cur_sum, new_max, rescale;
#pragma unroll
    for (int i = 0; i < Traits::RegVec::kRows; ++i) run_max(i, 0) = -INFINITY;

    typename Traits::RowMax row_max;
    typename Traits::RowSum row_sum;
    typename Traits::CopyVec copy_vec;
    typename Traits::ConvertHalf cast_acc;
    typename Traits::BroadcastSub broadcast_sub;
    typename Traits::BroadcastMul broadcast_mul;
    typename Traits::BroadcastDiv broadcast_div;
    typename Traits::BlockExp block_exp;
    typename Traits::VecMax vec_max;
    typename Traits::VecAdd vec_add;
    typename Traits::VecSub vec_sub;
    typename Traits::VecMul vec_mul;
    typename Traits::VecExp vec_exp;

    typename Traits::GlobalA gQ(Q);
    load_sq(gQ, sQ);
    __copy_async();
    __syncthreads();
    load_rq(sQ, rQ);

    const int iters = kN / kTN;
    for (int n = 0; n < iters; ++n) {
        typename Traits::GlobalB gK(K + size_t(n) * kTN * kK);
        typename Traits::GlobalC gV(V + (Traits::kVRowMajor ? size_t(n) * kTN * kP : size_t(n) * kTN));
        load_sk(gK, sK);
        load_sv(gV, sV);
        __copy_async();
        __syncthreads();

        load_rk(sK, rK);
        load_rv(sV, rV);
        __syncthreads();

        // scores = scale * Q·K
        attn_block.clear();
        compute::gemm(rQ, rK, attn_block);
#pragma unroll
        for (int i = 0; i < Traits::RegAcc::kRows; ++i)
#pragma unroll
            for (int j = 0; j < Traits::RegAcc::kCols; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) attn_block(i, j)(0, e) *= scale;

        // online softmax statistics (f32)
        row_max(attn_block, cur_max);
        vec_max(cur_max, run_max, new_max);
        vec_sub(run_max, new_max, rescale);
        vec_exp(rescale, rescale);  // exp(m_old - m_new); exp(-inf) = 0 on the first block

        broadcast_sub(new_max, attn_block);
        block_exp(attn_block, attn_block);
        row_sum(attn_block, cur_sum);

        vec_mul(run_sum, rescale, run_sum);
        vec_add(run_sum, cur_sum, run_sum);
        copy_vec(new_max, run_max);

        // O = O * rescale + P·V
        broadcast_mul(rescale, rO);
        cast_acc(attn_block, attn_half);
        compute::gemm(attn_half, rV, rO);
    }

    broadcast_div(run_sum, rO);

    typename Traits::RegDCast rO_out;
    typename Traits::ConvertO cast_o;
    cast_o(rO, rO_out);

    typename Traits::GlobalD gO(gO_ptr);
    typename Traits::DStorer storer_o;
    storer_o(rO_out, gO);
}

/// flash_attention with the K/V blocks double-buffered: block n + 1 goes global -> LDS directly (GlobalToSharedDirectLoader
/// into SharedRing stages) while block n is multiplied, one LDS-only barrier per block (wait_group_and_barrier) instead
/// of two __syncthreads() around a register-staged copy. Same Traits, same functors for everything else, same results.
/// (Reading Q and K as 16 x 32 / 32 x 16 MFMA operand tiles, one ds_read_b128 each, measured 8 % slower in this
/// kernel than the BaseTile pairs, so the operands stay BaseTiles.)
/// grid = (M / kTM, 1, batch), block = Traits::kThreads, dynamic LDS = Traits::kShmBytesPipelined.
template <typename InType, typename OutType, typename Traits>
__global__ void __launch_bounds__(Traits::kThreads)
    flash_attention_pipelined(const InType* dQ, const InType* dK, const InType* dV, OutType* dO, int kM, int kN,
                              float scale) {
    constexpr int kK = Traits::kK, kP = Traits::kP;
    constexpr int kTM = Traits::kTM, kTN = Traits::kTN;

    const InType* Q = dQ + blockIdx.z * (size_t(kM) * kK) + blockIdx.x * (kTM * kK);
    const InType* K = dK + blockIdx.z * (size_t(kN) * kK);
    const InType* V = dV + blockIdx.z * (size_t(kN) * kP);
    OutType* gO_ptr = dO + blockIdx.z * (size_t(kM) * kP) + blockIdx.x * (kTM * kP);

    extern __shared__ __align__(1024) unsigned char shared_buf[];
    auto* shm = reinterpret_cast<InType*>(shared_buf);
    typename Traits::RingB ringK(shm);
    typename Traits::RingC ringV(shm + Traits::RingB::kBytes / sizeof(InType));
    // Q is in LDS only until it has been read into registers: it uses the rings' bytes before the first block does
    typename Traits::SharedA sQ(shm);

    typename Traits::RegA rQ;
    typename Traits::RegB rK;
    typename Traits::RegC rV;
    typename Traits::DirectALoader load_sq;
    typename Traits::DirectBLoader load_sk;
    typename Traits::DirectCLoader load_sv;
    typename Traits::RegALoader load_rq;
    typename Traits::RegBLoader load_rk;
    typename Traits::RegCLoader load_rv;

    typename Traits::RegD rO;
    typename Traits::RegAcc attn_block;
    typename Traits::RegAccCast attn_half;
    typename Traits::RegVec run_max, run_sum, cur_max, cur_sum, new_max, rescale;
#pragma unroll
    for (int i = 0; i < Traits::RegVec::kRows; ++i) run_max(i, 0) = -INFINITY;

    typename Traits::RowMax row_max;
    typename Traits::RowSum row_sum;
    typename Traits::CopyVec copy_vec;
    typename Traits::ConvertHalf cast_acc;
    typename Traits::BroadcastSub broadcast_sub;
    typename Traits::BroadcastMul broadcast_mul;
    typename Traits::BroadcastDiv broadcast_div;
    typename Traits::BlockExp block_exp;
    typename Traits::VecMax vec_max;
    typename Traits::VecAdd vec_add;
    typename Traits::VecSub vec_sub;
    typename Traits::VecMul vec_mul;
    typename Traits::VecExp vec_exp;

    auto request_block = [&](int n, int stage) {
        typename Traits::GlobalB gK(K + size_t(n) * kTN * kK);
        typename Traits::GlobalC gV(V + (Traits::kVRowMajor ? size_t(n) * kTN * kP : size_t(n) * kTN));
        auto sK = ringK[stage];
        auto sV = ringV[stage];
        load_sk(gK, sK);
        load_sv(gV, sV);
    };

    typename Traits::GlobalA gQ(Q);
    load_sq(gQ, sQ);
    wait_group_and_barrier<0>();
    load_rq(sQ, rQ);
    wait_group_and_barrier<0>();  // everyone has read its Q: the bytes are free for the blocks
    request_block(0, 0);
    wait_group_and_barrier<0>();

    const int iters = kN / kTN;
    int stage = 0;
    for (int n = 0; n < iters; ++n) {
        if (n + 1 < iters) request_block(n + 1, stage ^ 1);
        commit_copy_group();  // keep the requests ahead of this block's work

        {
            auto sK = ringK[stage];
            auto sV = ringV[stage];
            load_rk(sK, rK);
            load_rv(sV, rV);
        }

        attn_block.clear();
        compute::gemm(rQ, rK, attn_block);
#pragma unroll
        for (int i = 0; i < Traits::RegAcc::kRows; ++i)
#pragma unroll
            for (int j = 0; j < Traits::RegAcc::kCols; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) attn_block(i, j)(0, e) *= scale;

        row_max(attn_block, cur_max);
        vec_max(cur_max, run_max, new_max);
        vec_sub(run_max, new_max, rescale);
        vec_exp(rescale, rescale);

        broadcast_sub(new_max, attn_block);
        block_exp(attn_block, attn_block);
        row_sum(attn_block, cur_sum);

        vec_mul(run_sum, rescale, run_sum);
        vec_add(run_sum, cur_sum, run_sum);
        copy_vec(new_max, run_max);

        broadcast_mul(rescale, rO);
        cast_acc(attn_block, attn_half);
        compute::gemm(attn_half, rV, rO);

        // block n + 1 has landed (this wavefront's part, then everyone's) and everyone has read block n
        wait_group_and_barrier<0>();
        stage ^= 1;
    }

    broadcast_div(run_sum, rO);
    typename Traits::RegDCast rO_out;
    typename Traits::ConvertO cast_o;
    cast_o(rO, rO_out);
    typename Traits::GlobalD gO(gO_ptr);
    typename Traits::DStorer storer_o;
    storer_o(rO_out, gO);
}

}  // namespace tiledcuda::kernels
