// The one-wavefront-per-SIMD FlashAttention-2 forward kernel (kernels/flash_attn_w64.hpp, what the long-sequence
// shapes run on) written with tile-library types and functors only, the way the reference composes its attention
// kernel from its L2 functors (src/kernels/flash_attn.cu:134-312; traits :18-131):
//   S = Q Kᵀ and O += P V as tile products on v_mfma_f32_32x32x16_f16 operand tiles (types/mfma_tile.hpp), every matrix
//   instruction placed by compute::ScheduledGemm::at<i, j, k>() (accumulators of O and the Q operand pinned in AGPRs);
//   K and V blocks of 64 keys through two interleaved 5-stage SharedRings filled by GlobalToSharedDirectPieces (one
//   direct-to-LDS load riding on a matrix instruction at a time); operand fragments requested three instructions
//   groups ahead with SharedToRegPieces (ds_read_b128, K) and SharedToRegTrPieces (ds_read_b64_tr_b16 in the order in
//   which the score accumulator holds its keys, V), waited for with wait_shared_reads<N>(); the softmax of 32 keys
//   sliced over the matrix instructions of the neighbouring 32 (compute::Exp2Raw, convert_pair_here); stage hand-over
//   with wait_group_and_barrier_keep_reads<N>(); the output through RegToSharedStorer / SharedToGlobalStorer.
// The arithmetic (which products are summed in which order, where values are rounded) is that of
// flash_attention_fwd_w64 with a row-major V: the results are bit-identical. Shapes are compile-time except the batch
// count, like every kernel written against the tile API. Requirements: head size 128, M % 256 == 0, N % 64 == 0,
// N >= 320 (Q passes through two ring stages before the fifth block needs them). Left out against the hand-indexed
// kernel: its loads that warm the L2 for the workgroup that follows on the same XCD, and its handling of a V stored
// column-major.
#pragma once

#include <type_traits>
#include <utility>

#include "cell/mod.hpp"
#include "types/mod.hpp"
#include "util/static_for.hpp"

namespace tiledcuda::kernels {

using namespace tiledcuda::cell;
using namespace tiledcuda::cell::copy;
namespace tl = tiledcuda::cell::tile_layout;

template <typename InType, const int kM_, const int kN_, const int kD_>
struct FlashW64TileTraits {
    static constexpr int kM = kM_, kN = kN_, kD = kD_;
    using WarpLayout = tl::RowMajor<4, 1>;
    static constexpr int kWaves = 4, kThreads = kWaves * kWaveSize;
    static constexpr int kTM = 64 * kWaves, kTN = 64, kHalf = 32, kStages = 5;
    static constexpr int kBlocks = kN / kTN;
    static_assert(kD == 128, "the step schedule is written for head size 128");
    static_assert(kM % kTM == 0 && kN % kTN == 0 && kBlocks >= kStages);

    using Shape = traits::MfmaTileShape<InType, traits::MfmaShape::k32x32x16>;

    // global views of one (batch, head) item
    using GlobalQ = GlobalTile<InType, tl::RowMajor<kTM, kD>>;
    using GlobalK = GlobalTile<InType, tl::ColMajor<kD, kTN>>;  // Kᵀ [d, keys], stored [keys, d]
    using GlobalV = GlobalTile<InType, tl::RowMajor<kTN, kD>>;
    using GlobalO = GlobalTile<InType, tl::RowMajor<kTM, kD>>;

    // LDS: a ring stage is a K block followed by a V block; Q passes once through stages 3 and 4
    using SharedK = SharedTile<InType, tl::ColMajor<kD, kTN>, true>;
    using SharedV = SharedTile<InType, tl::RowMajor<kTN, kD>, true, tl::LdsSwizzleTr<kD, sizeof(InType)>>;
    static constexpr int kBlockNumel = kTN * kD;
    using RingK = SharedRing<SharedK, kStages, 2 * kBlockNumel>;
    using RingV = SharedRing<SharedV, kStages, 2 * kBlockNumel>;
    using SharedQ = SharedTile<InType, tl::RowMajor<kTM, kD>, true>;
    using SharedO = SharedTile<InType, tl::RowMajor<kTM, kD>, true>;
    static constexpr int kShmBytes = kStages * 2 * kBlockNumel * int(sizeof(InType));  // 160 KiB
    static_assert(kShmBytes <= kMaxLdsBytes && 2 * 2 * kBlockNumel == kTM * kD, "Q fills exactly two stages");

    // the 32-key halves a step works on
    using KHalves = STileIterator<SharedK, TileShape<kD, kHalf>>;
    using VHalves = STileIterator<SharedV, TileShape<kHalf, kD>>;
    using SharedKHalf = decltype(std::declval<KHalves>()(0));
    using SharedVHalf = decltype(std::declval<VHalves>()(0));

    // register tiles of one wavefront (64 queries)
    using RegQ = RegTile<typename Shape::TileA, tl::RowMajor<2, kD / 16>>;   // A of S = Q Kᵀ, in AGPRs
    using RegK = RegTile<typename Shape::TileB, tl::ColMajor<kD / 16, 1>>;   // B of S: 32 keys, a fragment per k-step
    using RegS = RegTile<MfmaTileC32x32<float>, tl::RowMajor<2, 1>>;         // scores of 32 keys
    using RegP = RegTile<typename Shape::TileA, tl::RowMajor<2, 2>>;         // probabilities of 32 keys: A of O += P V
    using RegV = RegTile<typename Shape::TileB, tl::ColMajor<2, kD / 32>>;   // B of O += P V
    using RegO = RegTile<MfmaTileC32x32<float>, tl::RowMajor<2, kD / 32>>;   // in AGPRs
    using RegOut = RegTile<MfmaTileC32x32<InType>, tl::RowMajor<2, kD / 32>>;

    using QLoader = GlobalToSharedDirectLoader<SharedQ, WarpLayout>;
    using QFragments = SharedToRegLoader<RegQ, WarpLayout, WarpReuse::kRowReuseCont>;
    using PiecesK = GlobalToSharedDirectPieces<SharedK, WarpLayout, kD>;
    using PiecesV = GlobalToSharedDirectPieces<SharedV, WarpLayout, kD>;
    using KFragmentsNow = SharedToRegLoader<RegK, WarpLayout, WarpReuse::kColReuseCont>;
    using KFragments = SharedToRegPieces<RegK, SharedKHalf, WarpLayout, WarpReuse::kColReuseCont>;
    using VFragments = SharedToRegTrPieces<RegV, SharedVHalf, WarpLayout, WarpReuse::kColReuseCont, true>;
    using Scores = compute::ScheduledGemm<RegQ, RegK, RegS, compute::RegFile::kVgpr, compute::RegFile::kAgpr>;
    using Output = compute::ScheduledGemm<RegP, RegV, RegO, compute::RegFile::kAgpr, compute::RegFile::kVgpr>;
    using OutToShared = RegToSharedStorer<RegOut, WarpLayout>;
    using OutToGlobal = SharedToGlobalStreamStorer<SharedO, WarpLayout>;
    static_assert(PiecesK::kPieces == 4 && PiecesV::kPieces == 4, "a wavefront issues 8 loads per block, one per d-step");
};

/// grid = (kM / 256) * batch workgroups (1-D), block = 256, dynamic LDS = Traits::kShmBytes.
template <typename InType, typename Traits>
__global__ void __launch_bounds__(Traits::kThreads)
    flash_attention_tile_w64(const InType* dQ, const InType* dK, const InType* dV, InType* dO, int batch, float scale) {
    constexpr int kM = Traits::kM, kN = Traits::kN, kD = Traits::kD, kTN = Traits::kTN, nb = Traits::kBlocks;
    constexpr int kStages = Traits::kStages;
    using RegQ = typename Traits::RegQ;
    using RegK = typename Traits::RegK;
    using RegS = typename Traits::RegS;
    using RegP = typename Traits::RegP;
    using RegV = typename Traits::RegV;
    using RegO = typename Traits::RegO;
    using Scores = typename Traits::Scores;
    using Output = typename Traits::Output;
    extern __shared__ __align__(1024) unsigned char buf[];

    const int lane = lane_id();

    // query blocks of one (batch, head) item get workgroup ids congruent modulo 8: one XCD, K and V fetched once
    constexpr int q_blocks = kM / Traits::kTM;
    int head_i, q_block;
    if (batch % 8 == 0) {
        const int xcd = blockIdx.x & 7, rest = blockIdx.x >> 3;
        q_block = rest % q_blocks;
        head_i = (rest / q_blocks) * 8 + xcd;
    } else {
        q_block = blockIdx.x % q_blocks;
        head_i = blockIdx.x / q_blocks;
    }
    const size_t head = head_i;
    const InType* Qb = dQ + (head * kM + size_t(q_block) * Traits::kTM) * kD;
    const InType* Kh = dK + head * size_t(kN) * kD;
    const InType* Vh = dV + head * size_t(kN) * kD;
    InType* Ob = dO + (head * kM + size_t(q_block) * Traits::kTM) * kD;

    InType* shm = reinterpret_cast<InType*>(buf);
    typename Traits::RingK ringK(shm);
    typename Traits::RingV ringV(shm + Traits::kBlockNumel);
    typename Traits::SharedQ sQ(shm + 3 * 2 * Traits::kBlockNumel);  // stages 3 and 4

    typename Traits::PiecesK pieces_k;
    typename Traits::PiecesV pieces_v;
    typename Traits::KFragments k_frag;
    typename Traits::VFragments v_frag;

    // load s of this wavefront for key block `block` into ring stage `stage`: 4 pieces of K, then 4 of V
    auto block_load = [&](int stage, int block, int s) -> DirectLoad {
        return s < 4 ? pieces_k.piece(s, Kh + size_t(block) * kTN * kD, ringK[stage])
                     : pieces_v.piece(s - 4, Vh + size_t(block) * kTN * kD, ringV[stage]);
    };
    auto k_half = [&](int stage, int t) { return typename Traits::KHalves(ringK.stage_data(stage))(t); };
    auto v_half = [&](int stage, int t) { return typename Traits::VHalves(ringV.stage_data(stage))(t); };

    // ---- prologue: Q and block 0 are requested together (the cold latencies overlap); blocks 1 and 2 under the
    // first two score computations, blocks 3 and 4 (into the stages Q passed through) in the first block-iteration
    {
        typename Traits::QLoader load_q;
        typename Traits::GlobalQ gQ(Qb);
        load_q(gQ, sQ);
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) issue(block_load(0, 0, s));
    wait_group_and_barrier<0>();

    RegQ rQ;
    {
        typename Traits::QFragments read_q;
        read_q(sQ, rQ);
        // pre-multiplied by scale * log2(e): the scores come out of the matrix instruction in the log2 domain
        const float cscale = scale * 1.4426950408889634f;
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int s = 0; s < kD / 16; ++s) {
                _Float16* q = reinterpret_cast<_Float16*>(rQ(c, s).mutable_data());
#pragma unroll
                for (int e = 0; e < 8; ++e) q[e] = static_cast<_Float16>(static_cast<float>(q[e]) * cscale);
            }
        compute::pin_tiles<compute::RegFile::kAgpr>(rQ);
    }

    RegO rO;
    compute::clear_pinned(rO);

    RegS rS[2];     // score tiles of two consecutive halves, relative to the reference maximum
    RegP rP[2];     // their probabilities
    RegS neg_max;   // minus the reference maximum of this lane's query, in all 16 slots: where the score sums start
    float m_run[2], l_run[2];
    RegK rK;        // fragments in flight / in use: (k-step, 0)
    RegV rV;        // (k-step of the half, d tile)

    compute::Exp2Raw<float> exp2;
    using f16x2 = _Float16 __attribute__((ext_vector_type(2)));

    // scores of half `t` of the block in `stage` into rS[kBuf] (before the pipeline runs: plain reads), issuing this
    // wavefront's loads of block `load_block` behind the d-steps
    auto scores_only = [&](int stage, int t, auto buf_c, int load_block) {
        constexpr int kBuf = decltype(buf_c)::value;
        typename Traits::KFragmentsNow read_k;
        const auto sk = k_half(stage, t);
        RegK kf;
        read_k.load_one(sk, kf, 0, 0);
        static_for<kD / 16>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value;
            if constexpr (s + 1 < kD / 16) read_k.load_one(sk, kf, s + 1, 0);
            if constexpr (s == 0) {
                Scores::template at_from<0, 0, 0>(rQ, kf, rS[kBuf], neg_max(0, 0));
                Scores::template at_from<1, 0, 0>(rQ, kf, rS[kBuf], neg_max(1, 0));
            } else {
                Scores::template at<0, 0, s>(rQ, kf, rS[kBuf]);
                Scores::template at<1, 0, s>(rQ, kf, rS[kBuf]);
            }
            issue(block_load(load_block, load_block, s));
        });
    };

    // ---- half 0: exact maxima
    scores_only(0, 0, std::integral_constant<int, 0>{}, 1);
    asm volatile("s_nop 15\n\ts_nop 3");
    compute::pin_tiles<compute::RegFile::kVgpr>(rS[0]);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const auto& sc = rS[0](c, 0);
        float mx = sc(0);
#pragma unroll
        for (int e = 1; e < 16; ++e) mx = fmaxf(mx, sc(e));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        m_run[c] = mx;
        float lsum = 0.f;
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
            const float p0 = exp2(sc(e) - mx), p1 = exp2(sc(e + 1) - mx);
            const f16x2 pk = {static_cast<_Float16>(p0), static_cast<_Float16>(p1)};
            const unsigned int bits = __builtin_bit_cast(unsigned int, pk);
            __builtin_memcpy(rP[0](c, e / 8).mutable_data() + (e % 8), &bits, sizeof(bits));
            lsum += p0 + p1;
        }
        l_run[c] = lsum;
#pragma unroll
        for (int e = 0; e < 16; ++e) neg_max(c, 0)(e) = -mx;
    }
    scores_only(0, 1, std::integral_constant<int, 1>{}, 2);

    // ---- one pipelined step on half i: softmax of half i (rS[kCur] -> rP[kCur]), scores of half i + 1 into rS[kNxt]
    // (if kQk), O += P V with half i - 1 (rP[kNxt]). ring: stages of blocks J, J + 1, J + 2 and of the block being
    // loaded. kLoads: 0 none, 1 block `load_block`.
    // Fragments are requested kAhead d-steps before their matrix instructions, across step boundaries.
    struct Stages {
        int a, b, c, load;
    };
    constexpr int kAhead = 3;
    constexpr int kReadsV = 2, kReadsQk = 3;  // LDS read instructions per d-step

    auto step = [&](const Stages& ring, auto cur_c, auto qk_c, auto loads_c, auto next_qk_c, int load_block) {
        constexpr int kCur = decltype(cur_c)::value, kNxt = kCur ^ 1;
        constexpr bool kQk = decltype(qk_c)::value, kNextQk = decltype(next_qk_c)::value;
        constexpr int kLoads = decltype(loads_c)::value;
        // K of half i + 1, V of half i - 1, K of half i + 2, V of half i
        const auto sk = kCur == 1 ? k_half(ring.b, 0) : k_half(ring.b, 1);
        const auto sv = v_half(ring.a, kNxt);
        const auto sk_next = kCur == 1 ? k_half(ring.b, 1) : k_half(ring.c, 0);
        const auto sv_next = v_half(kCur == 1 ? ring.a : ring.b, kCur);
        float lh[2] = {0.f, 0.f}, lg[2] = {0.f, 0.f};
        float x0 = 0.f, x1 = 0.f, y0 = 0.f, y1 = 0.f;
        // probabilities of slots 2 d, 2 d + 1 of query tile c: to f16, into the A operand of the next product
        auto pack_pair = [&](auto c_c, auto d_c, float a0, float a1) {
            constexpr int c = decltype(c_c)::value, d = decltype(d_c)::value;
            compute::convert_pair_here(a0, a1, rP[kCur](c, d >> 2).mutable_data() + 2 * (d & 3));
        };
        using C0 = std::integral_constant<int, 0>;
        using C1 = std::integral_constant<int, 1>;
        static_for<8>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value;
            constexpr int sp = s + kAhead;
            if constexpr (sp < 8) {
                if constexpr (kQk) k_frag.template read<sp, 0>(sk, rK);
                v_frag.template read<sp / 4, sp & 3>(sv, rV);
                wait_shared_reads<kAhead * (kQk ? kReadsQk : kReadsV)>();
            } else {
                if constexpr (kNextQk) k_frag.template read<sp - 8, 0>(sk_next, rK);
                v_frag.template read<0, (sp - 8) & 3>(sv_next, rV);
                wait_shared_reads<(7 - s) * (kQk ? kReadsQk : kReadsV) + (sp - 7) * (kNextQk ? kReadsQk : kReadsV)>();
            }
            // slot A
            if constexpr (kQk) {
                if constexpr (s == 0) Scores::template at_from<0, 0, 0>(rQ, rK, rS[kNxt], neg_max(0, 0));
                else Scores::template at<0, 0, s>(rQ, rK, rS[kNxt]);
            }
            x0 = exp2(rS[kCur](0, 0)(2 * s));
            if constexpr (s > 0) pack_pair(C1{}, std::integral_constant<int, s - 1>{}, y0, y1);
            __builtin_amdgcn_sched_barrier(0);
            // slot B
            if constexpr (kQk) {
                if constexpr (s == 0) Scores::template at_from<1, 0, 0>(rQ, rK, rS[kNxt], neg_max(1, 0));
                else Scores::template at<1, 0, s>(rQ, rK, rS[kNxt]);
            }
            x1 = exp2(rS[kCur](0, 0)(2 * s + 1));
            if constexpr (s == 1) {
                lh[1] = y0;
                lg[1] = y1;
            } else if constexpr (s > 1) {
                lh[1] += y0;
                lg[1] += y1;
            }
            __builtin_amdgcn_sched_barrier(0);
            // slot C (with this wavefront's load s riding on the matrix instruction)
            if constexpr (kLoads == 1) {
                Output::template at<0, s & 3, s / 4>(rP[kNxt], rV, rO, block_load(ring.load, load_block, s));
            } else {
                Output::template at<0, s & 3, s / 4>(rP[kNxt], rV, rO);
            }
            y0 = exp2(rS[kCur](1, 0)(2 * s));
            pack_pair(C0{}, s_c, x0, x1);
            __builtin_amdgcn_sched_barrier(0);
            // slot D
            Output::template at<1, s & 3, s / 4>(rP[kNxt], rV, rO);
            y1 = exp2(rS[kCur](1, 0)(2 * s + 1));
            if constexpr (s == 0) {
                lh[0] = x0;
                lg[0] = x1;
            } else {
                lh[0] += x0;
                lg[0] += x1;
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        lh[1] += y0;
        lg[1] += y1;
        lh[0] += lg[0];
        lh[1] += lg[1];
        pack_pair(C1{}, std::integral_constant<int, 7>{}, y0, y1);
        // no probability of this half can have left f16 range while its sum stays below 2^14
        constexpr float kLimit = 16384.f;
        if (__any(!(fmaxf(lh[0], lh[1]) <= kLimit))) {
            // rare path: move the reference maxima, rescale, re-bias the scores already computed, recompute
            asm volatile("s_nop 15\n\ts_nop 3");
            if constexpr (kQk) compute::pin_tiles<compute::RegFile::kVgpr>(rS[kNxt]);
            compute::pin_tiles<compute::RegFile::kAgpr>(rO);
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                auto& sc = rS[kCur](c, 0);
                float mx = sc(0);
#pragma unroll
                for (int e = 1; e < 16; ++e) mx = fmaxf(mx, sc(e));
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                const float shift = mx > 8.0f ? mx : 0.f;
                const float alpha = exp2(-shift);
                m_run[c] += shift;
                l_run[c] *= alpha;
#pragma unroll
                for (int dt = 0; dt < kD / 32; ++dt)
#pragma unroll
                    for (int e = 0; e < 16; ++e) rO(c, dt)(e) *= alpha;
                if constexpr (kQk) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) rS[kNxt](c, 0)(e) -= shift;
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) neg_max(c, 0)(e) = -m_run[c];
                float lsum = 0.f;
#pragma unroll
                for (int e = 0; e < 16; e += 2) {
                    const float p0 = exp2(sc(e) - shift), p1 = exp2(sc(e + 1) - shift);
                    const f16x2 pk = {static_cast<_Float16>(p0), static_cast<_Float16>(p1)};
                    const unsigned int bits = __builtin_bit_cast(unsigned int, pk);
                    __builtin_memcpy(rP[kCur](c, e / 8).mutable_data() + (e % 8), &bits, sizeof(bits));
                    lsum += p0 + p1;
                }
                lh[c] = lsum;
            }
            compute::pin_tiles<compute::RegFile::kAgpr>(rO);
        }
        l_run[0] += lh[0];
        l_run[1] += lh[1];
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- block-iterations: J covers halves 2 J + 1 and 2 J + 2
    using Yes = std::true_type;
    using No = std::false_type;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    int J = 0;
    Stages ring{0, 1, 2, 4};
    auto advance = [&]() {
        ring.a = ring.b;
        ring.b = ring.c;
        ring.c = Traits::RingK::next(ring.c);
        ring.load = Traits::RingK::next(ring.load);
        ++J;
    };
    {
        // J = 0: blocks 3 and 4 go to the stages Q passed through (everyone has read its Q by now)
        wait_group_and_barrier_keep_reads<0>();
        // first fragments of step 1: K of half 2 (block 1), V of half 0 - behind the barrier: block 1 is complete only
        // when every wavefront's pieces of it have landed
        static_for<kAhead>([&](auto a_c) {
            constexpr int a = decltype(a_c)::value;
            k_frag.template read<a, 0>(k_half(1, 0), rK);
            v_frag.template read<0, a & 3>(v_half(0, 0), rV);
        });
        Stages first = ring;
        first.load = 3;
        step(first, I1{}, Yes{}, I1{}, Yes{}, 3);
        step(ring, I0{}, Yes{}, I1{}, Yes{}, 4);
        advance();
    }
    // (the block count is a constant here: left alone, the compiler unrolls these loops and the longer live ranges cost
    // registers the kernel does not have)
#pragma unroll 1
    for (; J + 4 < nb; advance()) {
        wait_group_and_barrier_keep_reads<8>();
        step(ring, I1{}, Yes{}, I1{}, Yes{}, J + 4);
        step(ring, I0{}, Yes{}, I0{}, Yes{}, 0);
    }
#pragma unroll 1
    for (; J + 2 < nb; advance()) {
        wait_group_and_barrier_keep_reads<0>();
        step(ring, I1{}, Yes{}, I0{}, Yes{}, 0);
        step(ring, I0{}, Yes{}, I0{}, Yes{}, 0);
    }
    if (J + 1 < nb) {
        step(ring, I1{}, Yes{}, I0{}, Yes{}, 0);
        step(ring, I0{}, Yes{}, I0{}, No{}, 0);
        advance();
    }
    step(ring, I1{}, No{}, I0{}, No{}, 0);
    {
        // O += P V with the last half (its first fragments were requested by the step before)
        const auto sv = v_half(ring.a, 1);
        static_for<8>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value;
            constexpr int sp = s + kAhead;
            if constexpr (sp < 8) {
                v_frag.template read<sp / 4, sp & 3>(sv, rV);
                wait_shared_reads<kAhead * kReadsV>();
            } else {
                wait_shared_reads<(7 - s) * kReadsV>();
            }
            Output::template at<0, s & 3, s / 4>(rP[1], rV, rO);
            Output::template at<1, s & 3, s / 4>(rP[1], rV, rO);
        });
    }

    // ---- epilogue: O = O / l, to f16, through LDS for row-contiguous 16-byte stores
    compute::settle_accumulators(rO);
    typename Traits::RegOut out;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const float l_tot = l_run[c] + __shfl_xor(l_run[c], 32, 64);
        const float inv_l = 1.0f / l_tot;
#pragma unroll
        for (int dt = 0; dt < kD / 32; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) out(c, dt)(e) = __float2half(rO(c, dt)(e) * inv_l);
    }
    wait_group<0>();
    __syncthreads();  // every wavefront is done with the K/V stages: the space is reused for O
    typename Traits::SharedO sO(shm);
    typename Traits::OutToShared to_shared;
    typename Traits::OutToGlobal to_global;
    typename Traits::GlobalO gO(Ob);
    to_shared(out, sO);
    __syncthreads();
    to_global(sO, gO);
}

}  // namespace tiledcuda::kernels
