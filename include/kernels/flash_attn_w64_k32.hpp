// FlashAttention-2 forward, one wavefront per SIMD, on v_mfma_f32_16x16x32_f16 - the f16 matrix instruction that
// contracts 32 indices per issue. Same design as kernels/flash_attn_tile_w64.hpp (which uses v_mfma_f32_32x32x16_f16)
// and written with the same tile-library functors, the way the reference composes its attention kernel from its L2
// functors (src/kernels/flash_attn.cu:134-312; traits :18-131):
//   a workgroup of 4 wavefronts owns 256 queries, a wavefront 64 (four 16-row tiles); K and V blocks of 64 keys pass
//   through two interleaved 5-stage SharedRings filled by GlobalToSharedDirectPieces (one direct-to-LDS load riding on a
//   matrix instruction at a time); S = Q Kᵀ and O += P V are tile products whose every instruction is placed by
//   compute::ScheduledGemm::at<i, j, k>() (O and the Q operand pinned in AGPRs, the scores in VGPRs); operand fragments
//   live in rings of four tiles and are requested three groups of instructions ahead through SharedToRegPieces
//   (ds_read_b128, K) and SharedToRegTrPieces (ds_read_b64_tr_b16, V, in the order in which two 16 x 16 score
//   accumulators hold their keys, so that the converted scores ARE the A operand of the second product) with addresses
//   bound to the ring stage (bind / read_bound_to / shift: no addition in front of a read), awaited with
//   wait_shared_reads<N>(); the softmax of 32 keys is sliced over the 64 matrix instructions of the neighbouring 32 (at
//   head size 128) - a v_exp_f32 behind every second one, the sums and conversions behind the others (compute::Exp2Raw,
//   convert_pair_here); stages are handed over with wait_group_and_barrier_keep_reads<N>(); the last three steps fetch
//   what the next workgroup on the XCD will ask for first; the output leaves through RegToSharedStorer /
//   SharedToGlobalStorer.
// Why a second instruction shape: under the chip's power limit the core clock follows the work, and a stream of
// 16x16x32 instructions sustains a clock about an eighth higher than the same arithmetic in 32x32x16 instructions
// (half the accumulator traffic per multiply-add). The price is issue time: what a wavefront alone on its SIMD places
// between two 16-cycle matrix instructions is not free (see the comment at `step`), so the schedule counts slots.
// Numerics: as flash_attention_fwd_w64 (Q pre-multiplied by scale * log2 e in f16, scores relative to a reference
// maximum that moves only when a partial sum could leave f16 range, f32 sums and output); the sums inside a matrix
// instruction cover 32 instead of 16 indices and the final division is a reciprocal and a product, so results differ
// from that kernel in the last bits.
// Requirements: head size 128 (V row-major [N, D] or column-major, the reference op's convention; see the traits) or 64
// (row-major V; a step then has 32 matrix instructions for the same softmax work and every one carries an exponential),
// M % 64 == 0 (wavefronts of a head's last block of 256 whose queries lie beyond M idle), N % 64 == 0, N >= 320 (Q passes
// through two ring stages before the fifth block needs them). M, N and the batch count are run-time values.
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

/// kVColMajor_: V is stored column-major [N, D], i.e. as the array Vᵀ [D, N] (the convention of the reference's op,
/// src/kernels/flash_attn.cu:314-327). Then a V block lies in LDS as two halves of 32 keys, column-major like K (lines
/// of 64 bytes along the keys), its fragments are plain 16-byte reads in the standard contraction order, and the keys
/// of a half are dealt to the two K operand tiles four at a time (copy::SharedToRegPieces<..., kDealtLines>), so that
/// the two score accumulators of a lane hold 8 consecutive keys.
template <typename InType, const int kD_, const bool kVColMajor_ = false>
struct FlashW64K32Traits {
    static constexpr int kD = kD_;
    static constexpr bool kVColMajor = kVColMajor_;
    using WarpLayout = tl::RowMajor<4, 1>;
    static constexpr int kWaves = 4, kThreads = kWaves * kWaveSize;
    static constexpr int kTM = 64 * kWaves, kTN = 64, kHalf = 32, kStages = 5;
    static_assert(kD == 128 || (kD == 64 && !kVColMajor), "the step schedule is written for head sizes 128 and 64 (row-major V)");

    using Shape = traits::MfmaTileShape<InType, traits::MfmaShape::k16x16x32>;
    static constexpr int kQTiles = 64 / 16;     // 16-row query tiles of a wavefront
    static constexpr int kKeyTiles = kHalf / 16;  // 16-key tiles of a half
    static constexpr int kDSteps = kD / 32;     // contraction steps of S = Q Kᵀ
    static constexpr int kDTiles = kD / 16;     // 16-column tiles of O
    static constexpr int kGroups = kDSteps * kKeyTiles;  // groups of a step: a K fragment and a V fragment each (8 or 4)
    static constexpr int kKtPerReg = 4 / kDSteps;         // key tiles that the ring of 4 K fragments spans (1 or 2)

    // global views of one query block / key block
    using GlobalQ = GlobalTile<InType, tl::RowMajor<kTM, kD>>;
    using GlobalO = GlobalTile<InType, tl::RowMajor<kTM, kD>>;

    // LDS: a ring stage is a K block followed by a V block; Q passes once through stages 3 and 4
    // Kᵀ [d, keys], stored [keys, d]
    using SharedK = std::conditional_t<kVColMajor, SharedTile<InType, tl::ColMajor<kD, kTN>, true, tl::LdsSwizzleDealt<kD, sizeof(InType)>>,
                                       SharedTile<InType, tl::ColMajor<kD, kTN>, true>>;
    // a V block [keys, d] row-major, or one of its two halves [32 keys, d] column-major (the other one 8 KiB further on)
    using SharedV = std::conditional_t<kVColMajor, SharedTile<InType, tl::ColMajor<kHalf, kD>, true>,
                                       SharedTile<InType, tl::RowMajor<kTN, kD>, true, tl::LdsSwizzleTr<kD, sizeof(InType), 8>>>;
    static constexpr int kBlockNumel = kTN * kD;
    using RingK = SharedRing<SharedK, kStages, 2 * kBlockNumel>;
    using RingV = SharedRing<SharedV, kStages, 2 * kBlockNumel>;
    using SharedQ = SharedTile<InType, tl::RowMajor<kTM, kD>, true>;
    using SharedO = SharedTile<InType, tl::RowMajor<kTM, kD>, true>;
    static constexpr int kShmBytes = kStages * 2 * kBlockNumel * int(sizeof(InType));  // 160 KiB (80 at head size 64)
    static_assert(kShmBytes <= kMaxLdsBytes && 2 * 2 * kBlockNumel == kTM * kD, "Q fills exactly two stages");

    // the 32-key halves a step works on
    using KHalves = STileIterator<SharedK, TileShape<kD, kHalf>>;
    using SharedKHalf = decltype(std::declval<KHalves>()(0));
    struct RowMajorVHalf {  // half t of a row-major block: a view of 32 of its 64 lines
        using Halves = STileIterator<SharedV, TileShape<kHalf, kD>>;
        using type = decltype(std::declval<Halves>()(0));
        DEVICE static type at(InType* block, int t) { return Halves(block)(t); }
    };
    struct ColMajorVHalf {  // half t of a column-major block: a tile of its own
        using type = SharedV;
        DEVICE static type at(InType* block, int t) { return SharedV(block + t * kHalf * kD); }
    };
    using VHalf = std::conditional_t<kVColMajor, ColMajorVHalf, RowMajorVHalf>;
    using SharedVHalf = typename VHalf::type;

    // register tiles of one wavefront (64 queries)
    using RegQ = RegTile<typename Shape::TileA, tl::RowMajor<kQTiles, kDSteps>>;     // A of S = Q Kᵀ, in AGPRs
    using RegK = RegTile<typename Shape::TileB, tl::ColMajor<kDSteps, kKtPerReg>>;   // B of S: a ring of 4 fragments
    using RegKAll = RegTile<typename Shape::TileB, tl::ColMajor<kDSteps, kKeyTiles>>; // what the fragment loader addresses
    using RegS = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kQTiles, kKtPerReg>>; // scores of 16 (or 32) keys
    using RegM = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kQTiles, 1>>;         // where the score sums start
    using RegP = RegTile<typename Shape::TileA, tl::RowMajor<kQTiles, 1>>;           // probabilities: A of O += P V
    using RegV = RegTile<typename Shape::TileB, tl::ColMajor<1, 4>>;                 // B of O += P V: a ring of 4 fragments
    using RegVAll = RegTile<typename Shape::TileB, tl::ColMajor<1, kDTiles>>;
    using RegO = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kQTiles, 4>>;         // 4 of the head size's 16-column tiles; in AGPRs
    using RegOut = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kQTiles, kDTiles>>;

    using QLoader = GlobalToSharedDirectLoader<SharedQ, WarpLayout>;
    using PiecesQ = GlobalToSharedDirectPieces<SharedQ, WarpLayout, kD>;  // the same copy a load at a time (the next item's Q)
    using QFragments = SharedToRegLoader<RegQ, WarpLayout, WarpReuse::kRowReuseCont>;
    using PiecesK = GlobalToSharedDirectPieces<SharedK, WarpLayout, kD>;
    // (a column-major V: the lines of a tile are N elements apart in memory, a run-time size)
    using PiecesV = GlobalToSharedDirectPieces<SharedV, WarpLayout, kVColMajor ? 0 : kD>;
    using KFragments = SharedToRegPieces<RegKAll, SharedKHalf, WarpLayout, WarpReuse::kColReuseCont, kVColMajor>;
    using VFragments = std::conditional_t<kVColMajor, SharedToRegPieces<RegVAll, SharedVHalf, WarpLayout, WarpReuse::kColReuseCont>,
                                          SharedToRegTrPieces<RegVAll, SharedVHalf, WarpLayout, WarpReuse::kColReuseCont, true>>;
    static constexpr int kReadsV = kVColMajor ? 1 : 2;  // LDS read instructions per V fragment
    using Scores = compute::ScheduledGemm<RegQ, RegK, RegS, compute::RegFile::kVgpr, compute::RegFile::kAgpr>;
    using Output = compute::ScheduledGemm<RegP, RegV, RegO, compute::RegFile::kAgpr, compute::RegFile::kVgpr>;
    using OutToShared = RegToSharedStorer<RegOut, WarpLayout>;
    using OutToGlobal = SharedToGlobalStreamStorer<SharedO, WarpLayout>;
    static constexpr int kLoadsK = PiecesK::kPieces;  // of a wavefront, per block: then as many of V
    static_assert(2 * kLoadsK == kGroups && PiecesV::kPieces == (kVColMajor ? kLoadsK / 2 : kLoadsK),
                  "a wavefront issues one load per group of the step that loads a block");
    static_assert(PiecesQ::kPieces == 2 * kGroups, "a wavefront fetches its 64 query rows with two steps' worth of loads");
    static_assert(kDTiles == kGroups && (kGroups == 8 || kGroups == 4), "a step has 8 or 4 groups: a K fragment and a V fragment each");
};

/// grid = min(ceil(M / 256) * batch, number of CUs) workgroups (1-D), block = 256, dynamic LDS = Traits::kShmBytes. A workgroup
/// takes the items (blocks of 256 queries of one batch item) blockIdx.x, blockIdx.x + gridDim.x, ... one after the
/// other: gridDim.x must be a multiple of 8 (or hold every item), so that a workgroup's items stay on its XCD's mapping.
template <typename InType, typename Traits>
__global__ void __launch_bounds__(Traits::kThreads)
    flash_attention_w64_k32(const InType* dQ, const InType* dK, const InType* dV, InType* dO, int batch, int kM, int kN,
                            float scale) {
    constexpr int kD = Traits::kD, kTN = Traits::kTN;
    constexpr int kQT = Traits::kQTiles, kDT = Traits::kDTiles, kStages = Traits::kStages;
    constexpr int kDS = Traits::kDSteps, kG = Traits::kGroups, kKtPerReg = Traits::kKtPerReg;
    constexpr int kSRegs = 2 / kKtPerReg, kORegs = kDT / 4;  // register tiles that hold a half's scores / the output
    using RegQ = typename Traits::RegQ;
    using RegK = typename Traits::RegK;
    using RegS = typename Traits::RegS;
    using RegM = typename Traits::RegM;
    using RegP = typename Traits::RegP;
    using RegV = typename Traits::RegV;
    using RegO = typename Traits::RegO;
    using Scores = typename Traits::Scores;
    using Output = typename Traits::Output;
    extern __shared__ __align__(1024) unsigned char buf[];
    const int nb = kN / kTN;

    // query blocks of one (batch, head) item get item numbers congruent modulo 8: one XCD, K and V fetched once
    const int q_blocks = (kM + Traits::kTM - 1) / Traits::kTM;
    const int items = q_blocks * batch;
    auto locate = [&](int w, size_t& head, int& q_block) {
        if (batch % 8 == 0) {
            const int xcd = w & 7, rest = w >> 3;
            q_block = rest % q_blocks;
            head = size_t(rest / q_blocks) * 8 + xcd;
        } else {
            q_block = w % q_blocks;
            head = size_t(w / q_blocks);
        }
    };
    const int wave_u = __builtin_amdgcn_readfirstlane(wave_id());
    // The ring stage of key block 0 of the current item, and whether the item's Q and first block are in LDS already
    // (the workgroup's previous item fetched them under its last steps).
    int s0 = 0;
    bool fetched = false;
#pragma unroll 1
    for (int w = blockIdx.x; w < items; w += gridDim.x) {
    size_t head;
    int q_block;
    locate(w, head, q_block);
    // kM need only be a multiple of 64: a wavefront of a head's last block whose 64 queries lie beyond kM takes part in
    // the loads of K and V and in the barriers, reads the block's first 64 rows of Q in place of its own and writes
    // nothing
    auto rows_of = [&](int qb) { return wave_u * 64 < kM - qb * Traits::kTM ? wave_u * 64 : 0; };
    const bool active = wave_u * 64 < kM - q_block * Traits::kTM;
    // (the loaders address a wavefront's rows from the tile's origin: the origin is moved instead)
    const InType* Qb = dQ + (long(head) * kM + long(q_block) * Traits::kTM + rows_of(q_block) - wave_u * 64) * kD;
    const InType* Kh = dK + head * size_t(kN) * kD;
    const InType* Vh = dV + head * size_t(kN) * kD;
    InType* Ob = dO + (head * kM + size_t(q_block) * Traits::kTM) * kD;
    // the workgroup's next item (without one: this item again, so that the schedule has one form)
    const InType *Qnext, *Knext, *Vnext;
    {
        size_t nhead;
        int nqb;
        locate(w + int(gridDim.x) < items ? w + int(gridDim.x) : w, nhead, nqb);
        Qnext = dQ + (long(nhead) * kM + long(nqb) * Traits::kTM + rows_of(nqb) - wave_u * 64) * kD;
        Knext = dK + nhead * size_t(kN) * kD;
        Vnext = dV + nhead * size_t(kN) * kD;
    }
    auto st = [&](int i) {  // ring stage of key block i < 5 of this item
        const int t = s0 + i;
        return t >= kStages ? t - kStages : t;
    };

    InType* shm = reinterpret_cast<InType*>(buf);
    typename Traits::RingK ringK(shm);
    typename Traits::RingV ringV(shm + Traits::kBlockNumel);
    // Q and O pass through LDS a wavefront at a time: each wavefront writes and reads only its own 64 rows (16 KiB, a
    // quarter of the tile). A 256-row tile laid over two ring stages that need not be neighbours in memory (the ring
    // wraps): wavefronts 0, 1 use stage `sa`, wavefronts 2, 3 stage `sb`; the pointer is where row 0 would be for this
    // wavefront's rows to land there.
    constexpr int kStageNumel = 2 * Traits::kBlockNumel, kWaveRowsNumel = 64 * kD;
    auto rows_over_two_stages = [&](int sa, int sb) -> InType* {
        return shm + (wave_u < 2 ? sa : sb) * kStageNumel + (wave_u & 1) * kWaveRowsNumel - wave_u * kWaveRowsNumel;
    };
    typename Traits::SharedQ sQ(rows_over_two_stages(st(3), st(4)));

    typename Traits::PiecesK pieces_k;
    typename Traits::PiecesV pieces_v = [&] {
        if constexpr (Traits::kVColMajor) return typename Traits::PiecesV(kN);
        else return typename Traits::PiecesV();
    }();
    typename Traits::KFragments k_frag;
    typename Traits::VFragments v_frag;

    // load s of this wavefront for key block `block` of the operands `Kb`, `Vb` into ring stage `stage`: the pieces of K,
    // then as many of V
    auto v_half = [&](int stage, int t) { return Traits::VHalf::at(ringV.stage_data(stage), t); };
    auto load_of = [&](const InType* Kb, const InType* Vb, int stage, int block, int s) -> DirectLoad {
        constexpr int kLK = Traits::kLoadsK;
        if (s < kLK) return pieces_k.piece(s, Kb + size_t(block) * kTN * kD, ringK[stage]);
        if constexpr (Traits::kVColMajor) {  // element (key, d) of V at Vb[d * kN + key]: two loads per half
            const int t = (s - kLK) >> 1;
            return pieces_v.piece((s - kLK) & 1, Vb + size_t(block) * kTN + t * Traits::kHalf, v_half(stage, t));
        } else {
            return pieces_v.piece(s - kLK, Vb + size_t(block) * kTN * kD, ringV[stage]);
        }
    };
    auto block_load = [&](int stage, int block, int s) -> DirectLoad { return load_of(Kh, Vh, stage, block, s); };
    auto k_half = [&](int stage, int t) { return typename Traits::KHalves(ringK.stage_data(stage))(t); };

    // ---- prologue: Q and block 0 are requested together (the cold latencies overlap); blocks 1 and 2 under the
    // first two score computations, blocks 3 and 4 (into the stages Q passed through) in the first block-iteration
    if (!fetched) {
        typename Traits::QLoader load_q;
        typename Traits::GlobalQ gQ(Qb);
        load_q(gQ, sQ);
#pragma unroll
        for (int s = 0; s < kG; ++s) issue(block_load(st(0), 0, s));
        wait_group_and_barrier<0>();
    }

    RegQ rQ;
    {
        typename Traits::QFragments read_q;
        read_q(sQ, rQ);
        // pre-multiplied by scale * log2(e): the scores come out of the matrix instruction in the log2 domain
        const float cscale = scale * 1.4426950408889634f;
#pragma unroll
        for (int c = 0; c < kQT; ++c)
#pragma unroll
            for (int s = 0; s < Traits::kDSteps; ++s) {
                _Float16* q = reinterpret_cast<_Float16*>(rQ(c, s).mutable_data());
#pragma unroll
                for (int e = 0; e < 8; ++e) q[e] = static_cast<_Float16>(static_cast<float>(q[e]) * cscale);
            }
        compute::pin_tiles<compute::RegFile::kAgpr>(rQ);
    }

    RegO rO[kORegs];  // d tiles 0..3 (and 4..7)
#pragma unroll
    for (int h = 0; h < kORegs; ++h) compute::clear_pinned(rO[h]);

    RegS rS[2][kSRegs];  // [half buffer][key tile / kKtPerReg]: score tiles of two consecutive halves, relative to the reference maximum
    RegP rP[2];     // their probabilities
    RegM neg_max;   // minus the reference maximum of this lane's query of each tile, in all 4 slots
    float m_run[kQT], l_run[kQT];
    RegK rK;        // ring of the fragments in flight / in use: fragment g lives in tile g % 4 (column-major order)
    RegV rV;

    compute::Exp2Raw<float> exp2;
    using f16x2 = _Float16 __attribute__((ext_vector_type(2)));
    // maximum over the 4 lane groups that share a query row
    auto row_max = [](float v) {
        v = fmaxf(v, __shfl_xor(v, 16, 64));
        return fmaxf(v, __shfl_xor(v, 32, 64));
    };

    // scores of half `t` of the block in `stage` into rS[kBuf] (before the pipeline runs: plain reads), issuing this
    // wavefront's loads of block `load_block` behind the groups
    auto scores_only = [&](int stage, int t, auto buf_c, int load_block) {
        constexpr int kBuf = decltype(buf_c)::value;
        const auto sk = k_half(stage, t);
        typename Traits::RegKAll kf;
        k_frag.template read<0, 0>(sk, kf);
        static_for<kG>([&](auto g_c) {
            constexpr int g = decltype(g_c)::value, ds = g % kDS, kt = g / kDS;
            if constexpr (g + 1 < kG) {
                k_frag.template read<(g + 1) % kDS, (g + 1) / kDS>(sk, kf);
                wait_shared_reads<1>();
            } else {
                wait_shared_reads<0>();
            }
            RegK one;
            one(ds, kt % kKtPerReg) = kf(ds, kt);
            static_for<kQT>([&](auto c_c) {
                constexpr int c = decltype(c_c)::value;
                if constexpr (ds == 0) Scores::template at_from<c, kt % kKtPerReg, 0>(rQ, one, rS[kBuf][kt / kKtPerReg], neg_max(c, 0));
                else Scores::template at<c, kt % kKtPerReg, ds>(rQ, one, rS[kBuf][kt / kKtPerReg]);
            });
            issue(block_load(st(load_block), load_block, g));
        });
    };

    // probabilities of one score tile's 4 keys: to f16, into 4 slots of the A operand, and their sum
    auto tile_softmax_now = [&](const BaseTileRowMajor<float>& sc, float shift, _Float16* dst) {
        const float p0 = exp2(sc(0, 0) - shift), p1 = exp2(sc(0, 1) - shift);
        const float p2 = exp2(sc(0, 2) - shift), p3 = exp2(sc(0, 3) - shift);
        const f16x2 lo = {static_cast<_Float16>(p0), static_cast<_Float16>(p1)};
        const f16x2 hi = {static_cast<_Float16>(p2), static_cast<_Float16>(p3)};
        __builtin_memcpy(dst, &lo, sizeof(lo));
        __builtin_memcpy(dst + 2, &hi, sizeof(hi));
        return (p0 + p1) + (p2 + p3);
    };

    // score tile (query tile c, key tile kt) of a half
    auto s_tile = [&](RegS(&rs)[kSRegs], int c, int kt) -> BaseTileRowMajor<float>& { return rs[kt / kKtPerReg](c, kt % kKtPerReg); };

    // ---- half 0: exact maxima
#pragma unroll
    for (int c = 0; c < kQT; ++c)
#pragma unroll
        for (int e = 0; e < 4; ++e) neg_max(c, 0)(0, e) = 0.f;
    compute::pin_tiles<compute::RegFile::kVgpr>(neg_max);
    scores_only(st(0), 0, std::integral_constant<int, 0>{}, 1);
    asm volatile("s_nop 15\n\ts_nop 3");
#pragma unroll
    for (int h = 0; h < kSRegs; ++h) compute::pin_tiles<compute::RegFile::kVgpr>(rS[0][h]);
#pragma unroll
    for (int c = 0; c < kQT; ++c) {
        float mx = s_tile(rS[0], c, 0)(0, 0);
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) mx = fmaxf(mx, s_tile(rS[0], c, kt)(0, e));
        mx = row_max(mx);
        m_run[c] = mx;
        _Float16* p = reinterpret_cast<_Float16*>(rP[0](c, 0).mutable_data());
        l_run[c] = tile_softmax_now(s_tile(rS[0], c, 0), mx, p) + tile_softmax_now(s_tile(rS[0], c, 1), mx, p + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) neg_max(c, 0)(0, e) = -mx;
    }
    compute::pin_tiles<compute::RegFile::kVgpr>(neg_max);
    scores_only(st(0), 1, std::integral_constant<int, 1>{}, 2);

    struct Stages {
        int a, b, c, load;
    };
    constexpr int kAhead = 3;
    constexpr int kReadsV = Traits::kReadsV, kReadsQk = kReadsV + 1;  // LDS read instructions per group
    constexpr int kHalfBytes = Traits::kHalf * kD * int(sizeof(InType));  // between the halves of a K or V block
    constexpr int kStageBytes = 2 * Traits::kBlockNumel * int(sizeof(InType));

    // The last three steps of an item have no ring loads left to issue and fetch what the workgroup's next item starts
    // with instead - its 256 query rows (kLoads == 2, 4: 8 of a wavefront's 16 loads each) and its first K / V block
    // (kLoads == 3) - into the three ring stages this item has left for good. The next item then starts computing at once.
    typename Traits::PiecesQ pieces_q;
    int next_s0 = 0;                                    // the stage of the next item's block 0
    typename Traits::SharedQ sQnext(shm);               // (set when the fetch begins)

    // A fragment's address moves on to the next ring stage between its read of half 1 of a block and its read of half 0
    // of the next: fragments 0..2 (requested at the end of a step for the next one) behind the first step of a
    // block-iteration, fragments 3..7 behind the second.
    auto shift_fragments = [&](const Stages& ring, auto first_c, auto last_c) {
        const int dK = (ring.c - ring.b) * kStageBytes, dV = (ring.b - ring.a) * kStageBytes;
        static_for<decltype(last_c)::value - decltype(first_c)::value>([&](auto i_c) {
            constexpr int f = decltype(first_c)::value + decltype(i_c)::value;
            k_frag.template shift<f % kDS, f / kDS>(dK);
            if constexpr (Traits::kVColMajor) v_frag.template shift<0, f>(dV);
            else v_frag.template shift<f>(dV);
        });
    };

    // ---- one pipelined step on half i: softmax of half i (rS[kCur] -> rP[kCur]), scores of half i + 1 into rS[kNxt]
    // (if kQk), O += P V with half i - 1 (rP[kNxt]). ring: stages of blocks J, J + 1, J + 2 and of the block being
    // loaded. kLoads: 0 none, 1 block `load_block`, 2 / 4 / 3 the next item's Q (first, second half) / first block.
    // A step is kG = 8 (head size 128) or 4 (64) groups of 8 matrix instructions: group g multiplies K fragment g (d-step
    // g % kDS of key tile g / kDS) with the 4 query tiles, then V fragment g (d tile g) with the 4 probability tiles, and
    // takes 32 / kG score values of half i through the softmax: score tile (query tile g / 2, key tile g % 2) with 8
    // groups, both key tiles of query tile g with 4. The fragments of group g + kAhead are requested inside group g (K
    // behind the fourth, V behind the eighth matrix instruction), through addresses bound to the ring stage (no
    // addition per read). What goes between two matrix instructions is measured, not guessed: every matrix instruction is followed
    // by its dose in this order (the barriers keep the compiler from pairing the matrix instructions up), and the doses
    // come in pairs of issue slots - a v_exp_f32 counts as two, everything else as one; a pair costs 4 cycles on top of
    // the matrix instruction's 16, a single slot costs as much, three or four cost 8. With 4 groups every matrix
    // instruction has an exponential to carry, and its dose is four slots (the exponential, the addition of the one before
    // to the sum, and a conversion or a fragment read).
    auto step = [&](const Stages& ring, auto cur_c, auto qk_c, auto loads_c, auto next_qk_c, int load_block) {
        constexpr int kCur = decltype(cur_c)::value, kNxt = kCur ^ 1;
        constexpr bool kQk = decltype(qk_c)::value, kNextQk = decltype(next_qk_c)::value;
        constexpr int kLoads = decltype(loads_c)::value;
        float lh[kQT] = {0.f, 0.f, 0.f, 0.f};
        float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        using I3 = std::integral_constant<int, 3>;
        static_for<kG>([&](auto g_c) {
            constexpr int g = decltype(g_c)::value;
            constexpr int gp = g + kAhead, f = gp % kG;
            // the fragments of group g + kAhead: halves 0 of the blocks in the first step of a block-iteration
            // (kCur == 1) until the step's end, halves 1 afterwards
            constexpr int kImm = ((gp < kG) == (kCur == 1)) ? 0 : kHalfBytes;
            constexpr bool kReadK = gp < kG ? kQk : kNextQk;
            // reads in flight that are younger than the fragments of this group and the next, at the top of the group
            // (the requests of this group are not yet issued): one wait per two groups
            constexpr int kPerGroup = kQk ? kReadsQk : kReadsV, kPerGroupNext = kNextQk ? kReadsQk : kReadsV;
            constexpr int kYounger = gp < kG ? (kAhead - 1) * kPerGroup : (kG - 1 - g) * kPerGroup + (gp - kG) * kPerGroupNext;
            if constexpr (g % 2 == 0) wait_shared_reads<kYounger - kPerGroup>();
            constexpr int ds = g % kDS, kt = g / kDS;  // the K fragment of this group
            auto score = [&](auto c_c) {
                constexpr int c = decltype(c_c)::value;
                if constexpr (kQk) {
                    if constexpr (ds == 0) Scores::template at_from<c, kt % kKtPerReg, 0>(rQ, rK, rS[kNxt][kt / kKtPerReg], neg_max(c, 0));
                    else Scores::template at<c, kt % kKtPerReg, ds>(rQ, rK, rS[kNxt][kt / kKtPerReg]);
                }
            };
            auto read_k = [&]() {
                if constexpr (kReadK) k_frag.template read_bound_to<f % kDS, f / kDS, kImm>(rK(f % kDS, (f / kDS) % kKtPerReg));
            };
            // the first matrix instruction of O += P V carries this group's load
            auto output0 = [&]() {
                if constexpr (kLoads == 1) {
                    Output::template at<0, g % 4, 0>(rP[kNxt], rV, rO[g / 4], block_load(ring.load, load_block, g));
                } else if constexpr (kLoads == 2 || kLoads == 4) {
                    Output::template at<0, g % 4, 0>(rP[kNxt], rV, rO[g / 4], pieces_q.piece(kLoads == 2 ? g : kG + g, Qnext, sQnext));
                } else if constexpr (kLoads == 3) {
                    Output::template at<0, g % 4, 0>(rP[kNxt], rV, rO[g / 4], load_of(Knext, Vnext, next_s0, 0, g));
                } else {
                    Output::template at<0, g % 4, 0>(rP[kNxt], rV, rO[g / 4]);
                }
            };
            if constexpr (kG == 8) {
                constexpr int sc = g / 2, st = g % 2;  // the score tile of half i this group takes through the softmax
                const auto& sv4 = rS[kCur][st](sc, 0);
                _Float16* pdst = reinterpret_cast<_Float16*>(rP[kCur](sc, 0).mutable_data()) + 4 * st;
                _Float16* pprev = reinterpret_cast<_Float16*>(rP[kCur]((g + 7) % 8 / 2, 0).mutable_data()) + 4 * ((g + 7) % 2);
                score(I0{});
                __builtin_amdgcn_sched_barrier(0);
                x[0] = exp2(sv4(0, 0));
                __builtin_amdgcn_sched_barrier(0);
                score(I1{});
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (g > 0) {  // the second pair of the group before
                    compute::convert_pair_here(x[2], x[3], reinterpret_cast<__half*>(pprev) + 2);
                    lh[(g - 1) / 2] += x[3];
                }
                __builtin_amdgcn_sched_barrier(0);
                score(I2{});
                __builtin_amdgcn_sched_barrier(0);
                x[1] = exp2(sv4(0, 1));
                __builtin_amdgcn_sched_barrier(0);
                score(I3{});
                __builtin_amdgcn_sched_barrier(0);
                lh[sc] += x[0];
                read_k();
                __builtin_amdgcn_sched_barrier(0);
                output0();
                __builtin_amdgcn_sched_barrier(0);
                x[2] = exp2(sv4(0, 2));
                __builtin_amdgcn_sched_barrier(0);
                Output::template at<1, g % 4, 0>(rP[kNxt], rV, rO[g / 4]);
                __builtin_amdgcn_sched_barrier(0);
                compute::convert_pair_here(x[0], x[1], reinterpret_cast<__half*>(pdst));
                lh[sc] += x[1];
                __builtin_amdgcn_sched_barrier(0);
                Output::template at<2, g % 4, 0>(rP[kNxt], rV, rO[g / 4]);
                __builtin_amdgcn_sched_barrier(0);
                x[3] = exp2(sv4(0, 3));
                __builtin_amdgcn_sched_barrier(0);
                Output::template at<3, g % 4, 0>(rP[kNxt], rV, rO[g / 4]);
                __builtin_amdgcn_sched_barrier(0);
                lh[sc] += x[2];
                v_frag.template read_bound_to<0, f, kImm>(rV(0, f % 4));
                __builtin_amdgcn_sched_barrier(0);
            } else {
                // query tile g of half i: x[0..3] its key tile 0, x[4..7] its key tile 1; the last pair and the last two
                // additions of a group wait for the first two gaps of the next one
                const auto& sv0 = rS[kCur][0](g, 0);
                const auto& sv1 = rS[kCur][0](g, 1);
                __half* pdst = reinterpret_cast<__half*>(rP[kCur](g, 0).mutable_data());
                __half* pprev = reinterpret_cast<__half*>(rP[kCur]((g + 3) % 4, 0).mutable_data());
                score(I0{});
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (g > 0) {
                    compute::convert_pair_here(x[6], x[7], pprev + 6);
                    lh[g - 1] += x[7];
                }
                x[0] = exp2(sv0(0, 0));
                __builtin_amdgcn_sched_barrier(0);
                score(I1{});
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (g > 0) lh[g - 1] += x[6];
                x[1] = exp2(sv0(0, 1));
                lh[g] += x[0];
                __builtin_amdgcn_sched_barrier(0);
                score(I2{});
                __builtin_amdgcn_sched_barrier(0);
                x[2] = exp2(sv0(0, 2));
                lh[g] += x[1];
                compute::convert_pair_here(x[0], x[1], pdst);
                __builtin_amdgcn_sched_barrier(0);
                score(I3{});
                __builtin_amdgcn_sched_barrier(0);
                x[3] = exp2(sv0(0, 3));
                lh[g] += x[2];
                read_k();
                __builtin_amdgcn_sched_barrier(0);
                output0();
                __builtin_amdgcn_sched_barrier(0);
                x[4] = exp2(sv1(0, 0));
                lh[g] += x[3];
                compute::convert_pair_here(x[2], x[3], pdst + 2);
                __builtin_amdgcn_sched_barrier(0);
                Output::template at<1, g % 4, 0>(rP[kNxt], rV, rO[g / 4]);
                __builtin_amdgcn_sched_barrier(0);
                x[5] = exp2(sv1(0, 1));
                lh[g] += x[4];
                __builtin_amdgcn_sched_barrier(0);
                Output::template at<2, g % 4, 0>(rP[kNxt], rV, rO[g / 4]);
                __builtin_amdgcn_sched_barrier(0);
                x[6] = exp2(sv1(0, 2));
                lh[g] += x[5];
                compute::convert_pair_here(x[4], x[5], pdst + 4);
                __builtin_amdgcn_sched_barrier(0);
                Output::template at<3, g % 4, 0>(rP[kNxt], rV, rO[g / 4]);
                __builtin_amdgcn_sched_barrier(0);
                x[7] = exp2(sv1(0, 3));
                v_frag.template read_bound_to<0, f, kImm>(rV(0, f % 4));
                __builtin_amdgcn_sched_barrier(0);
            }
        });
        if constexpr (kG == 8) {
            lh[kQT - 1] += x[3];
            compute::convert_pair_here(x[2], x[3], reinterpret_cast<__half*>(rP[kCur](kQT - 1, 0).mutable_data()) + 6);
        } else {
            lh[kQT - 1] += x[6] + x[7];
            compute::convert_pair_here(x[6], x[7], reinterpret_cast<__half*>(rP[kCur](kQT - 1, 0).mutable_data()) + 6);
        }
        // No probability of this half can have left f16 range while its sum stays below 2^14. The comparison first, then
        // work that does not depend on it, then the branch: the scalar unit sees the result of a vector comparison only
        // some 20 cycles after it was issued.
        constexpr float kLimit = 16384.f;
        unsigned long long over = __ballot(!(fmaxf(fmaxf(lh[0], lh[1]), fmaxf(lh[2], lh[3])) <= kLimit));
        asm volatile("" : "+s"(over));
        float l_before[kQT];  // (the half's sums may be infinite when the branch is taken: kept apart)
#pragma unroll
        for (int c = 0; c < kQT; ++c) {
            l_before[c] = l_run[c];
            l_run[c] += lh[c];
        }
        if constexpr (kCur == 1) shift_fragments(ring, std::integral_constant<int, 0>{}, std::integral_constant<int, 3>{});
        else shift_fragments(ring, std::integral_constant<int, 3>{}, std::integral_constant<int, kG>{});
        __builtin_amdgcn_sched_barrier(0);
        if (__builtin_expect(over != 0, 0)) {
            // rare path: move the reference maxima, rescale, re-bias the scores already computed, recompute
            asm volatile("s_nop 15\n\ts_nop 3");
            if constexpr (kQk) {
#pragma unroll
                for (int h = 0; h < kSRegs; ++h) compute::pin_tiles<compute::RegFile::kVgpr>(rS[kNxt][h]);
            }
#pragma unroll
            for (int h = 0; h < kORegs; ++h) compute::pin_tiles<compute::RegFile::kAgpr>(rO[h]);
#pragma unroll
            for (int c = 0; c < kQT; ++c) {
                float mx = s_tile(rS[kCur], c, 0)(0, 0);
#pragma unroll
                for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
                    for (int e = 0; e < 4; ++e) mx = fmaxf(mx, s_tile(rS[kCur], c, kt2)(0, e));
                mx = row_max(mx);
                const float shift = mx > 8.0f ? mx : 0.f;
                const float alpha = exp2(-shift);
                m_run[c] += shift;
#pragma unroll
                for (int h = 0; h < kORegs; ++h)
#pragma unroll
                    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                        for (int e = 0; e < 4; ++e) rO[h](c, dt)(0, e) *= alpha;
                if constexpr (kQk) {
#pragma unroll
                    for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
                        for (int e = 0; e < 4; ++e) s_tile(rS[kNxt], c, kt2)(0, e) -= shift;
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) neg_max(c, 0)(0, e) = -m_run[c];
                _Float16* p = reinterpret_cast<_Float16*>(rP[kCur](c, 0).mutable_data());
                const float lsum = tile_softmax_now(s_tile(rS[kCur], c, 0), shift, p) + tile_softmax_now(s_tile(rS[kCur], c, 1), shift, p + 4);
                l_run[c] = l_before[c] * alpha + lsum;
            }
            compute::pin_tiles<compute::RegFile::kVgpr>(neg_max);
#pragma unroll
            for (int h = 0; h < kORegs; ++h) compute::pin_tiles<compute::RegFile::kAgpr>(rO[h]);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- block-iterations: J covers halves 2 J + 1 and 2 J + 2
    using Yes = std::true_type;
    using No = std::false_type;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    int J = 0;
    Stages ring{st(0), st(1), st(2), st(4)};
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
        k_frag.bind(k_half(st(1), 0));
        v_frag.bind(v_half(st(0), 0));
        static_for<kAhead>([&](auto a_c) {
            constexpr int a = decltype(a_c)::value;
            k_frag.template read_bound_to<a % kDS, a / kDS>(rK(a % kDS, (a / kDS) % kKtPerReg));
            v_frag.template read_bound_to<0, a>(rV(0, a % 4));
        });
        Stages first = ring;
        first.load = st(3);
        step(first, I1{}, Yes{}, I1{}, Yes{}, 3);
        step(ring, I0{}, Yes{}, I1{}, Yes{}, 4);
        advance();
    }
    // (left alone, the compiler unrolls these loops and the longer live ranges cost registers the kernel does not have)
#pragma unroll 1
    for (; J + 4 < nb; advance()) {
        wait_group_and_barrier_keep_reads<kG>();
        step(ring, I1{}, Yes{}, I1{}, Yes{}, J + 4);
        step(ring, I0{}, Yes{}, I0{}, Yes{}, 0);
    }
#pragma unroll 1
    for (; J + 2 < nb; advance()) {
        wait_group_and_barrier_keep_reads<0>();
        step(ring, I1{}, Yes{}, I0{}, Yes{}, 0);
        step(ring, I0{}, Yes{}, I0{}, Yes{}, 0);
    }
    // The last three steps carry the next item's first loads. The stages they go to: this item's last two blocks sit
    // in ring.a and ring.b; the other three are free once every wavefront has left block nb - 3 (the barrier). Q goes to
    // the first two of them, the first K / V block to the third, which makes that one stage 0 of the next item's ring
    // (its Q then lies in its stages 3 and 4, where this item's did).
    const int last_a = ring.a, last_b = ring.b;
    {
        const int f0 = ring.c, f1 = Traits::RingK::next(f0);
        next_s0 = Traits::RingK::next(f1);
        wait_group_and_barrier_keep_reads<0>();
        sQnext = typename Traits::SharedQ(rows_over_two_stages(f0, f1));
    }
    using FetchQ0 = std::integral_constant<int, 2>;
    using FetchQ1 = std::integral_constant<int, 4>;
    using FetchKV = std::integral_constant<int, 3>;
    if (J + 1 < nb) {
        step(ring, I1{}, Yes{}, FetchQ0{}, Yes{}, 0);
        step(ring, I0{}, Yes{}, FetchQ1{}, No{}, 0);
        advance();
    }
    step(ring, I1{}, No{}, FetchKV{}, No{}, 0);
    {
        // O += P V with the last half (its first fragments were requested by the step before)
        static_for<kG>([&](auto g_c) {
            constexpr int g = decltype(g_c)::value;
            constexpr int gp = g + kAhead;
            if constexpr (gp < kG) {
                v_frag.template read_bound_to<0, gp, kHalfBytes>(rV(0, gp % 4));
                wait_shared_reads<kAhead * kReadsV>();
            } else {
                wait_shared_reads<(kG - 1 - g) * kReadsV>();
            }
            static_for<kQT>([&](auto c_c) { Output::template at<decltype(c_c)::value, g % 4, 0>(rP[1], rV, rO[g / 4]); });
        });
    }

    // ---- epilogue: O = O / l, to f16, through LDS for row-contiguous 16-byte stores (8-byte stores straight from the
    // accumulator layout were measured: three times slower)
#pragma unroll
    for (int h = 0; h < kORegs; ++h) compute::settle_accumulators(rO[h]);
    typename Traits::RegOut out;
#pragma unroll
    for (int c = 0; c < kQT; ++c) {
        float l_tot = l_run[c] + __shfl_xor(l_run[c], 16, 64);
        l_tot += __shfl_xor(l_tot, 32, 64);
        const float inv_l = __builtin_amdgcn_rcpf(l_tot);
#pragma unroll
        for (int dt = 0; dt < kDT; ++dt) {
            const auto& o = rO[dt / 4](c, dt % 4);
            __half* dst = reinterpret_cast<__half*>(out(c, dt).mutable_data());
            compute::convert_pair_here(o(0, 0) * inv_l, o(0, 1) * inv_l, dst);
            compute::convert_pair_here(o(0, 2) * inv_l, o(0, 3) * inv_l, dst + 2);
        }
    }
    // this wavefront's pieces of the next item's Q and first block have landed, then everyone's; and every wavefront is
    // done with the stages of the last two blocks, which take the output now (a wavefront's own rows only: nothing to
    // wait for between writing and reading them)
    wait_group<0>();
    __syncthreads();
    typename Traits::SharedO sO(rows_over_two_stages(last_a, last_b));
    typename Traits::OutToShared to_shared;
    typename Traits::OutToGlobal to_global;
    typename Traits::GlobalO gO(Ob);
    to_shared(out, sO);
    if (active) to_global(sO, gO);
    // the next item loads its blocks 1 and 2 into these two stages: not before everyone has read its rows back
    __builtin_amdgcn_s_barrier();
    s0 = next_s0;
    fetched = true;
    }  // items of this workgroup
}

}  // namespace tiledcuda::kernels
