// fp16 GEMM for gfx950 with one wavefront per SIMD: C[M, N] = A[M, K] · B, A row-major, B column-major (stored
// [N, K]), f32 accumulate, C row-major in f16 or f32. Same contract as kernels/gemm_pipelined.hpp (the multi-stage
// counterpart of the reference's examples/cpp/01_gemm/02_gemm_all_mem/gemm.hpp:103-155) and bit-identical results;
// what changes is how the 256 x 256 x 64 workgroup tile is mapped to the CU:
//   * 4 wavefronts (2 x 2), one per SIMD, each owning a 128 x 128 block of C: 64 v_mfma_f32_16x16x32_f16 per
//     32-wide k-substep for 16 ds_read_b128 (8 A + 8 B fragments) - a third less LDS traffic per MFMA than the
//     64 x 128 blocks of the 8-wavefront kernel, and on this part the matrix pipe's clock is set by power, so every
//     byte not moved is clock for the MFMAs;
//   * the 256 f32 accumulators per lane live in the AGPR half of the wavefront's 512 registers for the whole kernel.
//     The MFMAs are issued through inline assembly with AGPR-constrained operands: that pins the accumulators there
//     (the compiler, left alone, moves them through VGPRs) and fixes the instruction order, which is the point of a
//     one-wavefront-per-SIMD kernel - nothing else can fill the matrix pipe while this wavefront does something else;
//   * a tile of K is two phases of 64 MFMAs. Phase 1 (substep 0) also issues the 16 fragment reads of substep 1, one
//     per two MFMAs; then one LDS-only barrier per tile: tile kt+1 has landed, everyone has left tile kt's stage;
//     phase 2 (substep 1) also issues the reads of tile kt+1 / substep 0 and this wavefront's 16 direct-to-LDS loads
//     of tile kt+2 into the stage just vacated, one per four MFMAs (the CU's address unit takes one vector-memory
//     instruction per ~14 cycles, and a wavefront that has to wait for it issues no MFMAs). A load has one to two
//     phases to land;
//   * the loads address memory as scalar base + 32-bit lane offset (the k offset advances in scalar registers: no
//     vector ALU work per load), and each load is one asm statement with the MFMA that precedes it, which is the
//     wait state the load needs after the write of m0;
//   * no branches inside the loop over k (the last two tiles are peeled): a taken branch stalls the one instruction
//     stream that feeds the matrix pipe;
//   * LDS layout, XOR swizzle and XCD-aware tile order are those of gemm_pipelined.hpp; the f16 epilogue stages 16
//     rows at a time through 8 KiB of LDS per wavefront beyond the operand stages (no workgroup barrier, staging
//     overlapped with the 16-byte row-contiguous stores).
//   * a second tile width, 256 x 128 (GemmW128TraitsN<4>: a wavefront owns 128 x 64, 32 MFMAs per phase with 12 fragment
//     reads and 12 loads per tile), for products with too few 256 x 256 tiles to fill the chip. Its stages are 48 KiB, so
//     a third one fits, and it runs with three: the barrier in the middle of tile kt waits for tile kt + 1 with the loads
//     of tile kt + 2 still on their way, and phase 2 requests tile kt + 3 - three phases to land instead of one to two
//     (2048 x 2560 x 4096: 52.8 us with two stages, 45.9 us with three). Per multiply-add it moves half as much again
//     through LDS and the load path as the 256 x 256 tile, which is why it loses where that one fills the chip
//     (4096^3: 115 against 99 us).
// Because the compiler does not know these asm statements are MFMAs it inserts none of the wait states MFMA results
// need before other instructions read them; the only such reads are in the epilogue, and every accumulator passes
// through a waiting statement first (see below). M % 256 == 0, N a multiple of the tile width - or, with edge tiles
// (kEdges: rows clamped on the way in, stores guarded), any multiples of 16 - and K % 64 == 0 (checked by the launcher).
#pragma once

#include <type_traits>

#include "config.hpp"
#include "hip_utils.hpp"
#include "kernels/gemm_pipelined.hpp"  // detail::lds_barrier, detail::xcd_tile_coords

namespace tiledcuda::kernels {

/// kNT_: 16-column tiles of a wavefront's block of C: 8 (workgroup tile 256 x 256, two stages) or 4 (256 x 128, three
/// stages: for products with too few 256 x 256 tiles to fill the chip and too many 128 x 128 tiles for one round of the
/// K-splitting kernel).
template <const int kNT_ = 8>
struct GemmW128TraitsN {
    static constexpr int kNT = kNT_;
    static constexpr int kBM = 256, kBN = 2 * 16 * kNT, kBK = 64;
    static constexpr int kWaves = 4, kThreads = kWaves * kWaveSize;
    static constexpr int kWaveM = 128, kWaveN = 16 * kNT;
    static constexpr int kMT = kWaveM / 16;                     // 8 x kNT MFMA tiles of 16 x 16 per wavefront
    static constexpr int kRowBytes = kBK * 2;                   // 128
    static constexpr int kABytes = kBM * kRowBytes, kBBytes = kBN * kRowBytes;
    static constexpr int kStageBytes = kABytes + kBBytes;  // 64 KiB (48)
    static constexpr int kLoads = kBM / 8 / kWaves;        // 1 KiB load instructions of A per wavefront per stage
    static constexpr int kLoadsB = kBN / 8 / kWaves;       // ... of B: 8 (4)
    static constexpr int kFrags = 8 + kNT;                 // operand fragments of a substep
    static constexpr int kStages = kNT == 8 ? 2 : 3;       // the narrower tile's stages are 48 KiB: a third one fits
    static constexpr int kLdsBytesMain = kStages * kStageBytes;  // 128 KiB (144) of operand stages
    static constexpr int kEpilogueBytesPerWave = 2 * 16 * kWaveN * 2;  // f16 epilogue: two buffers of 16 rows
    static constexpr int kLdsBytes = kLdsBytesMain + kWaves * kEpilogueBytesPerWave;  // 160 KiB
    static_assert(kLoads == 8 && kMT == 8 && (kNT == 8 || kNT == 4), "the phase schedule below is written for these counts");
    static_assert(kLdsBytes <= kMaxLdsBytes);
};
using GemmW128Traits = GemmW128TraitsN<8>;

namespace detail {

/// acc += a · b on the matrix pipe, accumulator in AGPRs.
DEVICE void mfma_16x16x32_agpr(f32x4& acc, const f16x8& a, const f16x8& b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

/// The same MFMA, then a direct-to-LDS load of 16 bytes per lane from sbase + voff to lds_addr + 16 * lane. m0 is
/// written before the MFMA, which thereby is the wait state required between the write of m0 and the load.
DEVICE void mfma_16x16x32_agpr_then_load(f32x4& acc, const f16x8& a, const f16x8& b, unsigned int voff,
                                         const void* sbase, unsigned int lds_addr) {
    asm volatile(
        "s_mov_b32 m0, %5\n\t"
        "v_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n\t"
        "global_load_lds_dwordx4 %3, %4"
        : "+a"(acc)
        : "v"(a), "v"(b), "v"(voff), "s"(sbase), "s"(lds_addr)
        : "m0", "memory");
}

}  // namespace detail

/// C[i] = sum over z of partial[z][i] (f32 partial sums of a split-K product), 4 elements per lane. n % 4 == 0.
template <typename OutType>
__global__ void __launch_bounds__(256) splitk_reduce(const float* __restrict__ partial, OutType* __restrict__ C,
                                                     size_t n, int splits) {
    const size_t i = (size_t(blockIdx.x) * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    // (read once, written once: streamed both ways)
    f32x4 acc = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(partial + i));
    for (int z = 1; z < splits; ++z) {
        const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(partial + size_t(z) * n + i));
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += v[e];
    }
    if constexpr (sizeof(OutType) == 4) {
        __builtin_nontemporal_store(acc, reinterpret_cast<f32x4*>(C + i));
    } else {
        f16x4 h;
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = static_cast<_Float16>(acc[e]);
        __builtin_nontemporal_store(h, reinterpret_cast<f16x4*>(C + i));
    }
}

/// grid = ((M / 256) * (N / kBN), splits), block = 256, dynamic LDS = T::kLdsBytes.
/// lda / ldb: elements between consecutive rows of A / of the stored [N, K] array (K for dense operands; larger when
/// the operand is a column block of a wider matrix); ldc: elements between consecutive rows of C (N for a dense C;
/// larger when C is the leading block of a wider matrix). With splits > 1 workgroup row z multiplies the
/// K-range [z K, (z + 1) K) and writes plane z of C ([splits, M, N]; partial sums for splitk_reduce).
/// zero_words / zero_count: device words that the first workgroup sets to zero on the side (null / 0: none) - the
/// synchronisation words of a kernel that follows this one on the stream, cleared without a launch of their own.
/// kEdges: M and N need not be multiples of the tile (multiples of 16 suffice): the grid covers ceil(M / 256) x
/// ceil(N / kBN) tiles, rows beyond the edge are loaded from the last valid row (their products are computed and
/// dropped) and the stores are guarded. With 256 x 256 tiles K may be any multiple of 16 as well: the loop runs over
/// ceil(K / 64) tiles and the pieces of the last one beyond K are zeros in LDS. Nothing changes inside the loop over K
/// but for its last three tiles.
template <typename OutType, typename T = GemmW128Traits, bool kEdges = false>
__global__ void __launch_bounds__(T::kThreads)
    gemm_w128(const __half* __restrict__ A, const __half* __restrict__ Bt, OutType* __restrict__ C, int M, int N, int K,
              int lda, int ldb, int ldc, unsigned int* __restrict__ zero_words, int zero_count) {
    constexpr int kNT = T::kNT, kNumLoads = 8 + T::kLoadsB, kFrags = T::kFrags;
    extern __shared__ __align__(1024) unsigned char lds[];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int wave_m = wave >> 1, wave_n = wave & 1;
    if (zero_count > 0 && blockIdx.x == 0 && blockIdx.y == 0) {
        for (int i = threadIdx.x; i < zero_count; i += T::kThreads) zero_words[i] = 0u;
    }
    int tile_m, tile_n;
    detail::xcd_tile_coords(blockIdx.x, kEdges ? (M + T::kBM - 1) / T::kBM : M / T::kBM,
                            kEdges ? (N + T::kBN - 1) / T::kBN : N / T::kBN, tile_m, tile_n);
    const int m0 = tile_m * T::kBM, n0 = tile_n * T::kBN;

    // ---- global -> LDS: load instruction q of this wavefront (q < 8: A, else B) fills 8 rows of 128 bytes; lane i
    // writes physical 16-byte chunk i % 8 of row i / 8, which must hold logical chunk (i % 8) ^ ((row / 2) % 8)
    const int lrow = lane >> 3, lchk = lane & 7;
    unsigned int voff[kNumLoads];
#pragma unroll
    for (int q = 0; q < kNumLoads; ++q) {
        const int row = (q < 8 ? wave * T::kLoads + q : wave * T::kLoadsB + (q - 8)) * 8 + lrow;
        const int last = q < 8 ? M - 1 - m0 : N - 1 - n0;  // the tile's last row that exists
        voff[q] = static_cast<unsigned int>(kEdges && row > last ? last : row) * static_cast<unsigned int>(q < 8 ? lda : ldb) * 2u +
                  (lchk ^ ((row >> 1) & 7)) * 16;
    }
    // blockIdx.y = z selects the z-th K-range of length K of wider operands (split-K: lda, ldb >= gridDim.y * K) and
    // the z-th [M, N] plane of C; an ordinary launch has gridDim.y == 1
    const size_t z = blockIdx.y;
    const __half* a_base = A + size_t(m0) * lda + z * K;
    const __half* b_base = Bt + size_t(n0) * ldb + z * K;
    C += z * size_t(M) * ldc;
    const unsigned int lds_base = static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds));
    // the LDS destination of load q per stage: scalar registers of their own, so that the load's m0 is one s_mov away
    // (an addition per load, recomputed in the loop, was a third instruction behind the MFMA the load rides on)
    unsigned int dst_of[T::kStages][kNumLoads];
#pragma unroll
    for (int st = 0; st < T::kStages; ++st)
#pragma unroll
        for (int q = 0; q < kNumLoads; ++q) {
            dst_of[st][q] = __builtin_amdgcn_readfirstlane(lds_base + st * T::kStageBytes + (q < 8 ? 0 : T::kABytes) +
                                                           (q < 8 ? wave * T::kLoads + q : wave * T::kLoadsB + (q - 8)) * 1024);
            asm volatile("" : "+s"(dst_of[st][q]));
        }
    auto load_dst = [&](int stage, int q) __attribute__((always_inline)) -> unsigned int {
        if constexpr (T::kStages == 2) return stage ? dst_of[1][q] : dst_of[0][q];
        else return stage == 0 ? dst_of[0][q] : stage == 1 ? dst_of[1][q] : dst_of[2][q];
    };
    // Rows a multiple of 32 KiB apart put the same k-tile of every row of every panel into the same few memory
    // channels, and all workgroups walk K in step. Each XCD then starts at a different eighth of K and wraps around
    // (its workgroups stay in step with each other, which is what makes its L2 work): 7-14 % at K = 16384, nothing at
    // smaller K. The sum over K is then taken in rotated order: the same value on every run, but not bit for bit the
    // in-order sum of the other kernels (f32 rounding).
    // K a multiple of 16 (two-stage form with edge tiles only): the last tile of K is partial. Its 16-byte pieces that lie
    // beyond K are fetched from the row's first piece of that tile instead (tail_back[p]: how far back that is for loads of
    // parity p, 0 for pieces inside K) and overwritten with zeros in LDS once they have landed.
    constexpr bool kTail = kEdges && T::kStages == 2;
    const int ktiles = kTail ? (K + T::kBK - 1) / T::kBK : K / T::kBK;
    const int tail_pieces = kTail ? (K % T::kBK) / 8 : 0;  // 0: K is whole tiles
    unsigned int tail_back[2] = {0u, 0u};
    if constexpr (kTail) {
        if (tail_pieces != 0) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int piece = lchk ^ ((4 * p + (lrow >> 1)) & 7);  // logical piece this lane fetches in loads of parity p
                tail_back[p] = piece >= tail_pieces ? piece * 16u : 0u;
            }
        }
    }
    auto tail_voff = [&](int q) { return voff[q] - tail_back[q & 1]; };
    const int k_start = __builtin_amdgcn_readfirstlane(
        ((lda | ldb) & 16383) == 0 && ktiles >= 64 ? int(blockIdx.x & 7) * (ktiles / 8) : 0);
    auto load_src = [&](int kt, int q) -> const __half* {
        const int ks = kt + k_start >= ktiles ? kt + k_start - ktiles : kt + k_start;
        return (q < 8 ? a_base : b_base) + ks * T::kBK;
    };

    // ---- LDS -> registers: fragment r of a substep (r < 8: A rows 16 r.., else B rows 16 (r - 8)..); lane l holds
    // row l % 16, k = 8 (l / 16) .. +7 of the 32-wide substep = logical chunk 4 kk + l / 16 of its row
    const int frow = lane & 15, fquad = lane >> 4;
    // The lane's address of fragment 0 of A and of B, per stage and substep, in registers of their own (the XOR term
    // depends on lane % 16 only, so fragment r lies r * 2 KiB further on: an immediate) - the later stages begin 48 or
    // 64 KiB further on, which no immediate reaches.
    unsigned int frag_a[T::kStages][2], frag_b[T::kStages][2];  // [stage][kk]
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
        const unsigned int lane_off = frow * T::kRowBytes + (((4 * kk + fquad) ^ ((frow >> 1) & 7)) * 16);
#pragma unroll
        for (int st = 0; st < T::kStages; ++st) {
            frag_a[st][kk] = lds_base + st * T::kStageBytes + wave_m * T::kWaveM * T::kRowBytes + lane_off;
            frag_b[st][kk] = lds_base + st * T::kStageBytes + T::kABytes + wave_n * T::kWaveN * T::kRowBytes + lane_off;
            asm volatile("" : "+v"(frag_a[st][kk]), "+v"(frag_b[st][kk]));
        }
    }
    // (stage: a constant, or with two stages a run-time 0 / 1 in the tiles behind the unrolled loop)
    auto read_frag = [&](auto stage, int kk, int r) __attribute__((always_inline)) -> f16x8 {
        using lds_f16x8_ptr = __attribute__((address_space(3))) const f16x8*;
        unsigned int base;
        if constexpr (std::is_same_v<decltype(stage), int>) {  // (two stages only: the three-stage form never gets here)
            base = r < 8 ? (stage ? frag_a[1][kk] : frag_a[0][kk]) : (stage ? frag_b[1][kk] : frag_b[0][kk]);
        } else {
            base = r < 8 ? frag_a[decltype(stage)::value][kk] : frag_b[decltype(stage)::value][kk];
        }
        return *reinterpret_cast<lds_f16x8_ptr>(base + (r < 8 ? r : r - 8) * 16 * T::kRowBytes);
    };

    f16x8 fx[kFrags], fy[kFrags];  // fragments of substep 0 / substep 1: [0..7] A, [8..] B

    auto clamped = [&](int kt) { return kt < ktiles ? kt : ktiles - 1; };
    if constexpr (T::kStages == 3) {
        // three stages: tiles 0, 1, 2 (behind the end of K: the last tile again, so that every phase is the same code)
#pragma unroll
        for (int st = 0; st < 3; ++st)
#pragma unroll
            for (int q = 0; q < kNumLoads; ++q) detail::load_lds_16B_sbase(voff[q], load_src(clamped(st), q), load_dst(st, q));
    } else {
#pragma unroll
        for (int q = 0; q < kNumLoads; ++q)
            detail::load_lds_16B_sbase(kTail && ktiles == 1 ? tail_voff(q) : voff[q], load_src(0, q), load_dst(0, q));
        if (ktiles > 1) {
#pragma unroll
            for (int q = 0; q < kNumLoads; ++q)
                detail::load_lds_16B_sbase(kTail && ktiles == 2 ? tail_voff(q) : voff[q], load_src(1, q), load_dst(1, q));
        }
    }
    // the 256 accumulators are cleared while the first tiles are on their way (the empty asm statements keep the
    // compiler from sinking the clears below the barrier, where nothing would hide them)
    // the accumulators are pinned to the AGPR half row group by row group
    auto pin_row = [](f32x4 (&row)[kNT]) {
        if constexpr (kNT == 8)
            asm volatile("" : "+a"(row[0]), "+a"(row[1]), "+a"(row[2]), "+a"(row[3]), "+a"(row[4]), "+a"(row[5]), "+a"(row[6]), "+a"(row[7]));
        else
            asm volatile("" : "+a"(row[0]), "+a"(row[1]), "+a"(row[2]), "+a"(row[3]));
    };
    f32x4 acc[8][kNT];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int j = 0; j < kNT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        pin_row(acc[i]);
    }
    // this wavefront's part of tile 0 has landed; then everyone's
    // the pieces of a partial last tile that lie beyond K: zeros, once the loads into `stage` have landed
    auto zero_tail = [&](int stage) {
        using lds_u32x4_ptr = __attribute__((address_space(3))) u32x4*;
#pragma unroll
        for (int q = 0; q < kNumLoads; ++q)
            if (tail_back[q & 1] != 0u) *reinterpret_cast<lds_u32x4_ptr>(load_dst(stage, q) + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    };
    if constexpr (T::kStages == 3) {
        detail::lds_barrier<2 * kNumLoads>();
    } else if (ktiles > 1) {
        detail::lds_barrier<kNumLoads>();
    } else {
        if (kTail && tail_pieces != 0) {
            detail::wait_vmcnt<0>();
            zero_tail(0);
        }
        detail::lds_barrier<0>();
    }
#pragma unroll
    for (int r = 0; r < kFrags; ++r) fx[r] = read_frag(std::integral_constant<int, 0>{}, 0, r);

    // Order of the fragment reads of a phase: row group 0 of the next phase needs A fragment 0 and all B fragments.
    auto order = [](int r) { return r == 0 ? 0 : r <= kNT ? 7 + r : r - kNT; };
    // MFMA n of row group i works on tile (i, j): odd row groups walk their tiles backwards, so that one operand of
    // every MFMA, also the first of a row group, is the operand of the MFMA before it
    auto snake = [](int i, int n) { return (i & 1) ? kNT - 1 - n : n; };

    // One tile of K. kMore: there is a tile kt+1 (read its substep 0 during phase 2); kMore2: there is a tile kt+2
    // (load it during phase 2). Row group i = MFMA tiles (i, 0..7): the MFMA order is fixed by the asm statements, the
    // fragment reads (plain loads) are written where they should issue and the compiler keeps them there.
    // kTailLoads: the tile loaded here is the last one and may be partial. In the loop over K, unrolled by two, the stage
    // is a constant, so that every LDS address there is a register fixed for the kernel plus an immediate (with the stage a
    // run-time value a tile pays 8 vector additions in front of fragment reads and 26 scalar ones).
    auto tile = [&](int kt, auto more_c, auto more2_c, auto tail_loads_c, auto stage_v) __attribute__((always_inline)) {
        constexpr bool kMore = decltype(more_c)::value, kMore2 = decltype(more2_c)::value;
        constexpr bool kTailLoads = decltype(tail_loads_c)::value;
        const int stage = stage_v;  // an integral_constant in the unrolled loop, kt % 2 in the tiles behind it
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int n = 0; n < kNT; ++n) {
                const int j = snake(i, n);
                const int r = (kNT / 2) * i + (n >> 1);
                if ((n & 1) == 0 && r < kFrags) fy[order(r)] = read_frag(stage, 1, order(r));
                detail::mfma_16x16x32_agpr(acc[i][j], fx[8 + j], fx[i]);
            }
        }
        // this wavefront's part of tile kt+1 has landed and its reads of `stage` are done; then everyone's
        if constexpr (kTail && kMore && !kMore2) {  // tile kt+1 is the last one
            if (tail_pieces != 0) {
                detail::wait_vmcnt<0>();
                zero_tail(stage ^ 1);
            }
        }
        detail::lds_barrier<0>();
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int n = 0; n < kNT; ++n) {
                const int j = snake(i, n);
                const int r = (kNT / 2) * i + (n >> 1);
                if (kMore && (n & 1) == 0 && r < kFrags) fx[order(r)] = read_frag(stage ^ 1, 0, order(r));
                // one load per four MFMAs (256 x 256) or per two and a half (256 x 128: 12 loads over 32 MFMAs)
                const int m = kNT * i + n;  // (256 x 128: 12 loads over 32 MFMAs, behind MFMAs 0, 3, 6 of every 8)
                const int q = kNT == 8 ? 2 * i + (n >> 2) : (3 * m) / 8;
                const bool load_here = kNT == 8 ? (n & 3) == 1 : (3 * m) % 8 < 3;
                if (kMore2 && load_here && q < kNumLoads) {
                    detail::mfma_16x16x32_agpr_then_load(acc[i][j], fy[8 + j], fy[i], kTailLoads ? tail_voff(q) : voff[q],
                                                         load_src(kt + 2, q), load_dst(stage, q));
                } else {
                    detail::mfma_16x16x32_agpr(acc[i][j], fy[8 + j], fy[i]);
                }
            }
        }
    };
    // The same with three stages: tile kt + 1 landed a whole tile ago, the barrier in the middle waits for it with the
    // loads of tile kt + 2 still on their way, and phase 2 requests tile kt + 3 into the stage just vacated: a load has
    // three phases to land instead of one to two. Straight-line code: behind the end of K the loads fetch the last tile
    // again and the fragment reads fetch data nobody uses.
    auto tile3 = [&](int kt, auto stage_c, auto next_c) __attribute__((always_inline)) {
        constexpr int stage = decltype(stage_c)::value;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int n = 0; n < kNT; ++n) {
                const int j = snake(i, n);
                const int r = (kNT / 2) * i + (n >> 1);
                if ((n & 1) == 0 && r < kFrags) fy[order(r)] = read_frag(stage_c, 1, order(r));
                detail::mfma_16x16x32_agpr(acc[i][j], fx[8 + j], fx[i]);
            }
        }
        detail::lds_barrier<kNumLoads>();
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int n = 0; n < kNT; ++n) {
                const int j = snake(i, n);
                const int r = (kNT / 2) * i + (n >> 1);
                if ((n & 1) == 0 && r < kFrags) fx[order(r)] = read_frag(next_c, 0, order(r));
                const int m = kNT * i + n;  // 12 loads over 32 MFMAs: behind MFMAs 0, 3, 6 of every 8
                const int q = (3 * m) / 8;
                if ((3 * m) % 8 < 3 && q < kNumLoads) {
                    detail::mfma_16x16x32_agpr_then_load(acc[i][j], fy[8 + j], fy[i], voff[q], load_src(clamped(kt + 3), q),
                                                         load_dst(stage, q));
                } else {
                    detail::mfma_16x16x32_agpr(acc[i][j], fy[8 + j], fy[i]);
                }
            }
        }
    };
    if constexpr (T::kStages == 3) {
        // unrolled by three: the stage of every fragment read and load is a constant
        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;
        using S2 = std::integral_constant<int, 2>;
        int kt = 0;
        for (; kt + 2 < ktiles; kt += 3) {
            tile3(kt, S0{}, S1{});
            tile3(kt + 1, S1{}, S2{});
            tile3(kt + 2, S2{}, S0{});
        }
        if (kt < ktiles) tile3(kt, S0{}, S1{});
        if (kt + 1 < ktiles) tile3(kt + 1, S1{}, S2{});
        detail::wait_vmcnt<0>();  // (the last loads, of data nobody uses, have landed before the workgroup ends)
    } else {
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        constexpr int kTailTiles = kTail ? 1 : 0;  // (the tile that requests a partial last tile is not part of the loop)
        int kt = 0;
        for (; kt + 3 + kTailTiles < ktiles; kt += 2) {
            tile(kt, std::true_type{}, std::true_type{}, std::false_type{}, I0{});
            tile(kt + 1, std::true_type{}, std::true_type{}, std::false_type{}, I1{});
        }
        // the tiles behind the unrolled loop: one more that loads a tile, then the last two peeled
        for (; kt + 2 + kTailTiles < ktiles; ++kt) tile(kt, std::true_type{}, std::true_type{}, std::false_type{}, kt & 1);
        if constexpr (kTail) {  // the iteration that loads the last tile: with the offsets of a partial one
            if (kt + 2 < ktiles) {
                tile(kt, std::true_type{}, std::true_type{}, std::true_type{}, kt & 1);
                ++kt;
            }
        }
        if (kt + 1 < ktiles) {
            tile(kt, std::true_type{}, std::false_type{}, std::false_type{}, kt & 1);
            ++kt;
        }
        tile(kt, std::false_type{}, std::false_type{}, std::false_type{}, kt & 1);
    }

    // the compiler does not know the statements above are MFMAs: wait once for the last results, then pass every
    // accumulator through a statement that comes after the wait
    detail::mfma_results_wait();
#pragma unroll
    for (int i = 0; i < 8; ++i) pin_row(acc[i]);

    // C leaves through non-temporal stores of whole rows: the XCDs' L2s are not coherent with each other, so whatever a
    // kernel leaves dirty in them is written back when it ends, after the last wavefront - lines streamed out while
    // others still compute are not (f16, 4096^3: -1.5 %, 4096 x 4096 x 1024: -3.5 %)
    auto store_c = [](auto* p, const auto& v) { __builtin_nontemporal_store(v, p); };
    // ---- epilogue: acc[i][j][e] = C[16 i + lane % 16][16 j + 4 (lane / 16) + e] of the wavefront's block
    if constexpr (sizeof(OutType) == 2) {
        // f16: 16 rows at a time through a private LDS buffer (beyond the operand stages, so no workgroup barrier),
        // so that global stores are 16 bytes per lane and row-contiguous; two buffers per wavefront, so the
        // conversion and staging of rows 16 (i + 1).. overlap the stores of rows 16 i..
        constexpr int kPitch = T::kWaveN * 2;              // 256 (128) bytes per staged row
        constexpr int kSlotMask = (kPitch / 8 - 1) & ~1;   // 8-byte slots of a row are XOR-ed with 2 * row
        constexpr int kLanesPerRow = kPitch / 16, kRowsPerRead = kWaveSize / kLanesPerRow, kReads = 16 / kRowsPerRead;
        unsigned char* stg = lds + T::kLdsBytesMain + wave * T::kEpilogueBytesPerWave;
        // read-back: 16 (8) lanes x 16 B per row, 4 (8) rows per instruction
        const int rr = lane / kLanesPerRow, cc = lane % kLanesPerRow;
        OutType* cbase = C + size_t(m0 + wave_m * T::kWaveM) * ldc + n0 + wave_n * T::kWaveN;
        // LDS addresses of this lane's 8 staging writes and 4 read-backs of a row group (the same for every group but
        // for the buffer), computed once: with one wavefront per SIMD the epilogue is bound by instruction issue
        unsigned int waddr[kNT], raddr[kReads];
        const unsigned int stg_base = static_cast<unsigned int>(reinterpret_cast<uintptr_t>(stg));
#pragma unroll
        for (int j = 0; j < kNT; ++j) {
            const int slot = (j * 16 + 4 * fquad) >> 2;
            waddr[j] = stg_base + frow * kPitch + (slot ^ ((frow << 1) & kSlotMask)) * 8;
            asm volatile("" : "+v"(waddr[j]));
        }
#pragma unroll
        for (int it = 0; it < kReads; ++it) {
            const int row = it * kRowsPerRead + rr;
            raddr[it] = stg_base + row * kPitch + ((2 * cc) ^ ((row << 1) & kSlotMask)) * 8;
            asm volatile("" : "+v"(raddr[it]));
        }
        using lds_f16x4_ptr = __attribute__((address_space(3))) f16x4*;
        using lds_u32x4_ptr = __attribute__((address_space(3))) const u32x4*;
        unsigned char* crow = reinterpret_cast<unsigned char*>(cbase + size_t(rr) * ldc) + cc * 16;  // row rr of the block
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const unsigned int buf = (i & 1) * (16 * kPitch);
#pragma unroll
            for (int j = 0; j < kNT; ++j) {
                f16x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = static_cast<_Float16>(acc[i][j][e]);
                *reinterpret_cast<lds_f16x4_ptr>(waddr[j] + buf) = v;
            }
            // LDS operations of one wavefront execute in order: the reads below see the writes above
#pragma unroll
            for (int it = 0; it < kReads; ++it) {
                const u32x4 v = *reinterpret_cast<lds_u32x4_ptr>(raddr[it] + buf);
                if (!kEdges || (m0 + wave_m * T::kWaveM + i * 16 + it * kRowsPerRead + rr < M &&
                                n0 + wave_n * T::kWaveN + cc * 8 < N))
                    store_c(reinterpret_cast<u32x4*>(crow + size_t(i * 16 + it * kRowsPerRead) * ldc * sizeof(OutType)), v);
            }
        }
    } else {
        // f32: the same through one buffer of 16 rows (512 or 256 bytes each: the 16-byte slots of a row XOR-ed with the
        // row, so that the 16 rows a write instruction touches fall into different banks) - an accumulator register
        // holds 4 columns of 16 different rows, and 16-byte pieces of 16 rows per store instruction are what the
        // memory side handles worst
        constexpr int kPitch = T::kWaveN * 4;
        constexpr int kLanesPerRow = kPitch / 16, kRowsPerRead = kWaveSize / kLanesPerRow, kReads = 16 / kRowsPerRead;
        static_assert(16 * kPitch <= T::kEpilogueBytesPerWave);
        const unsigned int stg_base =
            static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds + T::kLdsBytesMain + wave * T::kEpilogueBytesPerWave));
        const int rr = lane / kLanesPerRow, cc = lane % kLanesPerRow;
        unsigned int waddr[kNT], raddr[kReads];
#pragma unroll
        for (int j = 0; j < kNT; ++j) {
            waddr[j] = stg_base + frow * kPitch + ((j * 4 + fquad) ^ frow) * 16;
            asm volatile("" : "+v"(waddr[j]));
        }
#pragma unroll
        for (int it = 0; it < kReads; ++it) {
            const int row = it * kRowsPerRead + rr;
            raddr[it] = stg_base + row * kPitch + (cc ^ row) * 16;
            asm volatile("" : "+v"(raddr[it]));
        }
        using lds_f32x4_ptr = __attribute__((address_space(3))) f32x4*;
        using lds_u32x4_ptr = __attribute__((address_space(3))) const u32x4*;
        OutType* cbase = C + size_t(m0 + wave_m * T::kWaveM) * ldc + n0 + wave_n * T::kWaveN;
        unsigned char* crow = reinterpret_cast<unsigned char*>(cbase + size_t(rr) * ldc) + cc * 16;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int j = 0; j < kNT; ++j) *reinterpret_cast<lds_f32x4_ptr>(waddr[j]) = acc[i][j];
            // LDS operations of one wavefront execute in order: the reads see the writes above, and the next group's
            // writes come behind them
#pragma unroll
            for (int it = 0; it < kReads; ++it) {
                const u32x4 v = *reinterpret_cast<lds_u32x4_ptr>(raddr[it]);
                if (!kEdges || (m0 + wave_m * T::kWaveM + i * 16 + it * kRowsPerRead + rr < M &&
                                n0 + wave_n * T::kWaveN + cc * 4 < N))
                    __builtin_nontemporal_store(
                        v, reinterpret_cast<u32x4*>(crow + size_t(i * 16 + it * kRowsPerRead) * ldc * sizeof(OutType)));
            }
        }
    }
}

}  // namespace tiledcuda::kernels
