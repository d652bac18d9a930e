// Pipelined fp16 GEMM for gfx950: C[M, N] = A[M, K] · B, A row-major, B column-major (stored
// [N, K]), f32 accumulate, C row-major in f16 or f32. This is the multi-stage kernel the
// reference's examples/cpp/01_gemm/02_gemm_all_mem/gemm.hpp:103-155 lacks (it has one LDS
// stage and waits for every load), built for the CDNA4 execution model:
//   * one workgroup of kWM x kWN wavefronts per kBM x kBN tile of C, accumulators resident in
//     registers for the whole K loop; the MFMA is v_mfma_f32_16x16x32_f16: on random operands the
//     matrix pipe is power-limited, and this shape sustains a ~12 % higher clock than
//     v_mfma_f32_32x32x16_f16 at the same LDS traffic (the kernel measured 15-20 % faster with it);
//   * A and B tiles go global -> LDS directly (global_load_lds_dwordx4, 16 B per lane, no
//     VGPR staging; staging through registers measured 10 % slower), kStages LDS buffers; the
//     loads of tile k+1 are issued during the first k-substep of tile k and awaited before the
//     last, which leaves them half a tile of MFMA time to land;
//   * LDS rows are kBK halves (128 B for kBK = 64); the 16-byte chunks of a row are
//     XOR-permuted with (row / 2) % 8 so that the ds_read_b128 of 16 consecutive rows at one
//     k-offset is bank-conflict free; the permutation is applied on the global-address side
//     because a direct-to-LDS load writes 64 lanes x 16 B contiguously;
//   * register double-buffering of the MFMA operands: the ds_reads of k-substep kk+1 are
//     issued before the MFMAs of substep kk; the barrier that hands over an LDS stage sits
//     before the last substep so its latency hides under that substep's MFMAs;
//   * the result is staged through LDS so that global stores are full 16-byte, row-contiguous;
//   * workgroup ids are remapped so that the 32 workgroups an XCD receives (ids congruent
//     modulo 8) form a compact block of tiles and share A / B panels in that XCD's L2.
// M % kBM == 0, N % kBN == 0, K % kBK == 0 are required (checked by the host launcher).
#pragma once

#include <utility>

#include "config.hpp"
#include "hip_utils.hpp"

namespace tiledcuda::kernels {

template <const int kBM_, const int kBN_, const int kBK_, const int kWM_, const int kWN_, const int kStages_ = 2>
struct PipelinedGemmTraits {
    static constexpr int kBM = kBM_, kBN = kBN_, kBK = kBK_, kWM = kWM_, kWN = kWN_, kStages = kStages_;
    static constexpr int kWaves = kWM * kWN;
    static constexpr int kThreads = kWaves * kWaveSize;

    static constexpr int kWaveM = kBM / kWM;  // rows of C per wavefront
    static constexpr int kWaveN = kBN / kWN;
    static constexpr int kMT = kWaveM / 16;  // 16x16 MFMA tiles per wavefront along M
    static constexpr int kNT = kWaveN / 16;
    static constexpr int kKS = kBK / 32;  // MFMA k-substeps (32 wide) per LDS tile

    static_assert(kBK == 64, "LDS rows are 128 bytes: kBK must be 64 halves");
    static_assert(kStages >= 2 && kStages <= 4, "2 LDS stages (a 256 x 256 x 64 stage is 64 KiB of the CU's 160 KiB) or a "
                                                "ring of 3 or 4 for the smaller tiles");
    static_assert(kWaveM % 16 == 0 && kWaveN % 16 == 0, "a wavefront owns whole 16x16 MFMA tiles");

    static constexpr int kRowBytes = kBK * 2;                    // 128
    static constexpr int kABytes = kBM * kRowBytes;              // one stage of A
    static constexpr int kBBytes = kBN * kRowBytes;              // one stage of B
    static constexpr int kStageBytes = kABytes + kBBytes;
    static constexpr int kRowsPerLoad = 1024 / kRowBytes;        // 8 rows per direct-to-LDS instruction
    static constexpr int kALoads = kBM / kRowsPerLoad / kWaves;  // instructions per wavefront per stage
    static constexpr int kBLoads = kBN / kRowsPerLoad / kWaves;
    static_assert(kBM % (kRowsPerLoad * kWaves) == 0 && kBN % (kRowsPerLoad * kWaves) == 0,
                  "the tile rows must divide evenly over the wavefronts' 8-row loads");

    // epilogue staging: every wavefront stages its kWaveM x kWaveN block, kEpiBytes per element
    static constexpr int kLdsBytesMain = kStages * kStageBytes;
    template <typename OutType>
    static constexpr int epilogue_bytes() {
        return kWaves * kWaveM * kWaveN * int(sizeof(OutType));
    }
    template <typename OutType>
    static constexpr int lds_bytes() {
        // f32 output is stored directly from registers (no staging), so only f16 needs the space
        return sizeof(OutType) == 2 && epilogue_bytes<OutType>() > kLdsBytesMain ? epilogue_bytes<OutType>()
                                                                                 : kLdsBytesMain;
    }
};

namespace detail {

/// f(integral_constant<int, 0>) ... f(integral_constant<int, kN - 1>): a loop whose index is a constant expression
/// (wait counts and instruction offsets below are immediates).
template <int kN, typename F, int... kIs>
DEVICE void static_for_impl(F&& f, std::integer_sequence<int, kIs...>) {
    (f(std::integral_constant<int, kIs>{}), ...);
}
template <int kN, typename F>
DEVICE void static_for(F&& f) {
    static_for_impl<kN>(f, std::make_integer_sequence<int, kN>{});
}

using lds_ptr_t = __attribute__((address_space(3))) void*;
using glb_ptr_t = const __attribute__((address_space(1))) void*;

/// 16 bytes per lane, global -> LDS, no register staging. `lds_wave_base` must be wave-uniform;
/// lane i's data lands at lds_wave_base + 16 * i.
DEVICE void load_lds_16B(const void* gptr, void* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((glb_ptr_t)gptr, (lds_ptr_t)lds_wave_base, 16, 0, 0);
}

/// Direct-to-LDS load of 16 bytes per lane (lane i's data lands at lds_wave_base + 16 i) issued as inline assembly, so
/// that the compiler does not know it writes LDS. With the builtin, the compiler makes every later LDS read (and every
/// barrier fence) wait for *all* outstanding direct-to-LDS loads (s_waitcnt vmcnt(0)), because it cannot prove that the
/// read does not alias a tile still in flight; that serialises a ring of stages to one tile at a time. Here the
/// kernel's own s_waitcnt vmcnt(N) before the barrier that hands a stage over is the only synchronisation.
/// kAgentScope: request at agent scope (sc1), past this XCD's L2, for data written by other workgroups in this launch.
template <bool kAgentScope = false>
DEVICE void load_lds_16B_untracked(const void* gptr, const void* lds_wave_base) {
    const unsigned int lds_addr = __builtin_amdgcn_readfirstlane(
        static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds_wave_base)));
    if constexpr (kAgentScope)
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off sc1" ::"v"(gptr), "s"(lds_addr) : "m0", "memory");
    else
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_addr) : "m0", "memory");
}

/// Untracked direct-to-LDS load of 16 bytes per lane from sbase + voff (a wave-uniform 64-bit base in scalar registers
/// plus a 32-bit byte offset per lane: no 64-bit address arithmetic per load) to lds_addr + 16 * lane.
DEVICE void load_lds_16B_sbase(unsigned int voff, const void* sbase, unsigned int lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr)
                 : "m0", "memory");
}

/// Wait until at most kVmcnt of this wavefront's vector-memory operations are outstanding (nothing else).
template <int kVmcnt>
DEVICE void wait_vmcnt() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0f70 | (kVmcnt & 0xF) | ((kVmcnt >> 4) << 14));  // vmcnt(kVmcnt), others at their maximum
    asm volatile("" ::: "memory");
}

/// MFMA results may be read by other instructions only a number of issue slots after the MFMA was issued, and where
/// the MFMAs are assembly statements the compiler does not know that and would not wait. One call of this after the
/// last MFMA (20 issue slots of 4 cycles each: the longest requirement, that of a 16-pass instruction, is 19), then
/// every accumulator passes through an (empty) volatile statement of its own before it is read: volatile statements
/// keep their order, so all of those come after this one. An s_nop of N + 1 slots costs 4 (N + 1) cycles - a wait per
/// accumulator, which is how this was first written, cost the GEMM epilogue 1024 cycles instead of 80.
DEVICE void mfma_results_wait() { asm volatile("s_nop 15\n\ts_nop 3"); }

/// Workgroup barrier that orders LDS accesses only. __syncthreads() also waits for every outstanding global memory
/// operation of the wavefront (s_waitcnt vmcnt(0): its workgroup fence covers the LDS writes of direct-to-LDS loads),
/// which would drain a ring of stages at every hand-over: tiles requested ahead must stay in flight across the barrier.
/// kVmcnt: additionally wait until at most that many of this wavefront's vector-memory operations are outstanding.
/// The empty asm statements keep the compiler from moving LDS accesses across the sequence (the two builtins are
/// declared as not touching memory).
template <int kVmcnt = 63>
DEVICE void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070 | (kVmcnt & 0xF) | ((kVmcnt >> 4) << 14));  // vmcnt(kVmcnt) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

/// Tile coordinates for workgroup `bid` of a grid of tiles_m x tiles_n tiles: ids that are
/// congruent modulo 8 (same XCD) are gathered into compact blocks of tiles. Any grid: with total = 8 q + r tiles the
/// first r XCDs hold q + 1 ids and the others q, each XCD takes a run of that many consecutive positions of a walk
/// through the grid in row panels 4 tiles tall (the last panel has the tiles_m % 4 rows that are left).
HOST_DEVICE void xcd_tile_coords(int bid, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
    const int total = tiles_m * tiles_n;
    constexpr int kXcds = 8;
    const int q = total / kXcds, r = total % kXcds;
    const int xcd = bid % kXcds;
    const int local = bid / kXcds;
    const int lin = xcd * q + (xcd < r ? xcd : r) + local;  // consecutive `lin` = same XCD
    const int whole = (tiles_m / 4) * 4 * tiles_n;          // positions inside panels of full height
    if (lin < whole) {
        const int panel = lin / (4 * tiles_n);
        const int in_panel = lin % (4 * tiles_n);
        tile_m = panel * 4 + in_panel % 4;
        tile_n = in_panel / 4;
    } else {
        const int height = tiles_m % 4;
        const int in_panel = lin - whole;
        tile_m = (tiles_m / 4) * 4 + in_panel % height;
        tile_n = in_panel / height;
    }
}

}  // namespace detail

/// kEdges: M, N and K need not be multiples of the tile (multiples of 16 suffice): the grid covers ceil(M / kBM) x
/// ceil(N / kBN) tiles, rows beyond the edge are loaded from the last valid row (their products are computed and
/// dropped) and the stores are guarded; the loop runs over ceil(K / kBK) tiles, and in the last one every lane loads
/// the 16-byte pieces that lie beyond K from the start of its row instead and, once they have landed, overwrites them
/// in LDS with zeros. ldc: elements between consecutive rows of C (N for a dense C).
template <typename Traits, typename OutType, bool kEdges = false>
__global__ void __launch_bounds__(Traits::kThreads)
    gemm_pipelined(const __half* __restrict__ A, const __half* __restrict__ Bt, OutType* __restrict__ C, int M, int N,
                   int K, int ldc) {
    constexpr int kBM = Traits::kBM, kBN = Traits::kBN, kBK = Traits::kBK;
    constexpr int kMT = Traits::kMT, kNT = Traits::kNT, kKS = Traits::kKS;

    extern __shared__ __align__(1024) unsigned char lds[];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int wave_m = wave / Traits::kWN;
    const int wave_n = wave % Traits::kWN;

    int tile_m, tile_n;
    detail::xcd_tile_coords(blockIdx.x, kEdges ? (M + kBM - 1) / kBM : M / kBM, kEdges ? (N + kBN - 1) / kBN : N / kBN,
                            tile_m, tile_n);
    const int m0 = tile_m * kBM;
    const int n0 = tile_n * kBN;

    // ---- global -> LDS addressing -------------------------------------------------------
    // Load instruction j of this wavefront fills LDS rows [8 * g, 8 * g + 8), g = wave * kLoads + j.
    // Lane i writes physical chunk p = i % 8 of row 8 * g + i / 8, which must hold logical chunk
    // p ^ ((row / 2) % 8).
    const int lrow = lane >> 3;  // row within the 8-row group
    const int lchk = lane & 7;   // physical 16-byte chunk
    // Each load's source is a wave-uniform base (the tile's first row at the k-tile, in scalar registers) plus a byte
    // offset per lane that is fixed for the whole kernel: one 32-bit register per load instruction. Offsets stay below
    // kBM * K * 2 bytes, so K up to 2^23 / (kBM / 256) fits.
    auto row_chunk = [&](int loads_per_wave, int j) {
        const int row = (wave * loads_per_wave + j) * Traits::kRowsPerLoad + lrow;
        return lchk ^ ((row >> 1) & 7);
    };
    unsigned int a_off[Traits::kALoads], b_off[Traits::kBLoads];
#pragma unroll
    for (int j = 0; j < Traits::kALoads; ++j) {
        const int row = (wave * Traits::kALoads + j) * Traits::kRowsPerLoad + lrow;
        a_off[j] = unsigned(kEdges && m0 + row >= M ? M - 1 - m0 : row) * unsigned(K) * 2u + row_chunk(Traits::kALoads, j) * 16;
    }
#pragma unroll
    for (int j = 0; j < Traits::kBLoads; ++j) {
        const int row = (wave * Traits::kBLoads + j) * Traits::kRowsPerLoad + lrow;
        b_off[j] = unsigned(kEdges && n0 + row >= N ? N - 1 - n0 : row) * unsigned(K) * 2u + row_chunk(Traits::kBLoads, j) * 16;
    }
    const unsigned char* a_tile = reinterpret_cast<const unsigned char*>(A + size_t(m0) * K);
    const unsigned char* b_tile = reinterpret_cast<const unsigned char*>(Bt + size_t(n0) * K);
    // kEdges: the k-tile that straddles K asks for pieces beyond the end of their row; those land in LDS and are
    // overwritten with zeros there (zero_k_tail), so any readable address serves: the offset is limited to the last
    // 16 bytes of the matrix, which only the last row's pieces exceed.
    const size_t a_left = (size_t(M - m0) * K - 8) * 2, b_left = (size_t(N - n0) * K - 8) * 2;
    const unsigned int a_limit = a_left < 0xfffffff0u ? unsigned(a_left) : 0xfffffff0u;
    const unsigned int b_limit = b_left < 0xfffffff0u ? unsigned(b_left) : 0xfffffff0u;
    auto a_src = [&](int j, int k0) -> const unsigned char* {
        const unsigned int off = a_off[j] + unsigned(k0) * 2u;
        return a_tile + (kEdges ? (off < a_limit ? off : a_limit) : off);
    };
    auto b_src = [&](int j, int k0) -> const unsigned char* {
        const unsigned int off = b_off[j] + unsigned(k0) * 2u;
        return b_tile + (kEdges ? (off < b_limit ? off : b_limit) : off);
    };
    // Issue part `part` of `nparts` of the loads of one stage (A instructions first, then B). Splitting a stage's
    // loads over the k-substeps keeps the vector-memory path evenly busy instead of bursting after the barrier.
    auto issue_part = [&](int stage, int k0, int part, int nparts) {
        unsigned char* sa = lds + stage * Traits::kStageBytes;
        unsigned char* sb = sa + Traits::kABytes;
        constexpr int kTot = Traits::kALoads + Traits::kBLoads;
        const int per = (kTot + nparts - 1) / nparts;
#pragma unroll
        for (int q = 0; q < kTot; ++q) {
            if (q / per != part) continue;
            if (q < Traits::kALoads)
                detail::load_lds_16B(a_src(q, k0), sa + (wave * Traits::kALoads + q) * 1024);
            else
                detail::load_lds_16B(b_src(q - Traits::kALoads, k0),
                                     sb + (wave * Traits::kBLoads + (q - Traits::kALoads)) * 1024);
        }
    };
    auto issue_stage = [&](int stage, int k0) { issue_part(stage, k0, 0, 1); };
    // kEdges, last k-tile when K % kBK != 0: what this lane loaded from beyond K (it sits at 16 * lane of each of this
    // wavefront's 1 KiB pieces) becomes zero. Call after the loads have landed, before the barrier that hands the stage over.
    auto zero_k_tail = [&](int stage, int k0) {
        unsigned char* sa = lds + stage * Traits::kStageBytes;
        unsigned char* sb = sa + Traits::kABytes;
        const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int q = 0; q < Traits::kALoads + Traits::kBLoads; ++q) {
            const bool is_a = q < Traits::kALoads;
            const int j = is_a ? q : q - Traits::kALoads;
            const int row = (wave * (is_a ? Traits::kALoads : Traits::kBLoads) + j) * Traits::kRowsPerLoad + lrow;
            const int chunk = lchk ^ ((row >> 1) & 7);
            if (k0 + chunk * 8 >= K)
                *reinterpret_cast<u32x4*>((is_a ? sa : sb) + (wave * (is_a ? Traits::kALoads : Traits::kBLoads) + j) * 1024 +
                                          lane * 16) = zero;
        }
    };

    // ---- LDS -> register addressing -----------------------------------------------------
    // 16x16x32 operand: lane l holds row l % 16, k = 8 * (l / 16) .. +7 of the 32-wide substep,
    // i.e. logical chunk 4 * kk + l / 16 of its row.
    const int frow = lane & 15;
    const int fquad = lane >> 4;
    auto read_frag = [&](const unsigned char* base, int row, int kk) -> f16x8 {
        const int chunk = (4 * kk + fquad) ^ ((row >> 1) & 7);
        return *reinterpret_cast<const f16x8*>(base + row * Traits::kRowBytes + chunk * 16);
    };

    f32x4 acc[kMT][kNT];
#pragma unroll
    for (int i = 0; i < kMT; ++i)
#pragma unroll
        for (int j = 0; j < kNT; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;

    f16x8 fa[2][kMT], fb[2][kNT];

    auto load_frags = [&](int buf, int stage, int kk) {
        const unsigned char* sa = lds + stage * Traits::kStageBytes;
        const unsigned char* sb = sa + Traits::kABytes;
#pragma unroll
        for (int i = 0; i < kMT; ++i) fa[buf][i] = read_frag(sa, wave_m * Traits::kWaveM + i * 16 + frow, kk);
#pragma unroll
        for (int j = 0; j < kNT; ++j) fb[buf][j] = read_frag(sb, wave_n * Traits::kWaveN + j * 16 + frow, kk);
    };
    auto mma = [&](int buf) {
#pragma unroll
        for (int i = 0; i < kMT; ++i)
#pragma unroll
            for (int j = 0; j < kNT; ++j)
                // operands swapped: the accumulator then holds C (not C^T): row l % 16, the 4 consecutive
                // columns 4 * (l / 16) .. +3
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
    };

    const int ktiles = kEdges ? (K + kBK - 1) / kBK : K / kBK;
    const bool k_tail = kEdges && K % kBK != 0;

    if constexpr (Traits::kStages > 2) {
        // ---- ring of kStages stages: kStages - 1 tiles in flight behind the one being multiplied ----------------
        // The loads are issued as assembly the compiler does not track (it would otherwise make every LDS read wait
        // for all of them); the kernel's own vmcnt waits before the barrier that hands a stage over are the
        // synchronisation. A small tile has few MFMAs per k-tile, so its loop is bound by the latency of one tile's
        // loads divided by the number of tiles in flight.
        constexpr int S = Traits::kStages;
        constexpr int L = Traits::kALoads + Traits::kBLoads;  // vector-memory operations per wavefront per tile
        static_assert((S - 2) * L <= 63, "the vmcnt field counts to 63");
        const unsigned int lds_base = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds)));
        auto issue_ring = [&](int stage, int k0) {
            const unsigned int sa = lds_base + stage * Traits::kStageBytes, sb = sa + Traits::kABytes;
#pragma unroll
            for (int q = 0; q < Traits::kALoads; ++q) {
                if constexpr (kEdges) {
                    const unsigned int off = a_off[q] + unsigned(k0) * 2u;
                    detail::load_lds_16B_sbase(off < a_limit ? off : a_limit, a_tile, sa + (wave * Traits::kALoads + q) * 1024);
                } else {
                    detail::load_lds_16B_sbase(a_off[q], a_tile + size_t(k0) * 2, sa + (wave * Traits::kALoads + q) * 1024);
                }
            }
#pragma unroll
            for (int q = 0; q < Traits::kBLoads; ++q) {
                if constexpr (kEdges) {
                    const unsigned int off = b_off[q] + unsigned(k0) * 2u;
                    detail::load_lds_16B_sbase(off < b_limit ? off : b_limit, b_tile, sb + (wave * Traits::kBLoads + q) * 1024);
                } else {
                    detail::load_lds_16B_sbase(b_off[q], b_tile + size_t(k0) * 2, sb + (wave * Traits::kBLoads + q) * 1024);
                }
            }
        };
        // wait until this wavefront's loads of a tile have landed, `behind` later tiles' loads still in flight
        auto wait_tile = [&](int behind) {
            if (behind >= S - 2) detail::wait_vmcnt<(S - 2) * L>();
            else if (S > 3 && behind == 1) detail::wait_vmcnt<L>();
            else detail::wait_vmcnt<0>();
        };
#pragma unroll
        for (int s = 0; s < S; ++s)
            if (s < ktiles) issue_ring(s, s * kBK);
        wait_tile(ktiles - 1 < S - 1 ? ktiles - 1 : S - 1);
        if (k_tail && ktiles == 1) zero_k_tail(0, 0);
        detail::lds_barrier<63>();
        load_frags(0, 0, 0);

        int stage = 0;
        for (int kt = 0; kt < ktiles; ++kt) {
            const int next_stage = stage + 1 == S ? 0 : stage + 1;
#pragma unroll
            for (int kk = 0; kk < kKS - 1; ++kk) {
                load_frags((kk + 1) & 1, stage, kk + 1);
                mma(kk & 1);
            }
            if (kt + 1 < ktiles) {
                // tile kt+1 is followed by tiles kt+2 .. min(kt+S-1, ktiles-1) (tile kt+S goes out after the barrier)
                const int behind = ktiles - 2 - kt;
                wait_tile(behind < S - 2 ? behind : S - 2);
                if (k_tail && kt + 2 == ktiles) zero_k_tail(next_stage, (kt + 1) * kBK);
                // every LDS read of `stage` has been issued; once they have returned everywhere it can be refilled
                detail::lds_barrier<63>();
                if (kt + S < ktiles) issue_ring(stage, (kt + S) * kBK);
                load_frags(kKS & 1, next_stage, 0);
            }
            mma((kKS - 1) & 1);
            stage = next_stage;
        }
    } else {
        // prologue: tile 0 -> stage 0
        issue_stage(0, 0);
        __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
        if (k_tail && ktiles == 1) zero_k_tail(0, 0);
        __syncthreads();
        load_frags(0, 0, 0);

        int stage = 0;
        for (int kt = 0; kt < ktiles; ++kt) {
            const int next_stage = stage ^ 1;
    #pragma unroll
            for (int kk = 0; kk < kKS - 1; ++kk) {
                // tile kt+1 goes to the other stage, which everyone left at the barrier of iteration kt-1;
                // its loads are issued during this iteration's first kKS-1 substeps
                if (kt + 1 < ktiles) issue_part(next_stage, (kt + 1) * kBK, kk, kKS - 1);
                load_frags((kk + 1) & 1, stage, kk + 1);
                mma(kk & 1);
            }
            // Every LDS read of `stage` has been issued; once they return, tile kt+1 has landed and all
            // wavefronts agree, the other stage can be read (and this one refilled in the next iteration).
            if (kt + 1 < ktiles) {
                __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
                if (k_tail && kt + 2 == ktiles) zero_k_tail(next_stage, (kt + 1) * kBK);
                __syncthreads();
                load_frags(kKS & 1, next_stage, 0);
            }
            mma((kKS - 1) & 1);
            stage = next_stage;
        }
    }

    // ---- epilogue -----------------------------------------------------------------------
    // acc[i][j][r]: row = lane % 16, col = 4 * (lane / 16) + r of the 16x16 tile.
    if constexpr (sizeof(OutType) == 2) {
        __syncthreads();  // everyone is done with the operand stages
        constexpr int kWaveN = Traits::kWaveN, kWaveM = Traits::kWaveM;
        static_assert((kWaveN & (kWaveN - 1)) == 0 && kWaveN >= 16 && kWaveN <= 512 && kWaveM % (kWaveSize / (kWaveN / 8)) == 0,
                      "f16 epilogue: a staged row is a power-of-two number of 16-byte pieces, read back by whole wavefronts");
        constexpr int kPitch = kWaveN * 2;  // bytes per staged row
        unsigned char* stg = lds + wave * (kWaveM * kPitch);
        // write: lane owns row i*16 + frow; 4 halves (8 B) at column j*16 + 4*fquad.
        // 8-byte slots of a row are XOR-ed with (row % 16) * 2 (bit 0 untouched, kept inside the row)
        // to spread banks.
        constexpr int kSlotMask = (kPitch / 8 - 1) & ~1;
#pragma unroll
        for (int i = 0; i < kMT; ++i) {
            const int row = i * 16 + frow;
#pragma unroll
            for (int j = 0; j < kNT; ++j) {
                const int slot = (j * 16 + 4 * fquad) >> 2;  // 8-byte slot index in the row
                const int pslot = slot ^ (((row & 15) << 1) & kSlotMask);
                f16x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = static_cast<_Float16>(acc[i][j][e]);
                *reinterpret_cast<f16x4*>(stg + row * kPitch + pslot * 8) = v;
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's staging writes are done
        // read back 16 B per lane, row-contiguous: kWaveN / 8 lanes per row
        constexpr int kLanesPerRow = kWaveN / 8;
        constexpr int kRowsPerIter = kWaveSize / kLanesPerRow;
        const int rr = lane / kLanesPerRow;
        const int cc = lane % kLanesPerRow;  // 16-byte chunk = 8-byte slots 2cc, 2cc+1
        OutType* cbase = C + size_t(m0 + wave_m * kWaveM) * ldc + n0 + wave_n * kWaveN;
#pragma unroll
        for (int it = 0; it < kWaveM / kRowsPerIter; ++it) {
            const int row = it * kRowsPerIter + rr;
            const int pslot = (2 * cc) ^ (((row & 15) << 1) & kSlotMask);
            const u32x4 v = *reinterpret_cast<const u32x4*>(stg + row * kPitch + pslot * 8);
            if (kEdges && (m0 + wave_m * kWaveM + row >= M || n0 + wave_n * kWaveN + cc * 8 >= N)) continue;
            *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(cbase + size_t(row) * ldc) + cc * 16) = v;
        }
    } else {
        OutType* cbase = C + size_t(m0 + wave_m * Traits::kWaveM) * ldc + n0 + wave_n * Traits::kWaveN;
#pragma unroll
        for (int i = 0; i < kMT; ++i) {
#pragma unroll
            for (int j = 0; j < kNT; ++j) {
                if (kEdges && (m0 + wave_m * Traits::kWaveM + i * 16 + frow >= M ||
                               n0 + wave_n * Traits::kWaveN + j * 16 + 4 * fquad >= N))
                    continue;
                *reinterpret_cast<f32x4*>(cbase + size_t(i * 16 + frow) * ldc + j * 16 + 4 * fquad) = acc[i][j];
            }
        }
    }
}

}  // namespace tiledcuda::kernels
