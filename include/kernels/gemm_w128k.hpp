// fp16 GEMM for gfx950 with one wavefront per SIMD and the four wavefronts of a workgroup splitting K: for products
// with too few 256 x 256 tiles to fill 256 CUs (2048^3 has 64) but enough 128 x 128 tiles. Same contract as
// kernels/gemm_w128.hpp (C[M, N] = A[M, K] . B, A row-major, B column-major = stored [N, K], f32 accumulate, C
// row-major f16 or f32; the multi-stage counterpart of the reference's examples/cpp/01_gemm/02_gemm_all_mem/gemm.hpp:103-155).
//   * With 128 x 128 workgroup tiles split 2 x 2 over wavefronts (64 x 64 each) every 16 matrix instructions need 8
//     ds_read_b128: four wavefronts then ask for 128 bytes of LDS per cycle at the matrix pipe's peak rate, which is
//     all the LDS delivers - that tiling is bound by LDS reads. Here every wavefront owns the WHOLE 128 x 128 tile
//     (16 reads per 64 instructions, half the LDS traffic, the gemm_w128 ratio) over a quarter of K: a tile of K is
//     128 wide, wavefront w multiplies columns 32 w .. 32 w + 31 of it. The four partial tiles are added through LDS
//     at the end, after which wavefront w holds rows 32 w .. 32 w + 31 of the result and stores them.
//   * The A part and the B part of a tile of K (128 rows of 256 bytes = 32 KiB each) pass through a ring of five 32 KiB
//     slots in the order A0 B0 A1 B1 A2 ... One phase per tile of K: 64 MFMAs, with the 16 fragment reads of the next
//     tile (one per two MFMAs) and this wavefront's 16 direct-to-LDS loads (one per four MFMAs, each in one statement
//     with its MFMA): first B of the tile after the next, then A of the one after that, into the two slots the current
//     tile came from; then one LDS-only barrier, which waits for that B part but not for the A part requested behind it.
//     B has most of a phase to land and A a phase more. (With two stages of 64 KiB the last load of a tile was
//     requested at the very end of the phase whose closing barrier waited for it, so a phase took as long as a load:
//     1.2 us at 2048^3 for 0.5 us of matrix work, whether the loads were issued one per four, three or two MFMAs. The
//     ring: 1536 x 1536 x 4096 32.4 -> 26.6 us, 2048^3 22.8 -> 21.9 us; a full third stage does not fit 160 KiB.)
//     Against the LDS-bound tiling: 2048^3 21.9 us against 26.8 us (the vendor library: 21-23.4 us).
//   * Accumulators in AGPRs through inline assembly, scalar-base addressing, XCD-aware tile order: as in gemm_w128.
// The sum over K is taken in four interleaved parts, so results differ from the other kernels by f32 rounding.
// The tile is 128 x 128 or 128 x 96 (GemmW128kTraitsN: the numbers above are those of the wider one).
// K % 128 == 0; M % 128 == 0 and N a multiple of the tile width, or with kEdges any M, N in multiples of 16: the grid
// then covers ceil(M / 128) x ceil(N / width) tiles, rows beyond the edge are loaded from the last valid row (their products are
// computed and dropped) and the stores are guarded per 16 x 16 block (checked by the launcher).
#pragma once

#include <type_traits>

#include "config.hpp"
#include "hip_utils.hpp"
#include "kernels/gemm_w128.hpp"  // detail::mfma_16x16x32_agpr{,_then_load}, load_lds_16B_sbase, lds_barrier

namespace tiledcuda::kernels {

/// kNT_: 16-column tiles of a workgroup's tile: 8 (128 x 128) or 6 (128 x 96, for products that would fill two thirds of
/// the chip with 128 x 128 tiles: a quarter more workgroups, each with a quarter less to multiply and an eighth less to
/// load).
template <const int kNT_ = 8>
struct GemmW128kTraitsN {
    static constexpr int kNT = kNT_;
    static constexpr int kBM = 128, kBN = 16 * kNT, kBK = 128;
    static constexpr int kWaves = 4, kThreads = kWaves * kWaveSize;
    static constexpr int kRowBytes = kBK * 2;                      // 256
    static constexpr int kABytes = kBM * kRowBytes, kBBytes = kBN * kRowBytes;
    static constexpr int kSlotBytes = kABytes;                     // a ring slot holds the A or the B part of a tile of K
    static constexpr int kSlots = 5;
    static constexpr int kLoads = kBM * kRowBytes / 1024 / kWaves;   // 1 KiB load instructions of A per wavefront
    static constexpr int kLoadsB = kBN * kRowBytes / 1024 / kWaves;  // ... of B: 8 (6)
    static constexpr int kFrags = 8 + kNT;                         // operand fragments of a phase
    static constexpr int kLdsBytes = kSlots * kSlotBytes;          // 160 KiB; the reduction reuses 128 of it
    static_assert(kLoads == 8 && (kNT == 8 || kNT == 6), "the phase schedule below is written for 8 + 8 or 8 + 6 loads per wavefront");
    static_assert(kLdsBytes <= kMaxLdsBytes && kBBytes <= kSlotBytes);
};
using GemmW128kTraits = GemmW128kTraitsN<8>;

/// grid = ((M / 128) * (N / kBN), splits), block = 256, dynamic LDS = T::kLdsBytes. lda / ldb / ldc: elements between
/// consecutive rows of A, of the stored [N, K] array and of C. kEdges: grid.x = ceil(M / 128) * ceil(N / kBN). With
/// splits > 1 workgroup row z multiplies the K-range [z K, (z + 1) K) of wider operands (lda, ldb >= splits * K) and
/// writes plane z of C ([splits, M, N]: partial sums for splitk_reduce).
template <typename OutType, bool kEdges = false, typename T = GemmW128kTraits>
__global__ void __launch_bounds__(T::kThreads)
    gemm_w128k(const __half* __restrict__ A, const __half* __restrict__ Bt, OutType* __restrict__ C, int M, int N, int K,
               int lda, int ldb, int ldc) {
    constexpr int kNT = T::kNT, kNumLoads = 8 + T::kLoadsB;
    extern __shared__ __align__(1024) unsigned char lds[];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    int tile_m, tile_n;
    detail::xcd_tile_coords(blockIdx.x, (M + T::kBM - 1) / T::kBM, (N + T::kBN - 1) / T::kBN, tile_m, tile_n);
    const int m0 = tile_m * T::kBM, n0 = tile_n * T::kBN;

    // ---- global -> LDS: load instruction q of this wavefront (q < 8: A, else B) fills 4 rows of 256 bytes; lane i
    // writes physical 16-byte chunk i % 16 of row i / 16, which must hold logical chunk (i % 16) ^ (row % 16).
    // kEdges: a row beyond the matrix is fetched from the last valid row instead (its LDS place and swizzle are its own)
    const int lrow = lane >> 4, lchk = lane & 15;
    unsigned int voff[kNumLoads];
#pragma unroll
    for (int q = 0; q < kNumLoads; ++q) {
        const int row = (q < 8 ? wave * T::kLoads + q : wave * T::kLoadsB + (q - 8)) * 4 + lrow;
        int src_row = row;
        if constexpr (kEdges) {
            const int last = (q < 8 ? M - m0 : N - n0) - 1;
            src_row = row < last ? row : last;
        }
        voff[q] = static_cast<unsigned int>(src_row) * static_cast<unsigned int>(q < 8 ? lda : ldb) * 2u + (lchk ^ (row & 15)) * 16;
    }
    const size_t z = blockIdx.y;
    const __half* a_base = A + size_t(m0) * lda + z * K;
    const __half* b_base = Bt + size_t(n0) * ldb + z * K;
    C += z * size_t(M) * ldc;
    const unsigned int lds_base = static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds));
    // The A and B parts of the tiles of K pass through a ring of five 32 KiB slots in the order A0 B0 A1 B1 A2 ...:
    // part u lives in slot u % 5 (A of tile t: u = 2 t, B: u = 2 t + 1).
    auto slot_bytes = [](int unit) -> unsigned int { return static_cast<unsigned int>(unit % T::kSlots) * T::kSlotBytes; };
    auto load_dst = [&](unsigned int slot, int q) -> unsigned int {
        return __builtin_amdgcn_readfirstlane(lds_base + slot +
                                              (q < 8 ? wave * T::kLoads + q : wave * T::kLoadsB + (q - 8)) * 1024);
    };
    auto load_src = [&](int kt, int q) -> const __half* { return (q < 8 ? a_base : b_base) + kt * T::kBK; };

    // ---- LDS -> registers: fragment r (r < 8: A rows 16 r .., else B rows 16 (r - 8) ..); lane l holds row l % 16,
    // k = 32 wave + 8 (l / 16) .. + 7 of the tile = logical chunk 4 wave + l / 16 of its row. The 16 rows a 16-lane
    // group reads have 16 different values of row % 16: 16 different chunks, no bank conflict.
    const int frow = lane & 15, fquad = lane >> 4;
    // The XOR term depends on lane % 16 only: the lane's address of fragment 0 of a slot is one register (frag_lane, fixed
    // for the kernel) plus the slot's offset - one addition per part and tile - and fragment r lies (r % 8) * 2 KiB
    // further on: an immediate.
    unsigned int frag_lane = lds_base + frow * T::kRowBytes + (((4 * wave + fquad) ^ frow) * 16);
    asm volatile("" : "+v"(frag_lane));
    auto read_frag = [&](unsigned int base_a, unsigned int base_b, int r) __attribute__((always_inline)) -> f16x8 {
        using lds_f16x8_ptr = __attribute__((address_space(3))) const f16x8*;
        return *reinterpret_cast<lds_f16x8_ptr>((r < 8 ? base_a : base_b) + (r & 7) * 16 * T::kRowBytes);
    };

    f16x8 fx[T::kFrags], fy[T::kFrags];  // fragments of the tile being multiplied / of the next one: [0..7] A, [8..] B
    const int ktiles = K / T::kBK;
    auto clamped = [&](int kt) { return kt < ktiles ? kt : ktiles - 1; };
    // prologue: A0 B0 A1 B1 A2 fill the ring
#pragma unroll
    for (int u = 0; u < T::kSlots; ++u) {
#pragma unroll
        for (int q = (u & 1) ? 8 : 0; q < ((u & 1) ? kNumLoads : 8); ++q)
            detail::load_lds_16B_sbase(voff[q], load_src(clamped(u >> 1), q), load_dst(u * T::kSlotBytes, q));
    }
    // the accumulators are pinned to the AGPR half row group by row group
    auto pin_row = [](f32x4 (&row)[kNT]) {
        if constexpr (kNT == 8)
            asm volatile("" : "+a"(row[0]), "+a"(row[1]), "+a"(row[2]), "+a"(row[3]), "+a"(row[4]), "+a"(row[5]), "+a"(row[6]), "+a"(row[7]));
        else
            asm volatile("" : "+a"(row[0]), "+a"(row[1]), "+a"(row[2]), "+a"(row[3]), "+a"(row[4]), "+a"(row[5]));
    };
    f32x4 acc[8][kNT];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int j = 0; j < kNT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        pin_row(acc[i]);
    }
    detail::lds_barrier<16 + T::kLoadsB>();  // tile 0 has landed (behind it: A1 B1 A2), for everyone
#pragma unroll
    for (int r = 0; r < T::kFrags; ++r) fx[r] = read_frag(frag_lane, frag_lane + T::kSlotBytes, r);

    // the order in which the fragments of the next tile are read: its first row group needs A fragment 0 and all of B
    auto order = [](int r) { return r == 0 ? 0 : r <= kNT ? 7 + r : r - kNT; };
    auto snake = [](int i, int n) { return (i & 1) ? kNT - 1 - n : n; };

    // One tile of K out of `cur`, reading the next tile's fragments into `nxt`, and loading B of tile kt + 2 and then A of
    // tile kt + 3 into the slots `cur`'s tile came from. B of a tile is requested first in its phase and has the rest
    // of it to land (the barrier at the top of the next phase waits for it, not for the A part requested behind it); A
    // has a phase more. With two 64 KiB stages the last load of a tile was requested at the very end of the phase
    // whose closing barrier waited for it: the phase took as long as a load.
    // Every phase is the same straight-line code: behind the last tile of K the fragment reads fetch stale data that
    // nobody uses and the loads fetch the last tile once more (clamped index) - cheaper than peeled copies of the
    // phase, whose control-flow merges made the compiler shuffle and spill accumulators between the assembly
    // statements, where it knows of no wait states.
    auto tile = [&](int kt, f16x8 (&cur)[T::kFrags], f16x8 (&nxt)[T::kFrags]) {
        unsigned int read_a = frag_lane + slot_bytes(2 * kt + 2), read_b = frag_lane + slot_bytes(2 * kt + 3);  // tile kt + 1
        asm volatile("" : "+v"(read_a), "+v"(read_b));  // (these two sums, not one per fragment)
        const unsigned int load_b = slot_bytes(2 * kt + 5), load_a = slot_bytes(2 * kt + 6);  // = the slots of tile kt
        const int kt_b = clamped(kt + 2), kt_a = clamped(kt + 3);
        // tile kt + 1 has landed (behind its B part: the A part of tile kt + 2) and this wavefront's reads of tile kt's
        // slots (issued during the previous phase) have returned; then everyone's
        detail::lds_barrier<8>();
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int n = 0; n < kNT; ++n) {
                const int j = snake(i, n);
                const int r = (kNT / 2) * i + (n >> 1);
                if ((n & 1) == 0 && r < T::kFrags) nxt[order(r)] = read_frag(read_a, read_b, order(r));
                const int s = 2 * i + (n >> 2);  // load slot of the phase: B of tile kt + 2 first, then A of tile kt + 3
                if ((n & 3) == 1 && s < kNumLoads) {
                    const int q = s < T::kLoadsB ? 8 + s : s - T::kLoadsB;
                    detail::mfma_16x16x32_agpr_then_load(acc[i][j], cur[8 + j], cur[i], voff[q],
                                                         load_src(q < 8 ? kt_a : kt_b, q), load_dst(q < 8 ? load_a : load_b, q));
                } else {
                    detail::mfma_16x16x32_agpr(acc[i][j], cur[8 + j], cur[i]);
                }
            }
        }
    };
    {
        int kt = 0;
        for (; kt + 1 < ktiles; kt += 2) {
            tile(kt, fx, fy);
            tile(kt + 1, fy, fx);
        }
        if (kt < ktiles) tile(kt, fx, fy);
    }

    detail::mfma_results_wait();
#pragma unroll
    for (int i = 0; i < 8; ++i) pin_row(acc[i]);

    // ---- the four partial tiles are added through LDS, two row groups (32 rows, 2 kNT MFMA tiles) per round. Every
    // wavefront writes its partial tiles of the round - tile t = kNT (row group % 2) + column tile, 1 KiB each, a
    // lane's f32x4 at 16 * lane: conflict-free and the same for writer and reader - and then sums the four partials
    // of tiles (kNT / 2) w .. + kNT / 2 - 1 into registers of its own. Which tiles a wavefront sums is a matter of LDS
    // addresses only: register indices are the same in all four wavefronts (an index that depended on the wavefront would
    // put the accumulators into scratch memory). Two buffers of 64 KiB alternate, so one barrier per round is enough: a
    // buffer is written again two rounds later, after the barrier of the round in between.
    // Wavefront w ends up with rows 32 r + 16 (w / 2) .. + 15 (r = 0 .. 3), column tiles (kNT / 2) (w % 2) .. + kNT / 2 - 1.
    detail::lds_barrier<0>();  // nothing is on its way into LDS any more, every wavefront is done with the operand stages
    using lds_f32x4_ptr = __attribute__((address_space(3))) f32x4*;
    constexpr int kPerRound = 2 * kNT, kMine = kNT / 2;
    f32x4 res[4][kMine];
#pragma unroll
    for (int round = 0; round < 4; ++round) {
        const unsigned int buf = lds_base + (round & 1) * (64 * 1024) + lane * 16;
#pragma unroll
        for (int t = 0; t < kPerRound; ++t)
            *reinterpret_cast<lds_f32x4_ptr>(buf + (wave * kPerRound + t) * 1024) = acc[2 * round + t / kNT][t % kNT];
        __syncthreads();
#pragma unroll
        for (int jj = 0; jj < kMine; ++jj) {
            f32x4 sum = *reinterpret_cast<lds_f32x4_ptr>(buf + (kMine * wave + jj) * 1024);
#pragma unroll
            for (int w = 1; w < 4; ++w) {
                const f32x4 v = *reinterpret_cast<lds_f32x4_ptr>(buf + (w * kPerRound + kMine * wave + jj) * 1024);
#pragma unroll
                for (int e = 0; e < 4; ++e) sum[e] += v[e];
            }
            res[round][jj] = sum;
        }
    }

    // ---- store: res[r][jj][e] = C[32 r + 16 (w / 2) + lane % 16][16 (kMine (w % 2) + jj) + 4 (lane / 16) + e] of the tile.
    // f16: the 16 rows of a round pass through 2 KiB of LDS of this wavefront's own (beyond the two reduction buffers; the
    // 8-byte slots of a row XOR-ed with twice the row) and leave as whole rows of 16 kMine elements through non-temporal
    // stores, 16 bytes per lane: 8-byte pieces of lines would have to be gathered by the L2, and lines left dirty there
    // are written back after the kernel's last wavefront.
    if constexpr (sizeof(OutType) == 2) {
        constexpr int kPitch = 16 * kMine * 2;                     // bytes per staged row: 128 (96)
        constexpr int kSlots = kPitch / 8;                         // 8-byte slots per row: 16 (12)
        constexpr int kChunks = kPitch / 16;                       // 16-byte pieces per row: 8 (6)
        constexpr int kPieces = 16 * kChunks;                      // per round: 128 (96)
        const unsigned int stg = lds_base + 128 * 1024 + wave * 2048;
        using lds_f16x4_ptr = __attribute__((address_space(3))) f16x4*;
        using lds_u32x4_ptr = __attribute__((address_space(3))) const u32x4*;
        // slot s of row q lies at slot s ^ (2 q % 16) where that stays inside the row (kSlots = 16), else unpermuted
        auto slot_of = [](int q, int s) { return kSlots == 16 ? s ^ ((2 * q) & 15) : s; };
        OutType* cblock = C + size_t(m0 + 16 * (wave >> 1)) * ldc + n0 + 16 * kMine * (wave & 1);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
            for (int jj = 0; jj < kMine; ++jj) {
                f16x4 h;
#pragma unroll
                for (int e = 0; e < 4; ++e) h[e] = static_cast<_Float16>(res[r][jj][e]);
                *reinterpret_cast<lds_f16x4_ptr>(stg + frow * kPitch + slot_of(frow, 4 * jj + fquad) * 8) = h;
            }
            // LDS operations of one wavefront execute in order: the reads see the writes above
#pragma unroll
            for (int it = 0; it < (kPieces + kWaveSize - 1) / kWaveSize; ++it) {
                const int piece = it * kWaveSize + lane;
                const int q = piece / kChunks, c = piece % kChunks;
                if (kPieces % kWaveSize != 0 && piece >= kPieces) continue;
                const u32x4 v = *reinterpret_cast<lds_u32x4_ptr>(stg + q * kPitch + slot_of(q, 2 * c) * 8);
                if constexpr (kEdges) {
                    // M and N are multiples of 16: a 16-byte piece lies inside the matrix or outside it as a whole
                    if (m0 + 32 * r + 16 * (wave >> 1) + q >= M || n0 + 16 * kMine * (wave & 1) + 8 * c >= N) continue;
                }
                __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(cblock + size_t(32 * r + q) * ldc + 8 * c));
            }
        }
    } else {
        // f32 (also the partial products of a split-K launch): the same with 16-byte slots, 4 KiB per wavefront
        constexpr int kPitch = 16 * kMine * 4;                     // bytes per staged row: 256 (192)
        constexpr int kChunks = kPitch / 16;                       // 16-byte pieces per row: 16 (12)
        constexpr int kPieces = 16 * kChunks;                      // per round: 256 (192)
        const unsigned int stg = lds_base + 128 * 1024 + wave * 4096;
        using lds_u32x4_ptr = __attribute__((address_space(3))) const u32x4*;
        auto slot_of = [](int q, int s) { return kChunks == 16 ? s ^ q : s; };
        OutType* cblock = C + size_t(m0 + 16 * (wave >> 1)) * ldc + n0 + 16 * kMine * (wave & 1);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
            for (int jj = 0; jj < kMine; ++jj)
                *reinterpret_cast<lds_f32x4_ptr>(stg + frow * kPitch + slot_of(frow, 4 * jj + fquad) * 16) = res[r][jj];
#pragma unroll
            for (int it = 0; it < kPieces / kWaveSize; ++it) {
                const int piece = it * kWaveSize + lane;
                const int q = piece / kChunks, c = piece % kChunks;
                const u32x4 v = *reinterpret_cast<lds_u32x4_ptr>(stg + q * kPitch + slot_of(q, c) * 16);
                if constexpr (kEdges) {
                    if (m0 + 32 * r + 16 * (wave >> 1) + q >= M || n0 + 16 * kMine * (wave & 1) + 4 * c >= N) continue;
                }
                __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(cblock + size_t(32 * r + q) * ldc + 4 * c));
            }
        }
    }
}

}  // namespace tiledcuda::kernels
