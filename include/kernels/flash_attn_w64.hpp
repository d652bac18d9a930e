// FlashAttention-2 forward for gfx950 with one wavefront per SIMD: O = softmax(scale · Q·Kᵀ)·V, f16 in/out, f32
// accumulation and statistics. Same contract and layouts as kernels/flash_attn_fwd.hpp (Q [M, D], K [N, D], V [N, D],
// O [M, D] row-major per batch item; the tuned counterpart of the reference's src/kernels/flash_attn.cu:134-312).
// What changes is how the work is mapped to the CU:
//   * a workgroup is 4 wavefronts, one per SIMD, each owning 64 query rows (two 32-query column tiles of Sᵀ / Oᵀ):
//     every K fragment and every Vᵀ fragment read from LDS feeds two MFMAs, which halves the LDS traffic per MFMA
//     against 32 queries per wavefront (there the LDS read rate, not the matrix pipe, was the limit);
//   * all matrix instructions are inline assembly. The 128 f32 accumulators of Oᵀ and the Q fragments live in
//     AGPRs, the score tiles and the probabilities in VGPRs; the instruction order is the one written here.
//     The compiler does not know these statements are MFMAs and inserts none of the wait states MFMA results need
//     before other instructions read them; the schedule below keeps every such read at least two MFMAs behind
//     the write, and the rare paths wait explicitly;
//   * the key sequence is processed in halves of 32 keys, software-pipelined inside the one instruction stream:
//     step i issues the 16 MFMAs of Sᵀ(i+1) = K·Qᵀ and the 16 MFMAs of Oᵀ += Vᵀ(i-1)·Pᵀ(i-1), interleaved
//     with the VALU work of the softmax of half i (per MFMA: one v_exp_f32, half a conversion, half a dot2), so
//     the matrix pipe and the vector ALU are both busy all the time and neither waits for the other;
//   * softmax without a running maximum in the common path: the score accumulators start at -m (m = reference
//     maximum of the query, handed to the first MFMA of a tile as its C operand), p = exp2(acc) is converted to
//     f16 and summed from the f16 values (v_dot2_f32_f16, so numerator and denominator see the same rounding);
//     only the sum of a half is checked: while it stays below 2^14 no probability can exceed 2^14, far inside f16
//     range, and a stale reference maximum is harmless (the final division cancels it). If the check fails (a score
//     more than 14 above its reference in the log2 domain), the maxima are moved, Oᵀ and the sums are rescaled, the
//     scores already computed for the next half are re-biased and the probabilities are recomputed;
//   * K/V blocks of 64 keys go global -> LDS directly into a ring of four stages, requested two blocks ahead, one
//     LDS-only barrier per block; swizzles and the transposing V reads are those of flash_attn_fwd.hpp.
// kVColMajor: V is stored column-major [N, D], i.e. as the array Vᵀ [D, N] (the convention of the reference's op,
// src/kernels/flash_attn.cu:424-456 with pytiledcuda/__init__.py:17-30). A row of Vᵀ then holds consecutive keys, and
// the A operand of Oᵀ += Vᵀ Pᵀ could be a plain ds_read_b128 if a lane needed 8 consecutive keys - which the
// accumulator of Sᵀ does not give (a lane half holds keys 4 h .. + 3 of every group of 8). So the keys are re-ordered
// where it is free: row i of a 32-key score tile is fed with key 16 ((i / 4) % 2) + 4 (i / 8) + i % 4 (just another
// row address for the K fragment read), which puts the 16 consecutive keys 16 h .. 16 h + 15 of the tile into lane
// half h, 8 consecutive ones per MFMA k-step: one ds_read_b128 per Vᵀ fragment, no transposing read. The swizzle of
// the K rows is chosen for that read order.
// M % 64 == 0 and N % 64 == 0 are required (checked by the host launcher); wavefronts of the last workgroup whose
// 64 queries lie beyond M take part in the loads and barriers and discard their result.
#pragma once

#include <type_traits>
#include <utility>

#include "config.hpp"
#include "hip_utils.hpp"
#include "kernels/flash_attn_fwd.hpp"  // FlashFwdTraits swizzles, detail::exchange32, detail::exp2_raw
#include "kernels/gemm_w128.hpp"       // detail::load_lds_16B_sbase, detail::lds_barrier

namespace tiledcuda::kernels {

template <const int kD_>
struct FlashW64Traits {
    static constexpr int kD = kD_, kWaves = 4, kBN = 64;
    static constexpr int kBM = 64 * kWaves;
    static constexpr int kThreads = kWaves * kWaveSize;
    static constexpr int kStages = 5;
    using Swz = FlashFwdTraits<kD, 8, kBN>;               // row size and swizzle functions
    static constexpr int kRowBytes = 2 * kD;
    static constexpr int kTileBytes = kBN * kRowBytes;    // one K or V block
    static constexpr int kHalfBytes = 32 * kRowBytes;     // 32 keys of it
    static constexpr int kStageBytes = 2 * kTileBytes;    // K + V
    static constexpr int kRowsPerLoad = 1024 / kRowBytes;
    static constexpr int kLoadsPerTile = kBN / kRowsPerLoad;
    static constexpr int kLoadsPerWave = 2 * kLoadsPerTile / kWaves;  // per block: K and V
    static constexpr int kDSteps = kD / 16;  // k-steps of Sᵀ = K Qᵀ
    static constexpr int kDTiles = kD / 32;  // 32-row tiles of Oᵀ
    static constexpr int kFragAhead = 3;     // d-steps between the request of a K / V fragment and its MFMAs
    static_assert(kD == 128, "the step schedule below is written for head size 128");
    static_assert(kLoadsPerWave == 8 && kDSteps == 8 && kDTiles == 4);
    static constexpr int kLdsBytes = kStages * kStageBytes;  // 160 KiB; the epilogue reuses 64 KiB of it
    static_assert(kLdsBytes <= kMaxLdsBytes);
};

namespace detail {

using f16x2 = _Float16 __attribute__((ext_vector_type(2)));

/// d = a · b + c, all of d and c in VGPRs, b in AGPRs (first MFMA of a score tile: c carries -m).
DEVICE void mfma32_score_first(f32x16& d, const f16x8& a, const f16x8& b, const f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "a"(b), "v"(c));
}
/// d += a · b, d in VGPRs, b in AGPRs.
DEVICE void mfma32_score(f32x16& d, const f16x8& a, const f16x8& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
}
/// d += a · b, d in AGPRs.
DEVICE void mfma32_out(f32x16& d, const f16x8& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(d) : "v"(a), "v"(b));
}
/// The same MFMA, then a direct-to-LDS load of 16 bytes per lane from sbase + voff to lds_addr + 16 * lane: m0 is written
/// before the MFMA, which thereby is the wait state required between the write of m0 and the load (no s_nop).
DEVICE void mfma32_out_then_load(f32x16& d, const f16x8& a, const u32x4& b, unsigned int voff, const void* sbase,
                                 unsigned int lds_addr) {
    asm volatile(
        "s_mov_b32 m0, %5\n\t"
        "v_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\t"
        "global_load_lds_dwordx4 %3, %4"
        : "+a"(d)
        : "v"(a), "v"(b), "v"(voff), "s"(sbase), "s"(lds_addr)
        : "m0", "memory");
}
/// LDS fragment reads issued as inline assembly, so that the waits are the kernel's own: the compiler's waits for LDS
/// reads it knows about are exact only inside a basic block; for fragments requested in one step of the pipeline
/// and consumed in the next (across loop back edges and the branch of the rare path) it falls back to waiting for
/// every read in flight, including the ones just issued for the following d-step. LDS reads return in order, so
/// lds_wait<N>() (at most N reads outstanding) before the MFMAs of a d-step waits for exactly that d-step's fragments.
DEVICE f16x8 lds_read_b128_untracked(unsigned int addr) {
    f16x8 r;
    asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(addr));
    return r;
}
/// Two transposing 8-byte reads (addr + kOff0, addr + kOff1) forming one 16-byte MFMA operand.
template <int kOff0, int kOff1>
DEVICE f16x8 lds_read_tr_pair_untracked(unsigned int addr) {
    f16x4 lo, hi;
    asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                 : "=&v"(lo), "=&v"(hi)
                 : "v"(addr), "n"(kOff0), "n"(kOff1));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
template <int kOutstanding>
DEVICE void lds_wait() {
    __builtin_amdgcn_s_waitcnt(0xC07F | (kOutstanding << 8));  // lgkmcnt(kOutstanding), nothing else
}

/// Two f32 -> one register of two f16 (round to nearest even), issued where it is written: left to the compiler, the
/// conversions of a whole step sink to their first use and run as one block that no MFMA hides. The sources may be
/// results of v_exp_f32: at least one other instruction must have been issued since (the callers' MFMAs are).
DEVICE unsigned int cvt_pk_f16_here(float a, float b) {
    unsigned int r;
    asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
DEVICE unsigned int pack_f16x2(float a, float b) {
    const f16x2 pk = {static_cast<_Float16>(a), static_cast<_Float16>(b)};
    return __builtin_bit_cast(unsigned int, pk);
}

/// Wait long enough for every MFMA issued so far to have written its result (32 wait states cover the longest
/// requirement) before `x` is touched by anything else.
/// After detail::mfma_results_wait(): the accumulator is read only behind that wait.
DEVICE void mfma_settle_v(f32x16& x) { asm volatile("" : "+v"(x)); }
DEVICE void mfma_settle_a(f32x16& x) { asm volatile("" : "+a"(x)); }

}  // namespace detail

/// grid = (M / 256) * batch workgroups (1-D), block = 256, dynamic LDS = Traits::kLdsBytes.
/// Workgroup ids congruent modulo 8 land on the same XCD: when the batch count is a multiple of 8 the query blocks
/// of one (batch, head) item all get such ids, so its K and V are fetched from HBM once.
template <typename Traits, bool kVColMajor = false>
__global__ void __launch_bounds__(Traits::kThreads)
    flash_attention_fwd_w64(const __half* __restrict__ Q, const __half* __restrict__ K, const __half* __restrict__ V,
                            __half* __restrict__ O, int batch, int M, int N, float scale) {
    using Swz = typename Traits::Swz;
    constexpr int kD = Traits::kD, kBN = Traits::kBN;
    constexpr int kRowBytes = Traits::kRowBytes;
    constexpr int kChunks = kRowBytes / 16;
    constexpr int kStages = Traits::kStages;
    constexpr int kL = Traits::kLoadsPerWave;
    extern __shared__ __align__(1024) unsigned char lds[];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int q32 = lane & 31;  // query (column of Sᵀ / Oᵀ) of this lane within a 32-query tile
    const int h = lane >> 5;    // lane half

    const int q_blocks = (M + Traits::kBM - 1) / Traits::kBM;
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
    const int m0 = q_block * Traits::kBM + wave * 64;
    const bool active = m0 < M;  // wave-uniform: this wavefront's 64 queries exist
    const __half* Qh = Q + (head * M + (active ? m0 : 0)) * kD;
    const __half* Kh = K + head * size_t(N) * kD;
    const __half* Vh = V + head * size_t(N) * kD;
    __half* Oh = O + (head * M + (active ? m0 : 0)) * kD;

    // Key order inside a 32-key half (see the header): score-tile row i holds key key_of_row(i); identity for a
    // row-major V. k_swizzle: XOR applied to the 16-byte chunk index of K row `row` of a block, chosen so that the 16
    // rows read by one pass of a fragment read (rows key_of_row(0..15) or (16..31)) get 16 different values.
    auto key_of_row = [](int i) { return kVColMajor ? 16 * ((i >> 2) & 1) + 4 * (i >> 3) + (i & 3) : i; };
    auto k_swizzle = [](int row) {
        return kVColMajor ? (((row >> 2) & 1) << 3) | (((row >> 4) & 1) << 2) | (row & 3) : Swz::k_swz(row);
    };
    const int nb = N / kBN;

    const unsigned int lds_base = static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds));

    // ---- global -> LDS: load instruction j of this wavefront for a block (j < kL / 2: K, else V) fills
    // kRowsPerLoad rows; the instructions of a block are dealt round-robin to the wavefronts
    const int lrow = lane / kChunks, lchk = lane % kChunks;
    unsigned int goff[kL];     // byte offset of this lane's 16 bytes inside the K (or V) block
    unsigned int ldst[kL];     // LDS byte offset of the instruction's 1 KiB inside a stage
#pragma unroll
    for (int j = 0; j < kL; ++j) {
        const bool is_v = j >= kL / 2;
        const int t = wave + Traits::kWaves * (is_v ? j - kL / 2 : j);  // 1 KiB slot of the tile
        const int row = t * Traits::kRowsPerLoad + lrow;
        if (is_v && kVColMajor) {
            // the V block is kD rows (d) of 64 keys = 128 bytes: 8 rows per instruction, chunks XOR-ed with (d / 2) % 8
            const int d = t * 8 + (lane >> 3);
            const int chunk8 = (lane & 7) ^ ((d >> 1) & 7);
            goff[j] = static_cast<unsigned int>(d * N + chunk8 * 8) * 2u;
        } else {
            const int chunk = is_v ? (lchk ^ (Swz::v_swz(row) << 1)) : (lchk ^ k_swizzle(row));
            goff[j] = static_cast<unsigned int>(row * kD + chunk * 8) * 2u;
        }
        ldst[j] = (is_v ? Traits::kTileBytes : 0) + t * 1024;
    }
    // stage_off: byte offset of the block's ring stage, (block % kStages) * kStageBytes (the loop keeps the offsets it
    // needs as running values: a remainder by 5 is a dozen scalar instructions, and every instruction of a lone wavefront
    // takes an issue slot)
    auto issue_load_at = [&](unsigned int stage_off, int block, int j) {
        const bool is_v = j >= kL / 2;
        const __half* src = (is_v && kVColMajor) ? Vh + size_t(block) * kBN : (is_v ? Vh : Kh) + size_t(block) * kBN * kD;
        const unsigned int dst = __builtin_amdgcn_readfirstlane(lds_base + stage_off + ldst[j]);
        detail::load_lds_16B_sbase(goff[j], src, dst);
    };
    auto issue_load = [&](int block, int j) { issue_load_at((block % kStages) * Traits::kStageBytes, block, j); };

    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using Yes = std::true_type;
    using No = std::false_type;

    // ---- LDS -> registers. Addresses are 32-bit LDS offsets: a per-lane part computed once (below) plus the
    // wave-uniform offset of the half being read (a scalar), so a fragment read costs one address addition.
    using lds_f16x8_ptr = const f16x8 __attribute__((address_space(3)))*;
    using fp16x4 = __fp16 __attribute__((ext_vector_type(4)));
    using lds_fp16x4_ptr = fp16x4 __attribute__((address_space(3)))*;
    // K fragment (A operand of Sᵀ = K Qᵀ) for d-step s: lane (row = lane % 32, h) holds K[row][16 s + 8 h .. + 7]
    // (of the key this lane's score-tile row stands for)
    unsigned int koff[Traits::kDSteps];
    const int krow = key_of_row(q32);
#pragma unroll
    for (int s = 0; s < Traits::kDSteps; ++s) {
        const int chunk = (2 * s + h) ^ k_swizzle(krow);  // the swizzle depends on row % 32 only
        koff[s] = lds_base + krow * kRowBytes + chunk * 16;
        asm volatile("" : "+v"(koff[s]));  // keep the eight offsets in registers (not rematerialised per use)
    }
    auto read_k = [&](unsigned int k_half_off, int s) -> f16x8 {
        return *reinterpret_cast<lds_f16x8_ptr>(koff[s] + k_half_off);
    };
    // the same read of the staged Q rows (row = lane % 32 of a 32-query tile, swizzled like a K block of a row-major V)
    auto read_q_staged = [&](unsigned int q_half_off, int s) -> f16x8 {
        const int chunk = (2 * s + h) ^ Swz::k_swz(q32);
        return *reinterpret_cast<lds_f16x8_ptr>(lds_base + q32 * kRowBytes + chunk * 16 + q_half_off);
    };
    // Vᵀ fragment (A operand of Oᵀ += Vᵀ Pᵀ) for d tile dt and k-step s2 of key half t of a block: lane
    // (d = 32 dt + lane % 32, h).
    // Row-major V: slot e = key 16 s2 + 8 (e / 4) + 4 h + e % 4 of the half, fetched with two transposing reads; within
    // a 16-lane group, lane L supplies the address of row kv0 + L / 4, columns dbase + 4 (L % 4) .. + 3.
    // Column-major V: slot e = key 16 h + 8 s2 + e of the half (the keys this lane half holds after the re-ordering),
    // 16 contiguous bytes of row d of the Vᵀ block: chunk 4 t + 2 h + s2, XOR-ed with (d / 2) % 8.
    const int g = lane >> 4, L16 = lane & 15;
    const int vrow_in = L16 >> 2;
    const int vcol_b = (16 * (g & 1) + 4 * (L16 & 3)) * 2;
    unsigned int voff[Traits::kDTiles];  // row-major V: per d tile; column-major V: per (t, s2)
#pragma unroll
    for (int dt = 0; dt < Traits::kDTiles; ++dt) {
        if (kVColMajor) {
            const int chunk = (4 * (dt >> 1) + 2 * h + (dt & 1)) ^ ((q32 >> 1) & 7);
            voff[dt] = lds_base + q32 * 128 + chunk * 16;
        } else {
            const int byte_in_row = 64 * dt + vcol_b;
            const int unit = (byte_in_row >> 5) ^ Swz::v_swz(vrow_in);  // every row read by this lane has row % 4 == vrow_in
            voff[dt] = lds_base + (4 * h + vrow_in) * kRowBytes + unit * 32 + (byte_in_row & 31);
        }
        asm volatile("" : "+v"(voff[dt]));
    }
    auto read_k_untracked = [&](unsigned int k_half_off, int s) -> f16x8 {
        return detail::lds_read_b128_untracked(koff[s] + k_half_off);
    };
    // v_blk_off: LDS offset of the V tile of the block; t_c, s2_c: key half of the block and k-step of the half
    auto read_v_untracked = [&](unsigned int v_blk_off, auto t_c, auto s2_c, int dt) -> f16x8 {
        constexpr int t = decltype(t_c)::value, s2 = decltype(s2_c)::value;
        if constexpr (kVColMajor) {
            return detail::lds_read_b128_untracked(voff[2 * t + s2] + v_blk_off + dt * (32 * 128));
        } else {
            constexpr int kRow0 = 32 * t + 16 * s2;
            return detail::lds_read_tr_pair_untracked<kRow0 * kRowBytes, (kRow0 + 8) * kRowBytes>(voff[dt] + v_blk_off);
        }
    };
    // LDS offset (relative to the ring) of the K rows of half `half_i` of the key sequence; V is kTileBytes further
    auto k_half = [&](int half_i) -> unsigned int {
        return ((half_i >> 1) % kStages) * Traits::kStageBytes + (half_i & 1) * Traits::kHalfBytes;
    };
    // LDS offset of the V tile of the block that half `half_i` belongs to
    auto v_block = [&](int half_i) -> unsigned int {
        return ((half_i >> 1) % kStages) * Traits::kStageBytes + Traits::kTileBytes;
    };

    // ---- prologue: Q and the first K/V blocks are requested together (so that the cold latencies overlap).
    // Q fragments (B operand of Sᵀ = K Qᵀ): lane (q, h) of column tile c holds Q[32 c + q][16 s + 8 h .. + 7].
    // Read straight from global memory that is 32 bytes from each of 32 rows per instruction; for sequences long
    // enough to matter the wavefront instead stages its 64 contiguous rows (16 KiB) through LDS like a K block
    // (coalesced 1 KiB loads, same swizzle, same fragment reads), in the two ring stages (3 and 4) that the K/V
    // blocks reach last; those two blocks are then requested in the first block-iteration.
    const bool q_via_lds = nb >= kStages;
    f16x8 qraw[2][Traits::kDSteps];
    if (q_via_lds) {
        const unsigned int q_stage = 3 * Traits::kStageBytes + wave * (64 * kRowBytes);
        if (active) {
#pragma unroll
            for (int t = 0; t < 64 / Traits::kRowsPerLoad; ++t) {
                const int row = t * Traits::kRowsPerLoad + lrow;
                const unsigned int off = static_cast<unsigned int>(row * kD + (lchk ^ Swz::k_swz(row)) * 8) * 2u;
                detail::load_lds_16B_sbase(off, Qh, __builtin_amdgcn_readfirstlane(lds_base + q_stage + t * 1024));
            }
        }
#pragma unroll
        for (int j = 0; j < kL; ++j) {
            issue_load(0, j);
        }
        // Only Q and block 0 are requested before the first scores: all workgroups of a round start together, and
        // what they request at once arrives at the rate of the memory system (three more blocks per workgroup
        // would be 20 MB more, and issuing a load blocks while the queues are full); blocks 1 and 2 are requested
        // under the first two score computations below, blocks 3 and 4 in the first block-iteration.
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_s_barrier();

#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int s = 0; s < Traits::kDSteps; ++s) qraw[c][s] = read_q_staged(q_stage + c * Traits::kHalfBytes, s);
    } else {
#pragma unroll
        for (int b = 0; b < kStages - 1; ++b)
            if (b < nb) {
#pragma unroll
                for (int j = 0; j < kL; ++j) issue_load(b, j);
            }
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int s = 0; s < Traits::kDSteps; ++s)
                qraw[c][s] = *reinterpret_cast<const f16x8*>(Qh + size_t(32 * c + q32) * kD + 16 * s + 8 * h);
    }
    if (!active) {
        // nothing of this wavefront's result is kept: feed zeros (what was read above is some other rows' data or,
        // for the staged path, whatever the stage held)
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int s = 0; s < Traits::kDSteps; ++s) qraw[c][s] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
    // pre-multiplied by scale * log2(e): the scores come out of the MFMA in the log2 domain
    const float cscale = scale * 1.4426950408889634f;
    f16x8 qf[2][Traits::kDSteps];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int s = 0; s < Traits::kDSteps; ++s) {
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[c][s][e] = static_cast<_Float16>(static_cast<float>(qraw[c][s][e]) * cscale);
        }
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int s = 0; s < Traits::kDSteps; ++s) asm volatile("" : "+a"(qf[c][s]));

    f32x16 o_acc[Traits::kDTiles][2];  // Oᵀ tiles (d tile, query tile), AGPRs
#pragma unroll
    for (int dt = 0; dt < Traits::kDTiles; ++dt)
#pragma unroll
        for (int c = 0; c < 2; ++c) {
#pragma unroll
            for (int e = 0; e < 16; ++e) o_acc[dt][c][e] = 0.f;
            asm volatile("" : "+a"(o_acc[dt][c]));
        }

    f32x16 s_acc[2][2];   // score tiles: [buffer][query tile], relative to the reference maximum
    u32x4 pf[2][2][2];    // probabilities as B operands, two f16 per element: [buffer][query tile][k-step of the half]
    f32x16 negm[2];       // -m of this lane's query of tile c, in all 16 slots (C operand of a tile's first MFMA)
    float m_run[2], l_run[2];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int e = 0; e < 16; ++e) negm[c][e] = 0.f;

    if (!q_via_lds) detail::lds_barrier<0>();  // everything requested so far has landed, for everyone


    // scores of half `half_i` into buffer `buf` (MFMAs only; used before the pipeline is running)
    auto qk_only = [&](int half_i, auto buf_c, int load_block) {
        constexpr int buf = decltype(buf_c)::value;
        const unsigned int sk = k_half(half_i);
        f16x8 kf[2];
        kf[0] = read_k(sk, 0);
#pragma unroll
        for (int s = 0; s < Traits::kDSteps; ++s) {
            if (s + 1 < Traits::kDSteps) kf[(s + 1) & 1] = read_k(sk, s + 1);
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                if (s == 0) detail::mfma32_score_first(s_acc[buf][c], kf[s & 1], qf[c][s], negm[c]);
                else detail::mfma32_score(s_acc[buf][c], kf[s & 1], qf[c][s]);
            }
            if (load_block > 0 && load_block < nb) issue_load(load_block, s);
        }
    };

    // ---- half 0: exact maximum
    qk_only(0, std::integral_constant<int, 0>{}, q_via_lds ? 1 : 0);
    detail::mfma_results_wait();
    detail::mfma_settle_v(s_acc[0][0]);
    detail::mfma_settle_v(s_acc[0][1]);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        float mx = s_acc[0][c][0];
#pragma unroll
        for (int e = 1; e < 16; ++e) mx = fmaxf(mx, s_acc[0][c][e]);
        mx = fmaxf(mx, detail::exchange32(mx));
        m_run[c] = mx;
        float lsum = 0.f;
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
            const float p0 = detail::exp2_raw(s_acc[0][c][e] - mx);
            const float p1 = detail::exp2_raw(s_acc[0][c][e + 1] - mx);
            pf[0][c][e / 8][(e % 8) / 2] = detail::pack_f16x2(p0, p1);
            lsum += p0 + p1;
        }
        l_run[c] = lsum;
#pragma unroll
        for (int e = 0; e < 16; ++e) negm[c][e] = -mx;
    }
    qk_only(1, std::integral_constant<int, 1>{}, q_via_lds ? 2 : 0);

    // ---- one pipelined step: softmax of half i (buffer kCur), scores of half i + 1 (if kQk) into the other
    // buffer, output update with half i - 1 (probabilities of the other buffer). kLoads: this wavefront also issues
    // its loads of block `load_block`, one per d-step. Fragments are requested kAhead d-steps before the MFMAs that
    // use them, across the boundaries between steps (with one wavefront per SIMD nothing else covers the LDS
    // latency): the last d-steps of a step request the first fragments of the next one (K of half i + 2 if
    // kNextQk, V of half i).
    constexpr int kAhead = Traits::kFragAhead, kRing = kAhead + 1;
    // LDS read instructions per d-step: the V fragment is two transposing reads or one ds_read_b128; plus the K one
    constexpr int kReadsV = kVColMajor ? 1 : 2, kReadsQk = kReadsV + 1;
    static_assert(8 % kRing == 0 && kAhead <= 3, "ring positions must repeat from one step to the next; the prefetch stays within the first k-step of the next half");
    f16x8 kf[kRing], vf[kRing];
    // Step i = 2 J + 1 (kCur = 1) or 2 J + 2 (kCur = 0) touches blocks J, J + 1, J + 2: `ring` holds their stage offsets
    // and that of the block being loaded.
    struct RingOffsets {
        unsigned int a, b, c, load;
    };
    const __half *warm_a = Kh, *warm_b = Kh;  // two 16 KiB runs that a step with warm-up loads fetches
    auto step = [&](const RingOffsets& ring, auto cur_c, auto qk_c, auto loads_c, auto next_qk_c, int load_block) {
        constexpr int kCur = decltype(cur_c)::value, kNxt = kCur ^ 1;
        constexpr bool kQk = decltype(qk_c)::value;
        constexpr int kLoads = decltype(loads_c)::value;  // 0: none, 1: block `load_block` of K and V, 2 / 3: warm-up loads
        constexpr bool kNextQk = decltype(next_qk_c)::value;
        // K of half i + 1 (block J + 1; its first half for odd i), V of half i - 1 (block J), K of half i + 2, V of half i
        const unsigned int sk = ring.b + (kCur == 1 ? 0 : Traits::kHalfBytes);
        const unsigned int sv = ring.a + Traits::kTileBytes;  // key half kNxt of that block
        const unsigned int sk_next = kCur == 1 ? ring.b + Traits::kHalfBytes : ring.c;
        const unsigned int sv_next = (kCur == 1 ? ring.a : ring.b) + Traits::kTileBytes;  // key half kCur of that block
        float lh[2] = {0.f, 0.f}, lg[2] = {0.f, 0.f};  // two partial sums per query tile (independent add chains)
        // VALU work of the same wavefront hides under its MFMAs only in small doses: one v_exp_f32 plus one or two
        // plain instructions directly behind each MFMA cost 2-3 cycles per MFMA, the same instructions in groups of
        // four or more cost their full issue time. So a d-step is four slots of one MFMA and its share of the
        // softmax (the pair of query tile 1 is converted and summed one d-step later), fenced from each other.
        float x0 = 0.f, x1 = 0.f, y0 = 0.f, y1 = 0.f;
        auto pack_pair = [&](auto c_c, auto d_c, float a0, float a1) {
            // probabilities of slots 2 d, 2 d + 1 of query tile c: to f16, into the B operand
            constexpr int c = decltype(c_c)::value, d = decltype(d_c)::value;
            pf[kCur][c][d >> 2][d & 3] = detail::cvt_pk_f16_here(a0, a1);
        };
        auto ex = [&](float v) { return detail::exp2_raw(v); };
        detail::static_for<8>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value;
            constexpr int sp = s + kAhead;
            if constexpr (sp < 8) {
                if (kQk) kf[sp % kRing] = read_k_untracked(sk, sp);
                if (sp < 4) vf[sp % kRing] = read_v_untracked(sv, std::integral_constant<int, kNxt>{}, C0{}, sp & 3);
                else vf[sp % kRing] = read_v_untracked(sv, std::integral_constant<int, kNxt>{}, C1{}, sp & 3);
                detail::lds_wait<kAhead * (kQk ? kReadsQk : kReadsV)>();
            } else {
                if (kNextQk) kf[sp % kRing] = read_k_untracked(sk_next, sp - 8);
                vf[sp % kRing] = read_v_untracked(sv_next, std::integral_constant<int, kCur>{}, C0{}, (sp - 8) & 3);
                // in flight after this wait: the fragments of the d-steps still ahead in this step (kReadsQk or kReadsV reads
                // each) and those just requested for the next step
                detail::lds_wait<(7 - s) * (kQk ? kReadsQk : kReadsV) + (sp - 7) * (kNextQk ? kReadsQk : kReadsV)>();
            }
            // slot A
            if (kQk) {
                if (s == 0) detail::mfma32_score_first(s_acc[kNxt][0], kf[s % kRing], qf[0][s], negm[0]);
                else detail::mfma32_score(s_acc[kNxt][0], kf[s % kRing], qf[0][s]);
            }
            x0 = ex(s_acc[kCur][0][2 * s]);
            if constexpr (s > 0) pack_pair(C1{}, std::integral_constant<int, s - 1>{}, y0, y1);
            __builtin_amdgcn_sched_barrier(0);
            // slot B
            if (kQk) {
                if (s == 0) detail::mfma32_score_first(s_acc[kNxt][1], kf[s % kRing], qf[1][s], negm[1]);
                else detail::mfma32_score(s_acc[kNxt][1], kf[s % kRing], qf[1][s]);
            }
            x1 = ex(s_acc[kCur][0][2 * s + 1]);
            if constexpr (s == 1) {  // the first pair starts the sums (no addition to zero: every instruction is a slot)
                lh[1] = y0;
                lg[1] = y1;
            } else if constexpr (s > 1) {
                lh[1] += y0;
                lg[1] += y1;
            }
            __builtin_amdgcn_sched_barrier(0);
            // slot C (with this wavefront's load s of the block being fetched riding on the MFMA)
            if constexpr (kLoads == 1) {
                const bool is_v = s >= kL / 2;
                const __half* src = (is_v && kVColMajor) ? Vh + size_t(load_block) * kBN
                                                         : (is_v ? Vh : Kh) + size_t(load_block) * kBN * kD;
                const unsigned int dst = __builtin_amdgcn_readfirstlane(lds_base + ring.load + ldst[s]);
                detail::mfma32_out_then_load(o_acc[s & 3][0], vf[s % kRing], pf[kNxt][0][s >> 2], goff[s], src, dst);
            } else if constexpr (kLoads == 2) {
                // 1 KiB of the 16 KiB run at warm_a (s < 4) or warm_b; the four wavefronts cover both runs
                const __half* src = (s < kL / 2 ? warm_a : warm_b) + (wave * (kL / 2) + (s & 3)) * 512;
                const unsigned int dst = __builtin_amdgcn_readfirstlane(lds_base + ring.load + ldst[s]);
                detail::mfma32_out_then_load(o_acc[s & 3][0], vf[s % kRing], pf[kNxt][0][s >> 2], lane * 16u, src, dst);
            } else if constexpr (kLoads == 3) {
                // as 2, but warm_b is the first block of a column-major V (128 pieces of 128 bytes, N elements apart):
                // fetched with the offsets of the ring loads of a V block
                const bool is_v = s >= kL / 2;
                const __half* src = is_v ? warm_b : warm_a + (wave * (kL / 2) + (s & 3)) * 512;
                const unsigned int dst = __builtin_amdgcn_readfirstlane(lds_base + ring.load + ldst[s]);
                detail::mfma32_out_then_load(o_acc[s & 3][0], vf[s % kRing], pf[kNxt][0][s >> 2],
                                             is_v ? goff[s] : lane * 16u, src, dst);
            } else {
                detail::mfma32_out(o_acc[s & 3][0], vf[s % kRing], pf[kNxt][0][s >> 2]);
            }
            y0 = ex(s_acc[kCur][1][2 * s]);
            pack_pair(C0{}, s_c, x0, x1);
            __builtin_amdgcn_sched_barrier(0);
            // slot D
            detail::mfma32_out(o_acc[s & 3][1], vf[s % kRing], pf[kNxt][1][s >> 2]);
            y1 = ex(s_acc[kCur][1][2 * s + 1]);
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
        // the check: no probability of this half can have left f16 range while its sum stays below 2^14
        constexpr float kLimit = 16384.f;
        if (__any(!(fmaxf(lh[0], lh[1]) <= kLimit))) {
            // rare path: move the reference maxima, rescale, re-bias, recompute
            detail::mfma_results_wait();
            if (kQk) {
                detail::mfma_settle_v(s_acc[kNxt][0]);
                detail::mfma_settle_v(s_acc[kNxt][1]);
            }
#pragma unroll
            for (int dt = 0; dt < Traits::kDTiles; ++dt)
#pragma unroll
                for (int c = 0; c < 2; ++c) detail::mfma_settle_a(o_acc[dt][c]);
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                float mx = s_acc[kCur][c][0];
#pragma unroll
                for (int e = 1; e < 16; ++e) mx = fmaxf(mx, s_acc[kCur][c][e]);
                mx = fmaxf(mx, detail::exchange32(mx));
                const float shift = mx > 8.0f ? mx : 0.f;  // queries whose scores stayed near their reference keep it
                const float alpha = detail::exp2_raw(-shift);
                m_run[c] += shift;
                l_run[c] *= alpha;
#pragma unroll
                for (int dt = 0; dt < Traits::kDTiles; ++dt)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o_acc[dt][c][e] *= alpha;
                if (kQk) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) s_acc[kNxt][c][e] -= shift;
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) negm[c][e] = -m_run[c];
                float lsum = 0.f;
#pragma unroll
                for (int e = 0; e < 16; e += 2) {
                    const float p0 = detail::exp2_raw(s_acc[kCur][c][e] - shift);
                    const float p1 = detail::exp2_raw(s_acc[kCur][c][e + 1] - shift);
                    pf[kCur][c][e / 8][(e % 8) / 2] = detail::pack_f16x2(p0, p1);
                    lsum += p0 + p1;
                }
                lh[c] = lsum;
            }
#pragma unroll
            for (int dt = 0; dt < Traits::kDTiles; ++dt)
#pragma unroll
                for (int c = 0; c < 2; ++c) asm volatile("" : "+a"(o_acc[dt][c]));
        }
        l_run[0] += lh[0];
        l_run[1] += lh[1];
        __builtin_amdgcn_sched_barrier(0);
    };

    // Hand-over of a stage: this wavefront's loads up to and including block J + 2 have landed (kPending newer
    // ones may stay in flight), then everyone's; and everyone has left block J - 1, whose stage block J + 4 goes to.
    // LDS reads in flight are fragment requests for the next d-steps and belong to younger stages: no lgkmcnt wait.
    auto hand_over = [&](auto pending_c) {
        constexpr int kPending = decltype(pending_c)::value;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070 | 0x0f00 | (kPending & 0xF) | ((kPending >> 4) << 14));  // vmcnt only
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    // first fragments of step 1: K of half 2 (block 1), V of half 0. With Q staged through LDS, block 1 was requested
    // only under the scores of half 0 and every wavefront fetched a quarter of it: the reads then go behind the first
    // hand-over (before it, another wavefront's quarter may still be on its way - seen as rare wrong rows when the
    // block missed the L2).
    auto first_fragments = [&]() {
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
            if (nb > 1) kf[a] = read_k_untracked(k_half(2), a);
            vf[a] = read_v_untracked(v_block(0), C0{}, C0{}, a & 3);
        }
    };
    if (!q_via_lds) first_fragments();
    // ---- block-iterations: J covers halves 2 J + 1 (odd) and 2 J + 2 (even)
    constexpr unsigned int kStageB = Traits::kStageBytes, kRingB = kStages * Traits::kStageBytes;
    auto next_stage = [&](unsigned int off) { return off + kStageB == kRingB ? 0u : off + kStageB; };
    int J = 0;
    RingOffsets ring{0u, kStageB, 2 * kStageB, 4 * kStageB};  // blocks 0, 1, 2; block J + 4 is loaded
    auto advance = [&]() {
        ring.a = ring.b;
        ring.b = ring.c;
        ring.c = next_stage(ring.c);
        ring.load = next_stage(ring.load);
        ++J;
    };
    if (q_via_lds) {
        // J = 0: blocks 3 and 4 go to the stages the Q tiles were staged in (everyone has read its Q by now)
        hand_over(std::integral_constant<int, 0>{});
        first_fragments();
        RingOffsets first = ring;
        first.load = 3 * kStageB;
        step(first, C1{}, Yes{}, Yes{}, Yes{}, 3);
        step(ring, C0{}, Yes{}, Yes{}, Yes{}, 4);
        advance();
    }
    for (; J + 4 < nb; advance()) {
        hand_over(std::integral_constant<int, kL>{});
        step(ring, C1{}, Yes{}, Yes{}, Yes{}, J + 4);
        step(ring, C0{}, Yes{}, No{}, Yes{}, 0);
    }
    // The workgroup that follows this one on the XCD (256 workgroups are resident, ids congruent mod 8 share an XCD:
    // id + 256) starts with a cold burst: its 256 query rows and the first block of its item's K and V. With no ring
    // loads left to issue, three of the last steps fetch those 96 KiB instead, into the ring stage that was vacated
    // last (the data is discarded: the point is that the lines are in this XCD's L2 when the next workgroup asks).
    {
        const unsigned int nid = blockIdx.x + 256;
        if (q_via_lds && nid < gridDim.x && J + 4 == nb) {  // two more block-iterations follow
            int nhead, nqb;
            if (batch % 8 == 0) {
                const int xcd = nid & 7, rest = nid >> 3;
                nqb = rest % q_blocks;
                nhead = (rest / q_blocks) * 8 + xcd;
            } else {
                nqb = nid % q_blocks;
                nhead = nid / q_blocks;
            }
            const int rows0 = nqb * Traits::kBM;
            // 64 query rows from row r of that workgroup's block (M % 64 == 0; rows beyond M: the last 64 instead)
            auto qrows = [&](int r) { return Q + (size_t(nhead) * M + (rows0 + r < M ? rows0 + r : M - 64)) * kD; };
            using Warm = std::integral_constant<int, 2>;
            hand_over(std::integral_constant<int, 0>{});
            warm_a = qrows(0), warm_b = qrows(64);
            step(ring, C1{}, Yes{}, Warm{}, Yes{}, 0);
            warm_a = qrows(128), warm_b = qrows(192);
            step(ring, C0{}, Yes{}, Warm{}, Yes{}, 0);
            advance();
            hand_over(std::integral_constant<int, 0>{});
            // K block 0 is 16 KiB of consecutive rows; so is a row-major V block (a column-major one is 128 pieces of
            // 128 bytes, which the offsets of the ring loads describe)
            warm_a = K + size_t(nhead) * N * kD;
            warm_b = V + size_t(nhead) * N * kD;
            step(ring, C1{}, Yes{}, std::integral_constant<int, kVColMajor ? 3 : 2>{}, Yes{}, 0);
            step(ring, C0{}, Yes{}, No{}, Yes{}, 0);
            advance();
        }
    }
    for (; J + 2 < nb; advance()) {
        hand_over(std::integral_constant<int, 0>{});
        step(ring, C1{}, Yes{}, No{}, Yes{}, 0);
        step(ring, C0{}, Yes{}, No{}, Yes{}, 0);
    }
    if (J + 1 < nb) {
        step(ring, C1{}, Yes{}, No{}, Yes{}, 0);
        step(ring, C0{}, Yes{}, No{}, No{}, 0);
        advance();
    }
    step(ring, C1{}, No{}, No{}, No{}, 0);
    {
        // the output update with the last half (its first fragments were requested by the step before)
        const unsigned int sv = v_block(2 * J + 1);
        detail::static_for<8>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value;
            constexpr int sp = s + kAhead;
            if constexpr (sp < 8) {
                if (sp < 4) vf[sp % kRing] = read_v_untracked(sv, C1{}, C0{}, sp & 3);
                else vf[sp % kRing] = read_v_untracked(sv, C1{}, C1{}, sp & 3);
                detail::lds_wait<kAhead * kReadsV>();
            } else {
                detail::lds_wait<(7 - s) * kReadsV>();
            }
#pragma unroll
            for (int c = 0; c < 2; ++c) detail::mfma32_out(o_acc[s & 3][c], vf[s % kRing], pf[1][c][s >> 2]);
        });
    }

    // ---- epilogue: O[q, d] = Oᵀ[d, q] / l. o_acc[dt][c][r]: d = 32 dt + 8 (r / 4) + 4 h + r % 4, q = 32 c + q32.
    detail::mfma_results_wait();
#pragma unroll
    for (int dt = 0; dt < Traits::kDTiles; ++dt)
#pragma unroll
        for (int c = 0; c < 2; ++c) detail::mfma_settle_a(o_acc[dt][c]);
    __builtin_amdgcn_s_waitcnt(0x0070 | 0x0f00);  // vmcnt(0): nothing of this wavefront is still on its way into LDS
    __syncthreads();  // all wavefronts are done with the K/V stages: reuse LDS for staging
    unsigned char* stg = lds + wave * (64 * kRowBytes);
    constexpr int kSlotMask = (kRowBytes / 8 - 1) & ~1;  // 8-byte slots of a staged row are XOR-ed with 2 * (row % 16)
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const float l_tot = l_run[c] + detail::exchange32(l_run[c]);
        const float inv_l = 1.0f / l_tot;
        const int row = 32 * c + q32;
#pragma unroll
        for (int dt = 0; dt < Traits::kDTiles; ++dt) {
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                f16x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = static_cast<_Float16>(o_acc[dt][c][4 * qd + e] * inv_l);
                const int slot = (32 * dt + 8 * qd + 4 * h) >> 2;
                const int pslot = slot ^ (((row & 15) << 1) & kSlotMask);
                *reinterpret_cast<f16x4*>(stg + row * kRowBytes + pslot * 8) = v;
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // this wavefront's staging writes are done (it reads only its own rows)
    constexpr int kLanesPerRow = kRowBytes / 16;
    constexpr int kRowsPerIter = kWaveSize / kLanesPerRow;
    const int rr = lane / kLanesPerRow, cc = lane % kLanesPerRow;
#pragma unroll
    for (int it = 0; it < 64 / kRowsPerIter; ++it) {
        const int row = it * kRowsPerIter + rr;
        const int pslot = (2 * cc) ^ (((row & 15) << 1) & kSlotMask);
        const u32x4 v = *reinterpret_cast<const u32x4*>(stg + row * kRowBytes + pslot * 8);
        if (active) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(Oh + size_t(row) * kD) + cc * 16));  // whole rows, streamed
    }
}

}  // namespace tiledcuda::kernels
