// FlashAttention-2 forward for gfx950, O = softmax(scale · Q·Kᵀ)·V, f16 in/out, f32 statistics.
// The tuned counterpart of kernels/flash_attn.hpp (which composes the generic 16x16 tile
// primitives, as the reference's src/kernels/flash_attn.cu:134-312 does). Layouts: Q [M, D],
// K [N, D], V [N, D], O [M, D] row-major per batch item (the usual [seq, head_dim]).
//
// Design (per workgroup: kWaves wavefronts x 32 query rows; K/V streamed in blocks of kBN keys):
//   * Sᵀ = K·Qᵀ with v_mfma_f32_32x32x16_f16: the accumulator of a 32x32 tile then gives every
//     lane 16 keys of ONE query (column = lane % 32), so the online-softmax row maximum and
//     row sum are in-lane reductions plus one exchange with lane ^ 32, and the rescale factor
//     is a per-lane scalar;
//   * Oᵀ = Vᵀ·Pᵀ: exp(Sᵀ - m) converted to f16 is directly the B operand (the contraction
//     index of an MFMA may be permuted freely as long as both operands agree: slot e of k-step
//     s of lane half h is key 16 s + 8 (e / 4) + 4 h + e % 4); Vᵀ comes from the row-major V
//     tile in LDS through the transposing read ds_read_b64_tr_b16, two per operand;
//   * Q stays in registers for the whole kernel (it is read from HBM once, where the
//     reference re-reads it for every key block, flash_attn.cu:241);
//   * K and V blocks go global -> LDS directly (16 B per lane, no register staging) into a ring of
//     three stages; one barrier per block; the loads are issued through inline assembly
//     (detail::load_lds_16B_untracked): with the builtin the compiler waits for the block just requested
//     (s_waitcnt vmcnt(0)) before the next LDS read, because it cannot prove that the read does not alias
//     the stage being filled, and the ring degenerates to one block at a time;
//   * the two wavefronts that share a SIMD run an iteration in different orders (scores of block j+1
//     first / last), so one of them feeds the matrix pipe while the other does the softmax VALU work;
//   * LDS rows are 2 * kD bytes. K: the 16-byte chunks of a row are XOR-ed with the row index
//     (ds_read_b128 of 16 consecutive rows at one chunk hits all 64 banks once). V: the
//     32-byte units of a row are XOR-ed with a function of the row so that the 4 rows x 32 B
//     read by each 16-lane group of a transposing read, and the two groups of a half-wave,
//     fall on distinct banks. Both permutations are applied on the global-address side;
//   * softmax runs in the log2 domain with as few VALU operations per score as possible: Q is
//     multiplied by scale * log2(e) once, when it is loaded; the accumulators of Sᵀ start at -m (the
//     running maximum of that query) instead of 0, so p = exp2(acc) with no subtraction; the maximum
//     is only moved when a block exceeds it by more than 2^8 ("lazy rescaling": a stale maximum is
//     harmless, p <= 2^8 stays far inside f16 / f32 range and the final division cancels it), which
//     makes the rescale of the output accumulators a rare, wave-uniform branch.
// M % (32 * kWaves) == 0 and N % kBN == 0 are required (checked by the host launcher).
#pragma once

#include "config.hpp"
#include "hip_utils.hpp"
#include "kernels/gemm_pipelined.hpp"  // detail::load_lds_16B

namespace tiledcuda::kernels {

template <const int kD_, const int kWaves_, const int kBN_ = 64>
struct FlashFwdTraits {
    static constexpr int kD = kD_, kWaves = kWaves_, kBN = kBN_;
    static constexpr int kBM = 32 * kWaves;
    static constexpr int kThreads = kWaves * kWaveSize;
    static constexpr int kStages = 3;
    static constexpr int kRowBytes = 2 * kD;             // 256 for D = 128
    static constexpr int kTileBytes = kBN * kRowBytes;   // one K or V block
    static constexpr int kStageBytes = 2 * kTileBytes;   // K + V
    static constexpr int kRowsPerLoad = 1024 / kRowBytes;
    static constexpr int kLoadsPerTile = kBN / kRowsPerLoad;  // 1 KiB instructions per K (or V) block
    static constexpr int kDSteps = kD / 16;   // k-steps of Sᵀ = K Qᵀ
    static constexpr int kDTiles = kD / 32;   // 32-row tiles of Oᵀ
    static constexpr int kKvTiles = kBN / 32; // 32-row tiles of Sᵀ
    static constexpr int kKvSteps = kBN / 16; // k-steps of Oᵀ = Vᵀ Pᵀ
    static_assert(kD == 128 || kD == 64, "head size 64 or 128");
    static_assert(kBN % 32 == 0);
    static constexpr int kLdsMain = kStages * kStageBytes;
    static constexpr int kLdsBytes = kLdsMain > kBM * kRowBytes ? kLdsMain : kBM * kRowBytes;

    /// XOR applied to the 16-byte chunk index of K row `row`.
    HOST_DEVICE static constexpr int k_swz(int row) { return row & (kRowBytes / 16 - 1) & 15; }
    /// XOR applied to the 32-byte unit index of V row `row`: rows 4 a .. 4 a + 3 at one unit, and the two
    /// 16-lane groups of a half-wave (adjacent units), must fall on 8 distinct 32-byte bank slots.
    /// 256-byte rows all start on bank 0: spread the 4 rows over units with 2 * (row % 4).
    /// 128-byte rows alternate between the two halves of the banks: only rows 2 apart collide: row & 2.
    HOST_DEVICE static constexpr int v_swz(int row) { return kRowBytes == 256 ? ((row & 3) << 1) : (row & 2); }
};

namespace detail {
DEVICE float exchange32(float v) { return __shfl_xor(v, 32, 64); }
/// 2^x as one v_exp_f32 (no range fix-ups: arguments here are <= 8 and results below 2^-126 may flush to 0).
DEVICE float exp2_raw(float x) { return __builtin_amdgcn_exp2f(x); }
}  // namespace detail

/// grid = (M / kBM) * batch workgroups (1-D), block = Traits::kThreads, dynamic LDS = Traits::kLdsBytes.
/// Workgroup ids that are congruent modulo 8 land on the same XCD (and share its L2): when the batch
/// count is a multiple of 8 the query blocks of one (batch, head) item all get such ids, so its K and V
/// are fetched from HBM once instead of once per XCD.
template <typename Traits>
__global__ void __launch_bounds__(Traits::kThreads)
    flash_attention_fwd(const __half* __restrict__ Q, const __half* __restrict__ K, const __half* __restrict__ V,
                        __half* __restrict__ O, int batch, int M, int N, float scale) {
    constexpr int kD = Traits::kD, kBN = Traits::kBN, kWaves = Traits::kWaves;
    constexpr int kRowBytes = Traits::kRowBytes;
    constexpr int kChunks = kRowBytes / 16;  // 16-byte chunks per row
    constexpr int kStages = Traits::kStages;
    extern __shared__ __align__(1024) unsigned char lds[];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int q32 = lane & 31;  // query (column of Sᵀ / Oᵀ) owned by this lane
    const int h = lane >> 5;    // lane half

    const int q_blocks = M / Traits::kBM;
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
    const int m0 = q_block * Traits::kBM + wave * 32;
    const __half* Qh = Q + (head * M + m0) * kD;
    const __half* Kh = K + head * size_t(N) * kD;
    const __half* Vh = V + head * size_t(N) * kD;
    __half* Oh = O + (head * M + m0) * kD;

    // ---- Q fragments: B operand of Sᵀ = K Qᵀ: lane (q, h) holds Q[q][16 s + 8 h .. + 7] for k-step s,
    // pre-multiplied by scale * log2(e) so that the scores come out of the MFMA in the log2 domain.
    // (filled after the first K/V blocks have been requested, so that the two cold latencies overlap)
    const float c = scale * 1.4426950408889634f;
    f16x8 qf[Traits::kDSteps];
    auto load_q = [&]() {
#pragma unroll
        for (int s = 0; s < Traits::kDSteps; ++s) {
            const f16x8 raw = *reinterpret_cast<const f16x8*>(Qh + size_t(q32) * kD + 16 * s + 8 * h);
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[s][e] = static_cast<_Float16>(static_cast<float>(raw[e]) * c);
        }
    };

    // ---- global -> LDS for a K/V block. One instruction fills kRowsPerLoad rows.
    // The 2 * kLoadsPerTile instructions of a block (K first, then V) are dealt round-robin to the wavefronts.
    constexpr int kLoadsPerBlock = 2 * Traits::kLoadsPerTile;
    constexpr int kLoadsPerWave = (kLoadsPerBlock + kWaves - 1) / kWaves;
    const int lrow = lane / kChunks;  // row within the instruction's rows
    const int lchk = lane % kChunks;  // physical 16-byte chunk
    auto issue_block = [&](int stage, int n0) {
        unsigned char* sk = lds + stage * Traits::kStageBytes;
#pragma unroll
        for (int j = 0; j < kLoadsPerWave; ++j) {
            const int idx = wave + j * kWaves;  // wave-uniform
            if (kLoadsPerBlock % kWaves == 0 || idx < kLoadsPerBlock) {
                const bool is_v = idx >= Traits::kLoadsPerTile;
                const int t = is_v ? idx - Traits::kLoadsPerTile : idx;
                const int row = t * Traits::kRowsPerLoad + lrow;
                // physical chunk lchk holds logical chunk lchk ^ swizzle(row)
                const int chunk = is_v ? (lchk ^ (Traits::v_swz(row) << 1)) : (lchk ^ Traits::k_swz(row));
                const __half* src = (is_v ? Vh : Kh) + size_t(n0 + row) * kD + chunk * 8;
                detail::load_lds_16B_untracked(src, sk + (is_v ? Traits::kTileBytes : 0) + t * 1024);
            }
        }
    };

    // ---- Sᵀ[kv, q] - m_init = K[kv, :] · (c Q[q, :]) - m_init: accumulators start at -m_init
    auto qk_block = [&](int stage, float m_init, f32x16 (&s_acc)[Traits::kKvTiles]) {
        const unsigned char* sk = lds + stage * Traits::kStageBytes;
#pragma unroll
        for (int t = 0; t < Traits::kKvTiles; ++t) {
#pragma unroll
            for (int e = 0; e < 16; ++e) s_acc[t][e] = -m_init;
            const int row = t * 32 + q32;  // key row read by this lane (A operand: row = lane % 32)
#pragma unroll
            for (int s = 0; s < Traits::kDSteps; ++s) {
                const int chunk = (2 * s + h) ^ Traits::k_swz(row);
                const f16x8 kf = *reinterpret_cast<const f16x8*>(sk + row * kRowBytes + chunk * 16);
                s_acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[s], s_acc[t], 0, 0, 0);
            }
        }
    };

    // ---- accumulators and statistics (log2 domain)
    f32x16 o_acc[Traits::kDTiles];
#pragma unroll
    for (int t = 0; t < Traits::kDTiles; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[t][e] = 0.f;
    float m_run = -INFINITY;  // reference maximum of this lane's query (same in lanes l and l ^ 32)
    float l_run = 0.f;        // this lane's share of the running sum

    const int nblocks = N / kBN;
    issue_block(0, 0);
    if (nblocks > 1) issue_block(1, kBN);
    load_q();  // requested after the K/V blocks: by the time Q has arrived and is converted, so have they
    __builtin_amdgcn_s_waitcnt(0x0070);
    __syncthreads();

    f32x16 s_cur[Traits::kKvTiles], s_nxt[Traits::kKvTiles];
    float m_init_cur = 0.f, m_init_nxt = 0.f;  // what the accumulators of s_cur / s_nxt were started at (negated)
    qk_block(0, m_init_cur, s_cur);

    constexpr float kLazy = 8.0f;
    const int g = lane >> 4, L = lane & 15;
    const int vrow_in = L >> 2;                            // 0..3: row within the 4-key group
    const int vcol_b = (16 * (g & 1) + 4 * (L & 3)) * 2;  // byte offset of the lane's 4 columns inside a 32-d tile

    // block maximum of s (relative to its m_init) for the query of this lane
    auto block_max = [&](const f32x16 (&s_acc)[Traits::kKvTiles]) -> float {
        float mx = s_acc[0][0];
#pragma unroll
        for (int t = 0; t < Traits::kKvTiles; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s_acc[t][e]);
        return fmaxf(mx, detail::exchange32(mx));
    };
    // Is the general path needed for a block whose accumulators started at m_init and whose maximum is mx?
    // Yes if the reference maximum must move (lazy rescaling) or if it moved after the accumulators were started.
    auto needs_general = [&](float m_init, float mx) -> bool {
        return __any((m_init + mx - m_run > kLazy) || (m_init != m_run));
    };

    float mx_cur = block_max(s_cur);
    bool general_cur = true;  // first block: m_run = -inf

    // The wavefronts of a workgroup run the three pieces of an iteration in two different orders, so that
    // the two wavefronts sharing a SIMD are out of phase: while one does softmax (VALU, transcendental),
    // the other feeds the matrix pipe.
    //   wavefronts 0-3: scores of block j+1 (MFMA), softmax of block j (VALU), output update with block j (MFMA)
    //   wavefronts 4-7: softmax of block j, output update with block j, scores of block j+1
    // (the wavefronts of a workgroup are dealt to the 4 SIMDs round-robin: w and w + 4 share one).
    const bool scores_first = ((wave >> 2) & 1) == 0;

    int stage = 0;
    for (int j = 0; j < nblocks; ++j) {
        const int stage_nxt = stage + 1 == kStages ? 0 : stage + 1;
        const bool has_next = j + 1 < nblocks;
        if (has_next) {
            __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0): my share of block j+1 (issued one iteration ago) landed
            __syncthreads();                      // everyone's share landed; everyone is done with block j-1
            if (j + 2 < nblocks) issue_block(stage_nxt + 1 == kStages ? 0 : stage_nxt + 1, (j + 2) * kBN);
        }

        if (has_next && scores_first) {
            m_init_nxt = (m_run == -INFINITY) ? 0.f : m_run;
            qk_block(stage_nxt, m_init_nxt, s_nxt);
        }

        // ---- probabilities of block j. This lane holds keys 32 t + 8 (r / 4) + 4 h + r % 4; s_cur = score - m_init_cur.
        float psum = 0.f;
        f16x8 pf[Traits::kKvSteps];
        if (general_cur) {
            // move the reference maximum if needed, rescale the output, exponentiate with the correction
            const float m_blk = m_init_cur + mx_cur;
            const bool upd = m_blk - m_run > kLazy;
            const float m_new = upd ? m_blk : m_run;
            const float alpha = detail::exp2_raw(m_run - m_new);  // exp2(-inf) = 0, exp2(0) = 1
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < Traits::kDTiles; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) o_acc[t][e] *= alpha;
            m_run = m_new;
            const float delta = m_init_cur - m_run;
#pragma unroll
            for (int t = 0; t < Traits::kKvTiles; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float p = detail::exp2_raw(s_cur[t][e] + delta);
                    psum += p;
                    pf[2 * t + e / 8][e % 8] = static_cast<_Float16>(p);
                }
        } else {
            // common case: m_init_cur == m_run and the maximum stays: p = exp2(s_cur)
#pragma unroll
            for (int t = 0; t < Traits::kKvTiles; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float p = detail::exp2_raw(s_cur[t][e]);
                    psum += p;
                    pf[2 * t + e / 8][e % 8] = static_cast<_Float16>(p);
                }
        }
        l_run += psum;

        // ---- Oᵀ[d, q] += Vᵀ[d, kv] · Pᵀ[kv, q]
        // A operand for (d tile dt, k-step s): lane (d = 32 dt + lane % 32, h), slot e = key 16 s + 8 (e / 4) + 4 h + e % 4,
        // fetched with two transposing reads (4 consecutive keys of one d each). Within a 16-lane group, lane L
        // supplies the address of row kv0 + L / 4, columns dbase + 4 (L % 4) .. + 3.
        const unsigned char* sv = lds + stage * Traits::kStageBytes + Traits::kTileBytes;
#pragma unroll
        for (int dt = 0; dt < Traits::kDTiles; ++dt) {
#pragma unroll
            for (int s = 0; s < Traits::kKvSteps; ++s) {
                f16x8 vf;
#pragma unroll
                for (int part = 0; part < 2; ++part) {
                    const int row = 16 * s + 8 * part + 4 * h + vrow_in;
                    const int byte_in_row = 64 * dt + vcol_b;  // multiple of 8
                    const int unit = (byte_in_row >> 5) ^ Traits::v_swz(row);
                    const unsigned char* p = sv + row * kRowBytes + unit * 32 + (byte_in_row & 31);
                    using fp16x4 = __fp16 __attribute__((ext_vector_type(4)));
                    const fp16x4 v4 = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
                        (fp16x4 __attribute__((address_space(3)))*)(p));
#pragma unroll
                    for (int e = 0; e < 4; ++e) vf[4 * part + e] = static_cast<_Float16>(v4[e]);
                }
                o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[s], o_acc[dt], 0, 0, 0);
            }
        }

        if (has_next) {
            if (scores_first) {
#pragma unroll
                for (int t = 0; t < Traits::kKvTiles; ++t) s_cur[t] = s_nxt[t];
                m_init_cur = m_init_nxt;
            } else {
                m_init_cur = m_run;  // m_run is finite here: at least one block has been processed
                qk_block(stage_nxt, m_init_cur, s_cur);
            }
            mx_cur = block_max(s_cur);
            general_cur = needs_general(m_init_cur, mx_cur);
        }
        stage = stage_nxt;
    }

    // ---- epilogue: O[q, d] = Oᵀ[d, q] / l. acc[dt][r]: d = 32 dt + 8 (r / 4) + 4 h + r % 4, q = q32.
    const float l_tot = l_run + detail::exchange32(l_run);
    const float inv_l = 1.0f / l_tot;
    __syncthreads();  // all wavefronts are done with the K/V stages: reuse LDS for staging
    unsigned char* stg = lds + wave * (32 * kRowBytes);
    // 8-byte slots of a staged row (4 consecutive d) are XOR-ed with 2 * (row % 16) within the row
    constexpr int kSlotMask = (kRowBytes / 8 - 1) & ~1;
#pragma unroll
    for (int dt = 0; dt < Traits::kDTiles; ++dt) {
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            f16x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = static_cast<_Float16>(o_acc[dt][4 * qd + e] * inv_l);
            const int slot = (32 * dt + 8 * qd + 4 * h) >> 2;
            const int pslot = slot ^ (((q32 & 15) << 1) & kSlotMask);
            *reinterpret_cast<f16x4*>(stg + q32 * kRowBytes + pslot * 8) = v;
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    constexpr int kLanesPerRow = kRowBytes / 16;
    constexpr int kRowsPerIter = kWaveSize / kLanesPerRow;
    const int rr = lane / kLanesPerRow, cc = lane % kLanesPerRow;
#pragma unroll
    for (int it = 0; it < 32 / kRowsPerIter; ++it) {
        const int row = it * kRowsPerIter + rr;
        const int pslot = (2 * cc) ^ (((row & 15) << 1) & kSlotMask);
        const u32x4 v = *reinterpret_cast<const u32x4*>(stg + row * kRowBytes + pslot * 8);
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(Oh + size_t(row) * kD) + cc * 16));  // whole rows, streamed
    }
}

/// Variant of flash_attention_fwd that overlaps the softmax with the matrix work inside one wavefront.
/// Iteration j computes the scores of block j+1 (accumulators started at -m_run), then runs the MFMAs of
/// Oᵀ += V_jᵀ P_jᵀ fused with the exp2 / sum / convert of block j+1 *speculating that no running maximum has to
/// move*: the VALU and transcendental instructions issue under the MFMAs of the same wavefront (measured: two
/// v_exp_f32 or six plain VALU operations hide under one 32x32x16 MFMA of the same wavefront, while VALU work of
/// the *other* wavefront of the SIMD overlaps poorly). The speculation is checked afterwards (any score of the
/// block more than 2^8 above its query's reference maximum?); if it fails, the maxima are moved, the output is
/// rescaled and the probabilities are recomputed from the scores, which are still in registers. Results are
/// the same as flash_attention_fwd's up to rounding. On inputs whose row maxima keep growing along the key
/// sequence the redo path runs often and this kernel is up to ~10 % slower than flash_attention_fwd; on inputs
/// whose maxima settle within the first blocks it is 5-8 % faster.
/// Same launch contract as flash_attention_fwd.
template <typename Traits>
__global__ void __launch_bounds__(Traits::kThreads)
    flash_attention_fwd_fused(const __half* __restrict__ Q, const __half* __restrict__ K, const __half* __restrict__ V,
                              __half* __restrict__ O, int batch, int M, int N, float scale) {
    constexpr int kD = Traits::kD, kBN = Traits::kBN, kWaves = Traits::kWaves;
    constexpr int kRowBytes = Traits::kRowBytes;
    constexpr int kChunks = kRowBytes / 16;
    constexpr int kStages = Traits::kStages;
    extern __shared__ __align__(1024) unsigned char lds[];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int q32 = lane & 31;  // query (column of Sᵀ / Oᵀ) owned by this lane
    const int h = lane >> 5;    // lane half

    const int q_blocks = M / Traits::kBM;
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
    const int m0 = q_block * Traits::kBM + wave * 32;
    const __half* Qh = Q + (head * M + m0) * kD;
    const __half* Kh = K + head * size_t(N) * kD;
    const __half* Vh = V + head * size_t(N) * kD;
    __half* Oh = O + (head * M + m0) * kD;

    // Q fragments, pre-multiplied by scale * log2(e)
    // (filled after the first K/V blocks have been requested, so that the two cold latencies overlap)
    const float c = scale * 1.4426950408889634f;
    f16x8 qf[Traits::kDSteps];
    auto load_q = [&]() {
#pragma unroll
        for (int s = 0; s < Traits::kDSteps; ++s) {
            const f16x8 raw = *reinterpret_cast<const f16x8*>(Qh + size_t(q32) * kD + 16 * s + 8 * h);
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[s][e] = static_cast<_Float16>(static_cast<float>(raw[e]) * c);
        }
    };

    // global -> LDS for a K/V block (same dealing and swizzles as flash_attention_fwd)
    constexpr int kLoadsPerBlock = 2 * Traits::kLoadsPerTile;
    constexpr int kLoadsPerWave = (kLoadsPerBlock + kWaves - 1) / kWaves;
    const int lrow = lane / kChunks;
    const int lchk = lane % kChunks;
    auto issue_block = [&](int stage, int n0) {
        unsigned char* sk = lds + stage * Traits::kStageBytes;
#pragma unroll
        for (int j = 0; j < kLoadsPerWave; ++j) {
            const int idx = wave + j * kWaves;  // wave-uniform
            if (kLoadsPerBlock % kWaves == 0 || idx < kLoadsPerBlock) {
                const bool is_v = idx >= Traits::kLoadsPerTile;
                const int t = is_v ? idx - Traits::kLoadsPerTile : idx;
                const int row = t * Traits::kRowsPerLoad + lrow;
                const int chunk = is_v ? (lchk ^ (Traits::v_swz(row) << 1)) : (lchk ^ Traits::k_swz(row));
                const __half* src = (is_v ? Vh : Kh) + size_t(n0 + row) * kD + chunk * 8;
                detail::load_lds_16B_untracked(src, sk + (is_v ? Traits::kTileBytes : 0) + t * 1024);
            }
        }
    };

    // Sᵀ[kv, q] - m_init: accumulators start at -m_init
    auto qk_block = [&](int stage, float m_init, f32x16 (&s_acc)[Traits::kKvTiles]) {
        const unsigned char* sk = lds + stage * Traits::kStageBytes;
#pragma unroll
        for (int t = 0; t < Traits::kKvTiles; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) s_acc[t][e] = -m_init;
#pragma unroll
        for (int s = 0; s < Traits::kDSteps; ++s)
#pragma unroll
            for (int t = 0; t < Traits::kKvTiles; ++t) {
                const int row = t * 32 + q32;
                const int chunk = (2 * s + h) ^ Traits::k_swz(row);
                const f16x8 kf = *reinterpret_cast<const f16x8*>(sk + row * kRowBytes + chunk * 16);
                s_acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[s], s_acc[t], 0, 0, 0);
            }
    };

    f32x16 o_acc[Traits::kDTiles];
#pragma unroll
    for (int t = 0; t < Traits::kDTiles; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[t][e] = 0.f;
    float m_run;        // reference maximum of this lane's query (same in lanes l and l ^ 32)
    float l_run = 0.f;  // this lane's share of the running sum

    const int nblocks = N / kBN;
    issue_block(0, 0);
    if (nblocks > 1) issue_block(1, kBN);
    load_q();  // requested after the K/V blocks: by the time Q has arrived and is converted, so have they
    __builtin_amdgcn_s_waitcnt(0x0070);
    __syncthreads();

    constexpr float kLazy = 8.0f;
    const int g = lane >> 4, L = lane & 15;
    const int vrow_in = L >> 2;
    const int vcol_b = (16 * (g & 1) + 4 * (L & 3)) * 2;

    auto block_max = [&](const f32x16 (&s_acc)[Traits::kKvTiles]) -> float {
        float mx = s_acc[0][0];
#pragma unroll
        for (int t = 0; t < Traits::kKvTiles; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s_acc[t][e]);
        return fmaxf(mx, detail::exchange32(mx));
    };

    // probabilities of block j as f16 B operands of Oᵀ += Vᵀ Pᵀ, carried between iterations
    f16x8 pf[Traits::kKvSteps];
    f32x16 s_nxt[Traits::kKvTiles];
    {
        // block 0: exact
        qk_block(0, 0.f, s_nxt);
        m_run = block_max(s_nxt);
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < Traits::kKvTiles; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float p = detail::exp2_raw(s_nxt[t][e] - m_run);
                psum += p;
                pf[2 * t + e / 8][e % 8] = static_cast<_Float16>(p);
            }
        l_run = psum;
    }

    auto pv_mfma = [&](const unsigned char* sv, int dt, int s2) {
        f16x8 vf;
#pragma unroll
        for (int part = 0; part < 2; ++part) {
            const int row = 16 * s2 + 8 * part + 4 * h + vrow_in;
            const int byte_in_row = 64 * dt + vcol_b;
            const int unit = (byte_in_row >> 5) ^ Traits::v_swz(row);
            const unsigned char* p = sv + row * kRowBytes + unit * 32 + (byte_in_row & 31);
            using fp16x4 = __fp16 __attribute__((ext_vector_type(4)));
            const fp16x4 v4 = __builtin_amdgcn_ds_read_tr16_b64_v4f16((fp16x4 __attribute__((address_space(3)))*)(p));
#pragma unroll
            for (int e = 0; e < 4; ++e) vf[4 * part + e] = static_cast<_Float16>(v4[e]);
        }
        o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[s2], o_acc[dt], 0, 0, 0);
    };

    int stage = 0;
    for (int j = 0; j + 1 < nblocks; ++j) {
        const int stage_nxt = stage + 1 == kStages ? 0 : stage + 1;
        __builtin_amdgcn_s_waitcnt(0x0070);  // block j+1 has landed (this wavefront's share)
        __syncthreads();                     // ... everyone's share; and everyone is done with block j-1
        if (j + 2 < nblocks) issue_block(stage_nxt + 1 == kStages ? 0 : stage_nxt + 1, (j + 2) * kBN);

        // scores of block j+1 relative to m_run (MFMA only)
        qk_block(stage_nxt, m_run, s_nxt);
        __builtin_amdgcn_sched_barrier(0);

        // fused: output update with block j (MFMA + transposing reads) and the speculative probabilities of
        // block j+1 (VALU)
        const unsigned char* sv = lds + stage * Traits::kStageBytes + Traits::kTileBytes;
        f16x8 pn[Traits::kKvSteps];
        float psum = 0.f;
        float mxn = s_nxt[0][0];
#pragma unroll
        for (int t = 0; t < Traits::kKvTiles; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                mxn = fmaxf(mxn, s_nxt[t][e]);
                const float p = detail::exp2_raw(s_nxt[t][e]);
                psum += p;
                pn[2 * t + e / 8][e % 8] = static_cast<_Float16>(p);
            }
#pragma unroll
        for (int dt = 0; dt < Traits::kDTiles; ++dt)
#pragma unroll
            for (int s2 = 0; s2 < Traits::kKvSteps; ++s2) pv_mfma(sv, dt, s2);
        // pin the speculative results here: without this the compiler sinks their computation below the branch
        // that follows, out of the shadow of the MFMAs
#pragma unroll
        for (int s2 = 0; s2 < Traits::kKvSteps; ++s2) asm volatile("" : "+v"(pn[s2]));
        asm volatile("" : "+v"(psum), "+v"(mxn));
        __builtin_amdgcn_sched_barrier(0);

        // the speculation holds unless some score of the block exceeds its query's reference maximum by 2^kLazy
        if (__any(mxn > kLazy)) {
            mxn = fmaxf(mxn, detail::exchange32(mxn));
            const bool upd = mxn > kLazy;
            const float m_new = upd ? m_run + mxn : m_run;
            const float alpha = detail::exp2_raw(m_run - m_new);
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < Traits::kDTiles; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) o_acc[t][e] *= alpha;
            const float delta = m_run - m_new;
            m_run = m_new;
            psum = 0.f;
#pragma unroll
            for (int t = 0; t < Traits::kKvTiles; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float p = detail::exp2_raw(s_nxt[t][e] + delta);
                    psum += p;
                    pn[2 * t + e / 8][e % 8] = static_cast<_Float16>(p);
                }
        }
        l_run += psum;
#pragma unroll
        for (int s2 = 0; s2 < Traits::kKvSteps; ++s2) pf[s2] = pn[s2];
        stage = stage_nxt;
    }
    {
        // last block: only its output update is left
        const unsigned char* sv = lds + stage * Traits::kStageBytes + Traits::kTileBytes;
#pragma unroll
        for (int dt = 0; dt < Traits::kDTiles; ++dt)
#pragma unroll
            for (int s2 = 0; s2 < Traits::kKvSteps; ++s2) pv_mfma(sv, dt, s2);
    }

    // epilogue: O[q, d] = Oᵀ[d, q] / l, staged through LDS for 16-byte row-contiguous stores
    const float l_tot = l_run + detail::exchange32(l_run);
    const float inv_l = 1.0f / l_tot;
    __syncthreads();  // all wavefronts are done with the K/V stages
    unsigned char* stg = lds + wave * (32 * kRowBytes);
    constexpr int kSlotMask = (kRowBytes / 8 - 1) & ~1;
#pragma unroll
    for (int dt = 0; dt < Traits::kDTiles; ++dt) {
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            f16x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = static_cast<_Float16>(o_acc[dt][4 * qd + e] * inv_l);
            const int slot = (32 * dt + 8 * qd + 4 * h) >> 2;
            const int pslot = slot ^ (((q32 & 15) << 1) & kSlotMask);
            *reinterpret_cast<f16x4*>(stg + q32 * kRowBytes + pslot * 8) = v;
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    constexpr int kLanesPerRow = kRowBytes / 16;
    constexpr int kRowsPerIter = kWaveSize / kLanesPerRow;
    const int rr = lane / kLanesPerRow, cc = lane % kLanesPerRow;
#pragma unroll
    for (int it = 0; it < 32 / kRowsPerIter; ++it) {
        const int row = it * kRowsPerIter + rr;
        const int pslot = (2 * cc) ^ (((row & 15) << 1) & kSlotMask);
        const u32x4 v = *reinterpret_cast<const u32x4*>(stg + row * kRowBytes + pslot * 8);
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(Oh + size_t(row) * kD) + cc * 16));  // whole rows, streamed
    }
}

}  // namespace tiledcuda::kernels
