// The time loop of the fused LSTM layer as ONE launch, weight-stationary, for gfx950: after the input half of the
// gates of all T steps has been computed by one large GEMM (pre[T, B, 4H] = x · W[:, :I]ᵀ, f32 or f16), this kernel runs the
// recurrence gates_t = pre_t + h_{t-1} · W[:, I:]ᵀ + bias, c_t = σ(f) c_{t-1} + σ(i) tanh(g), h_t = σ(o) tanh(c_t)
// for t = 0 .. T-1 without returning to the host. Same contract and gate order (i, f, g, o) as kernels/lstm_fwd.hpp.
// The reference has no LSTM kernel (its Makefile:3 only names a test).
//
// What bounds a step of the launch-per-step kernels is not arithmetic (B = 256 rows) but streaming the 8 MiB of
// recurrent weights through every CU again and the fixed cost of a dependent launch. Here nothing but h moves:
//   * the chip is used as 8 independent machines. An XCD (32 CUs, one L2) owns 32 batch rows and a complete copy of
//     the recurrent weights W[:, I:] (4H x H f16 = 8 MiB for H = 1024), spread over its CUs' registers: a CU owns 32
//     hidden units x 4 gates = 128 weight rows = 256 KiB, a wavefront (one per SIMD) 8 units x 4 gates x H columns =
//     64 KiB = 256 registers per lane, held as the 64 A-operand fragments of v_mfma_f32_32x32x16_f16 (the matrix
//     instructions read A and B from either register file, so the weights fill the AGPR half). W is read from memory
//     once per layer;
//   * a step of a CU: the 32 x H block h_{t-1} of its XCD (64 KiB, contiguous in h_all) goes global -> LDS directly in
//     four pieces (rows of 128 contiguous bytes per request), each wavefront multiplies its weights with all of it
//     (64 MFMAs, accumulator rows = batch, so the four gates of a (row, unit) are four registers of one lane), adds
//     pre_t (fetched a step ahead) and the bias, updates its 32 x 8 cell values (registers, for all T steps) and
//     stores its 32 x 8 piece of h_t;
//   * h is exchanged only between the 32 CUs of an XCD, through that XCD's L2: plain stores (the vector L1 writes
//     through), loads that bypass the L1 (sc1), and one counter per XCD: a CU adds 1 when its stores of h_t have been
//     acknowledged, and polls for 32 (t + 1) before it loads h_t. No traffic crosses XCDs, no cache is flushed. (A
//     counter per quarter of the hidden units, polled right before that quarter is requested, was measured: the
//     three extra polls and barriers cost 0.7 us per step, far more than the skew between the CUs they could hide);
//   * workgroups whose ids are equal modulo 8 form a group (the dispatcher deals workgroups to the XCDs in turn, so
//     they share an XCD); that they really do is checked from the hardware's XCC_ID before the first exchange. The
//     launch needs every workgroup resident at once (grid = number of CUs, one workgroup per CU by register use),
//     which holds when the GPU is not shared with another kernel that never finishes; every wait is bounded by
//     `spin_ticks` (100 MHz ticks): when it expires, or when a group is spread over several XCDs, the workgroup
//     raises the error word and exits, and so does, in turn, every workgroup that waits for it. The outputs are then
//     invalid; the host reads the word.
// sync: 128-byte aligned device words, all zero at launch: [g] the XCDs group g runs on (one bit each), [8] error,
// [32 (g + 1)] the step counter of group g (128 bytes apart). Requirements: H in {256, 512, 768, 1024} (a CU always owns
// 32 hidden units, so a group is H / 32 CUs of its XCD and a wavefront's weights are H / 4 registers: 1024 is the
// register budget), B % 32 == 0, B <= 256 (8 XCDs), grid == 8 * H / 32 workgroups of 256 threads.
#pragma once

#include <type_traits>

#include "config.hpp"
#include "hip_utils.hpp"
#include "kernels/gemm_pipelined.hpp"  // detail::lds_barrier
#include "kernels/lstm_fwd.hpp"        // detail::sigmoid_fast, tanh_fast

namespace tiledcuda::kernels {

template <const int kH_>
struct LstmRecurrentTraits {
    static constexpr int kH = kH_;
    static constexpr int kRows = 32;          // batch rows per XCD
    static constexpr int kUnitsPerCu = 32;    // hidden units a workgroup owns
    static constexpr int kCusPerXcd = kH / kUnitsPerCu;  // workgroups that share the rows of an XCD: 32 for H = 1024
    static constexpr int kXcds = 8;
    static constexpr int kWaves = 4, kThreads = kWaves * kWaveSize;
    static constexpr int kUnitsPerWave = kUnitsPerCu / kWaves;  // 8 (x 4 gates = the 32 rows of an MFMA operand)
    static constexpr int kKSteps = kH / 16;                      // MFMAs per step and wavefront (64 for H = 1024)
    static constexpr int kRowBytes = kH * 2;
    static constexpr int kHBytes = kRows * kRowBytes;    // h_{t-1} of the XCD's rows: 64 KiB for H = 1024
    static constexpr int kStagingBytes = kWaves * 2 * 32 * 256;  // what the weights pass through on their way in
    static constexpr int kLdsBytes = kHBytes > kStagingBytes ? kHBytes : kStagingBytes;
    static constexpr int kPieces = 4;                    // h arrives in 4 pieces of kKSteps / 4 k-steps
    static constexpr int kStepsPerPiece = kKSteps / kPieces;
    static constexpr int kLoadsPerWave = kHBytes / 1024 / kWaves;  // one-KiB load instructions (16 for H = 1024)
    static constexpr int kLoadsPerPiece = kLoadsPerWave / kPieces;
    static constexpr int kGrid = kXcds * kCusPerXcd;
    static constexpr int kSyncWords = 32 * (kXcds + 1);
    static constexpr int kErrorWord = 8;
    static_assert(kH % 256 == 0 && kH >= 256 && kH <= 1024,
                  "a wavefront's weights are H / 4 registers per lane (at most the 256 AGPRs), a piece of h is a whole "
                  "number of load instructions and an even number of k-steps");
    static_assert(kUnitsPerWave == 8 && kLoadsPerWave == kLoadsPerPiece * kPieces && kStepsPerPiece == 4 * kLoadsPerPiece);
};

namespace detail {
/// Direct-to-LDS load of 16 bytes per lane that bypasses the vector L1 (device scope): for data other CUs wrote
/// during this launch. Untracked by the compiler, like load_lds_16B_untracked.
DEVICE void load_lds_16B_untracked_sc1(const void* gptr, unsigned int lds_wave_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off sc1" ::"v"(gptr), "s"(lds_wave_base)
                 : "m0", "memory");
}

/// acc += w · h on the matrix pipe with the A operand (the stationary weights) in AGPRs; / the same starting from zero.
DEVICE void mfma32_weights_in_agprs(f32x16& acc, const f16x8& w, const f16x8& h) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "a"(w), "v"(h));
}
DEVICE void mfma32_weights_in_agprs_zero(f32x16& acc, const f16x8& w, const f16x8& h) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "a"(w), "v"(h));
}
/// sigmoid(a) * tanh(b) as one quotient: (1 - E_b) / ((1 + E_a) (1 + E_b)) with E_a = e^-a, E_b = e^-2b - two v_exp_f32
/// and ONE v_rcp_f32 where the factors taken separately need two of each (the cell update sits on the critical path of
/// every step, and these instructions run at a quarter of the rate). b is clamped to +-20, where tanh is 1 to f32
/// precision and E_b stays finite; E_a may overflow (a < -88): the quotient is then 0, the limit.
DEVICE float sigmoid_times_tanh(float a, float b) {
    const float ea = __expf(-a), eb = __expf(-2.0f * __builtin_amdgcn_fmed3f(b, -20.0f, 20.0f));
    return (1.0f - eb) * __builtin_amdgcn_rcpf((1.0f + ea) * (1.0f + eb));
}
}  // namespace detail

/// pre: [T, B, 4H] f32 or f16 (PreType; gate-major columns, as W's rows); W: [4H, ldw] f16, the recurrent block starts at column
/// w_col0; bias [4H] f16; h0 [B, H] f16 or null (zeros); c0 [B, H] f32 or null; h_all [T, B, H] f16; c_out [B, H] f32.
/// peers: workgroups per XCD to wait for (kCusPerXcd; anything else only to exercise the bounded wait).
template <typename Traits, typename PreType = float>
__global__ void __launch_bounds__(Traits::kThreads)
    lstm_recurrent_xcd(const PreType* __restrict__ pre, const __half* __restrict__ W, int ldw, int w_col0,
                       const __half* __restrict__ bias, const __half* __restrict__ h0, const float* __restrict__ c0,
                       __half* h_all, float* __restrict__ c_out, int T, int B, unsigned int* sync,
                       unsigned long long spin_ticks, unsigned int peers) {
    constexpr int kH = Traits::kH;
    extern __shared__ __align__(1024) unsigned char lds[];
    __shared__ int s_abort;  // set by the polling lane when it gives up

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());

    // ---- where am I: the dispatcher deals workgroups to the XCDs in turn, so workgroups b with equal b % 8 share an
    // XCD: group g = b % 8 owns batch rows 32 g .., the workgroup is number b / 8 in it. The kernel does not rely on
    // that: every workgroup ORs the XCD it really runs on (hardware register XCC_ID, bits 3:0) into its group's word,
    // and the first wait of the time loop checks that the group saw one XCD only.
    const int group = blockIdx.x % Traits::kXcds, slot = blockIdx.x / Traits::kXcds;
    const int row0 = group * Traits::kRows;
    if (row0 >= B) return;
    const unsigned int xcc = __builtin_amdgcn_s_getreg(20 | (0 << 6) | ((4 - 1) << 11));
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_or(sync + group, 1u << xcc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_abort = 0;
    }
    unsigned int* counter = sync + 32 * (group + 1);

    // ---- the wavefront's weights: operand row n = 8 gate + j is weight row gate * H + unit0 + j; the lane holds row
    // lane % 32, columns 16 ks + 8 (lane / 32) .. + 7 of k-step ks
    const int frow = lane & 31, fhalf = lane >> 5;
    const int unit0 = slot * Traits::kUnitsPerCu + wave * Traits::kUnitsPerWave;
    f16x8 wf[Traits::kKSteps];
    auto load_weights = [&]() {
        // A lane's share of a fragment is 16 bytes of one weight row, so loading fragments straight from memory asks
        // for 32-byte pieces of 32 rows per instruction; instead the wavefront's 32 rows x 2 KiB pass through its
        // quarter of the LDS (not yet in use) in 8 chunks of 32 rows x 256 B (8 k-steps), loaded directly to LDS in
        // runs of 256 contiguous bytes (4 rows per instruction), two chunks in flight, and read back as fragments.
        // Physical 16-byte chunk p of row r holds logical chunk p ^ (r % 16) (conflict-free ds_read_b128).
        constexpr int kChunks = Traits::kKSteps / 8, kChunkBytes = 32 * 256;
        const unsigned int stage = static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds)) + wave * (2 * kChunkBytes);
        const int lr = lane >> 4, lc = lane & 15;
        const __half* wsrc[8];  // this lane's source for load instruction q of a chunk: row 4 q + lr
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const int n = 4 * q + lr;
            wsrc[q] = W + size_t((n >> 3) * kH + unit0 + (n & 7)) * ldw + w_col0 + (lc ^ (n & 15)) * 8;
        }
        auto issue_chunk = [&](int c) {
#pragma unroll
            for (int q = 0; q < 8; ++q)
                detail::load_lds_16B_untracked_sc1(wsrc[q] + c * 128,
                                                   __builtin_amdgcn_readfirstlane(stage + (c & 1) * kChunkBytes + q * 1024));
        };
        issue_chunk(0);
        issue_chunk(1);
        using lds_ptr = __attribute__((address_space(3))) const f16x8*;
#pragma unroll
        for (int c = 0; c < kChunks; ++c) {
            // chunk c has landed when at most the 8 loads of chunk c + 1 are outstanding
            if (c + 1 < kChunks) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
            for (int s = 0; s < 8; ++s)
                wf[8 * c + s] = *reinterpret_cast<lds_ptr>(stage + (c & 1) * kChunkBytes + frow * 256 +
                                                           (((2 * s + fhalf) ^ (frow & 15)) * 16));
            if (c + 2 < kChunks) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the reads are done before the buffer is refilled
                issue_chunk(c + 2);
            }
        }
        // into the AGPR half, where the MFMAs below take them from
#pragma unroll
        for (int ks = 0; ks < Traits::kKSteps; ++ks) asm volatile("" : "+a"(wf[ks]));
    };
    // Without an initial hidden state step 0 multiplies nothing: the weights are fetched behind it (64 MiB through the
    // fabric for the chip, ~10 us), and the XCD's first exchange of h runs under that fetch.

    // ---- the lane's share of the cell update: accumulator register 4 g + e is gate g of batch row row0 + lane % 32,
    // hidden unit unit0 + 4 (lane / 32) + e
    const int b = row0 + frow;
    const int hid = unit0 + 4 * fhalf;
    f32x4 c_state = {0.f, 0.f, 0.f, 0.f};
    if (c0) c_state = *reinterpret_cast<const f32x4*>(c0 + size_t(b) * kH + hid);
    // four consecutive pre-activations of one gate: one 16-byte or 8-byte load; widened to f32 only where the values
    // are used (a conversion next to the load would make the compiler wait for the load, and with it for every older
    // load of the wavefront, right there)
    using PreRaw = std::conditional_t<sizeof(PreType) == 4, f32x4, f16x4>;
    auto load_pre = [&](size_t row, int g) -> PreRaw {
        return *reinterpret_cast<const PreRaw*>(pre + row * (4 * kH) + g * kH + hid);
    };
    auto widen_pre = [](const PreRaw& v) -> f32x4 {
        return f32x4{static_cast<float>(v[0]), static_cast<float>(v[1]), static_cast<float>(v[2]), static_cast<float>(v[3])};
    };
    f32x4 bias_v[4], pre_v[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const f16x4 bv = *reinterpret_cast<const f16x4*>(bias + g * kH + hid);
#pragma unroll
        for (int e = 0; e < 4; ++e) bias_v[g][e] = static_cast<float>(bv[e]);
        pre_v[g] = widen_pre(load_pre(size_t(b), g)) + bias_v[g];
    }

    // ---- global -> LDS: load instruction j (0 .. kLoadsPerWave - 1) of wavefront w brings rows 8 w .. 8 w + 7, logical
    // 16-byte chunks 8 j .. 8 j + 7 (k-steps 4 j .. 4 j + 3): 128 contiguous bytes per row.
    // The landing place of an instruction is 1 KiB of LDS, so h is stored piecewise: block (j, w) = [8 rows][8 chunks
    // of 16 B]; inside a block, physical chunk p of row r holds logical chunk p ^ key(r), key(r) = (r % 8) ^ (r / 8 % 2):
    // the ds_read_b128 of 16 consecutive rows at one k-offset then touches every bank once (rows of equal parity share
    // a bank half: their 8 keys differ). The permutation is applied on the global-address side.
    const unsigned int lds_base = static_cast<unsigned int>(reinterpret_cast<uintptr_t>(lds));
    const int lrow = 8 * wave + (lane >> 3), lchk = lane & 7;
    auto key = [](int r) { return (r & 7) ^ ((r >> 3) & 1); };
    // (piece p: this wavefront's loads kLoadsPerPiece p .. kLoadsPerPiece (p + 1) - 1, a quarter of the hidden units)
    auto issue_h_piece = [&](const __half* src_rows, int p) {
#pragma unroll
        for (int jj = 0; jj < Traits::kLoadsPerPiece; ++jj) {
            const int j = p * Traits::kLoadsPerPiece + jj;
            const int chunk = 8 * j + (lchk ^ key(lrow));
            detail::load_lds_16B_untracked_sc1(src_rows + size_t(lrow) * kH + chunk * 8,
                                               __builtin_amdgcn_readfirstlane(lds_base + (j * Traits::kWaves + wave) * 1024));
        }
    };
    // fragment of k-step ks: row frow, logical chunk 2 ks + fhalf -> block (j = ks / 4, w = frow / 8), inside the block
    // row frow % 8, physical chunk ((2 ks + fhalf) % 8) ^ key(frow)
    const unsigned int frag_base = lds_base + (frow >> 3) * 1024 + (frow & 7) * 128;
    auto read_frag = [&](int ks) -> f16x8 {
        const int c = ((2 * ks + fhalf) & 7) ^ key(frow);
        using lds_ptr = __attribute__((address_space(3))) const f16x8*;
        return *reinterpret_cast<lds_ptr>(frag_base + (ks >> 2) * (Traits::kWaves * 1024) + c * 16);
    };

    f32x16 acc0, acc1;
    constexpr int kSPP = Traits::kStepsPerPiece, kLPP = Traits::kLoadsPerPiece;
    auto read_piece = [&](f16x8(&f)[kSPP], int p) {
#pragma unroll
        for (int s = 0; s < kSPP; ++s) f[s] = read_frag(kSPP * p + s);
    };
    // The MFMAs of piece p, and between them the fragment reads of piece p + 1 (one read per MFMA: issued in a block
    // they would hold up the matrix pipe for as long as eight MFMAs take). Weights first: accumulator rows = batch,
    // register quad = gate; two accumulators, so that consecutive MFMAs do not depend on each other; the first two
    // of a step start from zero.
    auto mfma_piece = [&](const f16x8(&f)[kSPP], f16x8(&next)[kSPP], int p) {
#pragma unroll
        for (int s = 0; s < kSPP; ++s) {
            f32x16& acc = (s & 1) ? acc1 : acc0;
            if (p == 0 && s < 2) detail::mfma32_weights_in_agprs_zero(acc, wf[s], f[s]);
            else detail::mfma32_weights_in_agprs(acc, wf[kSPP * p + s], f[s]);
            if (p + 1 < Traits::kPieces) next[s] = read_frag(kSPP * (p + 1) + s);
        }
    };

    constexpr unsigned long long kNoLimit = ~0ull;
    // one time step; kHasH = false: step 0 without an initial hidden state (nothing to multiply)
    auto time_step = [&](int t, auto has_h_c) {
        constexpr bool kHasH = decltype(has_h_c)::value;
        const __half* h_prev = t == 0 ? h0 : h_all + size_t(t - 1) * B * kH;
        if constexpr (!kHasH) {
#pragma unroll
            for (int e = 0; e < 16; ++e) acc0[e] = acc1[e] = 0.f;
        }
        if constexpr (kHasH) {
            // ---- everybody's piece of h_{t-1} is in the L2 when the XCD's counter has reached peers * t
            if (t > 0 && threadIdx.x == 0) {
                const unsigned int target = peers * unsigned(t);
                const unsigned long long t_start = __builtin_amdgcn_s_memrealtime();
                while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                    if (spin_ticks != kNoLimit && __builtin_amdgcn_s_memrealtime() - t_start > spin_ticks) {
                        s_abort = 1;
                        __hip_atomic_store(sync + Traits::kErrorWord, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
                // everybody's OR was acknowledged before its first arrival: one XCD per group, or the exchange through
                // the L2 is not coherent and the launch must not go on
                if (t == 1 && __hip_atomic_load(sync + group, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != (1u << xcc)) {
                    s_abort = 1;
                    __hip_atomic_store(sync + Traits::kErrorWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            // the poll is over; everyone has finished reading the previous h from LDS (they stored h_{t-1} after it)
            detail::lds_barrier<0>();
            if (__builtin_amdgcn_readfirstlane(*const_cast<volatile int*>(&s_abort))) return false;
            const __half* src_rows = h_prev + size_t(row0) * kH;
#pragma unroll
            for (int p = 0; p < Traits::kPieces; ++p) issue_h_piece(src_rows, p);
        }
        // pre-activations of the next step, a step ahead (independent of h)
        PreRaw pre_next[4];
        if (t + 1 < T) {
#pragma unroll
            for (int g = 0; g < 4; ++g) pre_next[g] = load_pre(size_t(t + 1) * B + b, g);
        }
        if constexpr (kHasH) {
            // Piece p (this wavefront's loads kLPP p .. kLPP (p + 1) - 1) has landed when at most the loads issued after
            // it are outstanding (the later pieces and the 4 loads of pre_next); then, behind the barrier, everyone's.
            // The fragments of piece p + 1 are read between the MFMAs of piece p, so the barrier of piece p + 1 comes
            // first.
            f16x8 fa[kSPP], fb[kSPP];
            if (t + 1 < T) detail::lds_barrier<3 * kLPP + 4>();
            else detail::lds_barrier<3 * kLPP>();
            read_piece(fa, 0);
            if (t + 1 < T) detail::lds_barrier<2 * kLPP + 4>();
            else detail::lds_barrier<2 * kLPP>();
            mfma_piece(fa, fb, 0);
            if (t + 1 < T) detail::lds_barrier<kLPP + 4>();
            else detail::lds_barrier<kLPP>();
            mfma_piece(fb, fa, 1);
            if (t + 1 < T) detail::lds_barrier<0 + 4>();
            else detail::lds_barrier<0>();
            mfma_piece(fa, fb, 2);
            mfma_piece(fb, fa, 3);
            // the compiler does not know the statements above are MFMAs: wait for the last results
            detail::mfma_results_wait();
            asm volatile("" : "+v"(acc0), "+v"(acc1));
        }

        // ---- cell update and this lane's 4 units of h_t
        f16x4 h_new;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // (pre_v already holds the bias)
            const float gi = acc0[0 + e] + acc1[0 + e] + pre_v[0][e];
            const float gf = acc0[4 + e] + acc1[4 + e] + pre_v[1][e];
            const float gg = acc0[8 + e] + acc1[8 + e] + pre_v[2][e];
            const float go = acc0[12 + e] + acc1[12 + e] + pre_v[3][e];
            const float cn = detail::sigmoid_fast(gf) * c_state[e] + detail::sigmoid_times_tanh(gi, gg);
            c_state[e] = cn;
            h_new[e] = static_cast<_Float16>(detail::sigmoid_times_tanh(go, cn));
        }
        *reinterpret_cast<f16x4*>(h_all + (size_t(t) * B + b) * kH + hid) = h_new;
        if (t + 1 < T) {
#pragma unroll
            for (int g = 0; g < 4; ++g) pre_v[g] = widen_pre(pre_next[g]) + bias_v[g];  // (while the stores are under way)
            // arrival: every wavefront's stores of h_t have been acknowledged by the L2, then one lane counts
            detail::lds_barrier<0>();
            if (threadIdx.x == 0) __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return true;
    };
    // Without an initial hidden state step 0 multiplies nothing: it runs first, and the weights are fetched behind it
    // (64 MiB through the fabric for the chip, ~10 us) while the XCD's first exchange of h is under way.
    const int t0 = h0 ? 0 : 1;
    if (!h0) time_step(0, std::false_type{});
    if (t0 < T) load_weights();
    for (int t = t0; t < T; ++t)
        if (!time_step(t, std::true_type{})) return;
    *reinterpret_cast<f32x4*>(c_out + size_t(b) * kH + hid) = c_state;
}

/// Zeroes the synchronisation words before a launch of lstm_recurrent_xcd (a kernel, not a memset: it may be recorded
/// into a HIP graph). One workgroup of kSyncWords threads. (The layer entry point lets the projection GEMM that precedes
/// the recurrence do this instead; the kernel is for callers that launch the recurrence on its own.)
__global__ void lstm_recurrent_clear_sync(unsigned int* sync) { sync[threadIdx.x] = 0u; }

}  // namespace tiledcuda::kernels
