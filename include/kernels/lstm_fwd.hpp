// One time step of the fused LSTM layer, streaming variant for gfx950 (the tuned counterpart of
// kernels/lstm.hpp). Same contract: gates = concat(x_t, h_{t-1}) · Wᵀ + bias (W [4H, I+H], gate
// order i, f, g, o), c_t = σ(f) c_{t-1} + σ(i) tanh(g), h_t = σ(o) tanh(c_t); f16 operands, f32
// gates and cell state. The reference has no LSTM kernel (Makefile:3 only names a test).
//
// The step is a [B x (I+H)] x [(I+H) x 4H] product with almost no reuse (B = 256), so it is bound by
// moving W (and the activations) through L2 and LDS, not by the MFMAs:
//   * a workgroup owns 64 batch rows x 16 hidden units and computes all four gates for them; the 64
//     weight rows of the tile are ordered [wavefront column][gate][8 hidden units], so that with
//     v_mfma_f32_32x32x16_f16 (operands swapped) register quad r / 4 of a lane is gate r / 4 of the
//     same (batch row, hidden unit): the cell update is lane-local and the gate matrix never exists
//     in memory;
//   * the workgroup has 8 wavefronts in two groups of 2 x 2: group 0 multiplies the first 64 k-columns
//     of every stage, group 1 the other 64 (two wavefronts per SIMD, so one group's LDS reads and barrier
//     waits hide under the other's MFMAs); the two partial sums are added through LDS at the end;
//   * A (x_t or h_{t-1}) and W tiles of 128 k-columns go global -> LDS directly (16 B per lane) into a
//     ring of kStages stages; every request covers 256 contiguous bytes of a row (W is walked
//     column-block by column-block with a 4 KiB row pitch, so short requests waste DRAM pages);
//     kStages - 1 stages (4 x 32 KiB per CU) are in flight, which is what hides the HBM / L2 latency of
//     a streaming kernel; one barrier per stage;
//   * LDS rows are 256 B with the 16-byte chunks XOR-ed by row % 16 (bank-conflict-free
//     ds_read_b128 for the 32-row MFMA operands), applied on the global-address side;
//   * workgroup ids are mapped so that the four batch tiles that share a W slice get ids that are
//     congruent modulo 8 (same XCD): the slice is fetched from HBM once and served from that XCD's L2.
#pragma once

#include "config.hpp"
#include "hip_utils.hpp"
#include "kernels/gemm_pipelined.hpp"  // detail::load_lds_16B

namespace tiledcuda::kernels {

template <const int kI_, const int kH_, const int kStages_ = 5>
struct LstmFwdTraits {
    static constexpr int kI = kI_, kH = kH_, kStages = kStages_;
    static constexpr int kKK = kI + kH;
    static constexpr int kTM = 64;   // batch rows per workgroup
    static constexpr int kTH = 16;   // hidden units per workgroup (x 4 gates = 64 weight rows)
    static constexpr int kBK = 128;  // k-columns per stage: 256 contiguous bytes per row and request
    static constexpr int kGroups = 2;  // wavefront groups; group g multiplies k-columns 64 g .. 64 g + 63 of a stage
    static constexpr int kWaves = 4 * kGroups;
    static constexpr int kThreads = kWaves * kWaveSize;
    static constexpr int kRowBytes = 2 * kBK;                      // 256
    static constexpr int kTileBytes = 64 * kRowBytes;              // A or W tile: 16 KiB
    static constexpr int kStageBytes = 2 * kTileBytes;             // 32 KiB
    static constexpr int kLoadsPerWave = 4;                        // 32 one-KiB instructions per stage / 8 wavefronts
    static constexpr int kLdsBytes = kStages * kStageBytes;
    // kI == kH == 0: the sizes are kernel arguments (I % 128 == 0, H % 128 == 0, checked by the launcher)
    static constexpr bool kRuntimeShape = kI == 0 && kH == 0;
    static_assert(kI % kBK == 0 && kH % kBK == 0 && kH % kTH == 0);
    static_assert((kH / kTH) % 8 == 0, "the workgroup map deals hidden tiles to the 8 XCDs");
    static_assert(kStages >= 2 && (kStages - 2) * kLoadsPerWave <= 63, "vmcnt is a 6-bit counter");
    static_assert(kLdsBytes <= kMaxLdsBytes);
};

namespace detail {
// v_exp_f32 and v_rcp_f32 (1 ulp), no IEEE division sequence: the cell update is 20 such pairs per lane and step
DEVICE float sigmoid_fast(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
DEVICE float tanh_fast(float x) { return 1.0f - 2.0f * __builtin_amdgcn_rcpf(__expf(2.0f * x) + 1.0f); }

template <int N>
DEVICE void wait_vmcnt_lgkm0() {
    __builtin_amdgcn_s_waitcnt(0x0070 | (N & 0xF) | ((N >> 4) << 14));
}

}  // namespace detail

/// grid = (B / 64) * (H / 16) workgroups (1-D), block = 512, dynamic LDS = Traits::kLdsBytes.
/// h_in == nullptr: h_{t-1} = 0; c_in == nullptr: c_{t-1} = 0. h_out must not alias h_in.
/// kHoisted: the input half of the gates, x_t · W[:, :I]ᵀ, was computed beforehand for the whole sequence (one large
/// GEMM) and is passed as pre_t [B, 4H] f32; the step then streams only h_{t-1} and W[:, I:] (half the bytes) and x_t
/// is not read.
/// I, H: the sizes, used by LstmFwdTraits<0, 0> (any multiples of 128); the other instantiations have them as constants.
template <typename Traits, bool kHoisted = false>
__global__ void __launch_bounds__(Traits::kThreads)
    lstm_cell_fwd(const __half* __restrict__ x_t, const __half* __restrict__ h_in, const __half* __restrict__ W,
                  const __half* __restrict__ bias, const float* c_in, float* c_out, __half* __restrict__ h_out,
                  int B, const float* __restrict__ pre_t, int I, int H) {
    constexpr int kBK = Traits::kBK;
    const int kI = Traits::kRuntimeShape ? I : Traits::kI, kH = Traits::kRuntimeShape ? H : Traits::kH;
    const int kKK = kI + kH;
    constexpr int S = Traits::kStages, L = Traits::kLoadsPerWave;
    extern __shared__ __align__(1024) unsigned char lds[];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int group = wave >> 2;  // which k-tile of a stage this wavefront multiplies
    const int wave_m = (wave >> 1) & 1, wave_n = wave & 1;

    // workgroup -> (batch tile, hidden tile): the m_tiles workgroups of one hidden tile share id % 8
    const int m_tiles = B / Traits::kTM;
    const int bid = blockIdx.x;
    const int xcd = bid & 7, rest = bid >> 3;
    const int m_tile = rest % m_tiles;
    const int h_tile = (rest / m_tiles) * 8 + xcd;
    const int row0 = m_tile * Traits::kTM;
    const int hid0 = h_tile * Traits::kTH;

    // ---- global -> LDS. A stage is [A tile, W tile], 64 rows of 256 B each. Instruction t (0..31) of a stage
    // fills 4 rows: t < 16: A rows 4 t .. + 3; t >= 16: W tile rows 4 (t - 16) .. + 3, where W tile row
    // 32 wn + 8 gate + jj is weight row gate * H + hid0 + 8 wn + jj. Wavefront w issues t = 4 w .. 4 w + 3.
    // Physical 16-byte chunk p of row r holds logical chunk p ^ (r % 16).
    const int lrow = lane >> 4, lchk = lane & 15;
    const int k_begin = kHoisted ? kI : 0;
    const int k_end = h_in ? kKK : kI;
    const int ktiles = (k_end - k_begin) / kBK;
    auto issue_stage = [&](int stage, int kt) {
        const int k0 = k_begin + kt * kBK;
        unsigned char* sbase = lds + stage * Traits::kStageBytes;
#pragma unroll
        for (int j = 0; j < L; ++j) {
            const int t = wave * L + j;  // 0..31, wave-uniform
            const int row = (t & 15) * 4 + lrow;
            const int chunk = lchk ^ (row & 15);
            const __half* src;
            if (t < 16) {
                src = k0 < kI ? x_t + size_t(row0 + row) * kI + k0 + chunk * 8
                              : h_in + size_t(row0 + row) * kH + (k0 - kI) + chunk * 8;
            } else {
                const int wrow = ((row >> 3) & 3) * kH + hid0 + 8 * (row >> 5) + (row & 7);
                src = W + size_t(wrow) * kKK + k0 + chunk * 8;
            }
            detail::load_lds_16B_untracked(src, sbase + t * 1024);
        }
    };

    const int frow = lane & 31, fhalf = lane >> 5;
    // operand fragment of k-substep kk (0..3) of this group's half of the stage
    auto read_frag = [&](const unsigned char* base, int row, int kk) -> f16x8 {
        const int chunk = (8 * group + 2 * kk + fhalf) ^ (row & 15);
        return *reinterpret_cast<const f16x8*>(base + row * Traits::kRowBytes + chunk * 16);
    };

    // ---- operands of the cell update, fetched now so that their latency hides under the k loop
    const int b = row0 + wave_m * 32 + frow;
    const int hid = hid0 + 8 * wave_n + 4 * fhalf;
    f32x4 c_prev = {0.f, 0.f, 0.f, 0.f};
    f16x4 bias_v[4];
    f32x4 pre_v[4];
    if (group == 0) {
        if (c_in) c_prev = *reinterpret_cast<const f32x4*>(c_in + size_t(b) * kH + hid);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            bias_v[g] = *reinterpret_cast<const f16x4*>(bias + g * kH + hid);
            if constexpr (kHoisted) pre_v[g] = *reinterpret_cast<const f32x4*>(pre_t + size_t(b) * (4 * kH) + g * kH + hid);
        }
    }

    // two accumulators: consecutive MFMAs do not depend on each other
    f32x16 acc0, acc1;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc0[e] = acc1[e] = 0.f;

    // prologue: stages 0 .. S-2 in flight
#pragma unroll
    for (int s = 0; s < S - 1; ++s)
        if (s < ktiles) issue_stage(s, s);

    int stage = 0;
    int fill = S - 1;
    for (int p = 0; p < ktiles; ++p) {
        // Stage p has landed when at most the stages issued after it are outstanding. Full pipeline: S - 2
        // stages of L loads each; in the tail (fewer stages issued after p) wait for everything.
        if (p + S - 2 <= ktiles - 1) detail::wait_vmcnt_lgkm0<(S - 2) * L>();
        else detail::wait_vmcnt_lgkm0<0>();
        detail::lds_barrier();  // everyone's share of stage p landed; everyone finished reading stage p-1 (= `fill`)
        if (p + S - 1 < ktiles) issue_stage(fill, p + S - 1);

        {
            const unsigned char* sa = lds + stage * Traits::kStageBytes;
            const unsigned char* sw = sa + Traits::kTileBytes;
            f16x8 fa[4], fw[4];
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                fa[kk] = read_frag(sa, wave_m * 32 + frow, kk);
                fw[kk] = read_frag(sw, wave_n * 32 + frow, kk);
            }
            // operands swapped: accumulator rows = batch, register quad = gate
            acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[0], fa[0], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[1], fa[1], acc1, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[2], fa[2], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[3], fa[3], acc1, 0, 0, 0);
        }
        fill = stage;
        stage = stage + 1 == S ? 0 : stage + 1;
    }
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = acc0[e] + acc1[e];

    // ---- add the two groups' partial sums: group 1 parks its accumulators in LDS (16 f32 per lane)
    detail::lds_barrier();  // all reads of the last stage are done
    float* park = reinterpret_cast<float*>(lds) + ((wave & 3) * 64 + lane) * 16;
    if (group == 1) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            f32x4 v = {acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
            *reinterpret_cast<f32x4*>(park + 4 * q) = v;
        }
    }
    detail::lds_barrier();
    if (group == 1) return;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(park + 4 * q);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[4 * q + e] += v[e];
    }

    // ---- cell update. acc[4 g + e]: batch row = row0 + 32 wave_m + lane % 32, gate g,
    // hidden unit = hid0 + 8 wave_n + 4 (lane / 32) + e (c_prev and the biases were fetched before the k loop).
    f32x4 c_new;
    f16x4 h_new;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float gi = acc[0 + e] + static_cast<float>(bias_v[0][e]);
        float gf = acc[4 + e] + static_cast<float>(bias_v[1][e]);
        float gg = acc[8 + e] + static_cast<float>(bias_v[2][e]);
        float go = acc[12 + e] + static_cast<float>(bias_v[3][e]);
        if constexpr (kHoisted) {
            gi += pre_v[0][e];
            gf += pre_v[1][e];
            gg += pre_v[2][e];
            go += pre_v[3][e];
        }
        const float cn = detail::sigmoid_fast(gf) * c_prev[e] + detail::sigmoid_fast(gi) * detail::tanh_fast(gg);
        c_new[e] = cn;
        h_new[e] = static_cast<_Float16>(detail::sigmoid_fast(go) * detail::tanh_fast(cn));
    }
    *reinterpret_cast<f32x4*>(c_out + size_t(b) * kH + hid) = c_new;
    *reinterpret_cast<f16x4*>(h_out + size_t(b) * kH + hid) = h_new;
}

}  // namespace tiledcuda::kernels
