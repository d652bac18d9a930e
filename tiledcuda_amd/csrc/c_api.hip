// Implementation of the C-ABI declared in include/tcu_c_api.h: argument checks, shape
// dispatch and kernel launches. No device memory is allocated here and no stream is
// synchronised (but for tcu_lstm_persistent_status, whose purpose it is); errors become status codes plus a
// thread-local message.
#include "tcu_c_api.h"

#include "kernels/b2b_gemm_fwd.hpp"
#include "kernels/flash_attn_fwd.hpp"
#include "kernels/flash_attn_tile_w64.hpp"
#include "kernels/flash_attn_w64_k32.hpp"
#include "kernels/flash_attn_w64.hpp"
#include "kernels/gemm_pipelined.hpp"
#include "kernels/gemm_ragged.hpp"
#include "kernels/gemm_w128.hpp"
#include "kernels/gemm_w128k.hpp"
#include "kernels/lstm_fwd.hpp"
#include "kernels/lstm_ragged.hpp"
#include "kernels/lstm_recurrent.hpp"
#include "kernels/mod.hpp"

#include <climits>
#include <cstdlib>
#include <mutex>
#include <set>
#include <algorithm>
#include <string>
#include <tuple>
#include <type_traits>
#include <utility>

using namespace tiledcuda;
using namespace tiledcuda::kernels;
namespace tl = tiledcuda::cell::tile_layout;

namespace {

thread_local std::string g_last_error;

// kernels whose dynamic-LDS limit has already been raised, per device
std::mutex g_attr_mutex;
std::set<std::pair<const void*, int>> g_attr_done;

int fail(int code, const std::string& msg) {
    g_last_error = msg;
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    return fail(TCU_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

/// Launch with dynamic LDS; raises the limit when the kernel needs more than the default. The kernel's parameter types
/// are taken from the kernel pointer and every argument is converted to its parameter's type before its address goes
/// into the argument array: an argument of another width or a wrong count is a compile error, not a garbled launch.
template <typename... Params, typename... Args>
int launch(void (*kernel)(Params...), dim3 grid, dim3 block, int lds_bytes, hipStream_t stream, Args&&... args) {
    static_assert(sizeof...(Params) == sizeof...(Args), "launch: argument count differs from the kernel's parameter count");
    static_assert((std::is_convertible_v<Args&&, Params> && ...), "launch: an argument does not convert to its parameter's type");
    if (lds_bytes > kMaxLdsBytes) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "kernel needs more LDS than a CU has");
    if (lds_bytes > 48 * 1024) {
        // once per kernel function (and per device: the attribute is per device)
        int device = 0;
        (void)hipGetDevice(&device);
        const auto key = std::make_pair(reinterpret_cast<const void*>(kernel), device);
        bool known;
        {
            std::lock_guard<std::mutex> lock(g_attr_mutex);
            known = g_attr_done.count(key) != 0;
        }
        if (!known) {
            // (every instantiation is launched with one fixed size; asking for the CU's whole LDS would be refused
            // for a kernel that also has static LDS)
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
            std::lock_guard<std::mutex> lock(g_attr_mutex);
            g_attr_done.insert(key);
        }
    }
    // the launch's own return value: an error left behind earlier by unrelated code of the calling thread is neither
    // reported as this launch's nor cleared
    std::tuple<std::remove_cv_t<Params>...> params(std::forward<Args>(args)...);
    void* argv[sizeof...(Params) + 1];
    [&]<size_t... kIs>(std::index_sequence<kIs...>) {
        ((argv[kIs] = static_cast<void*>(&std::get<kIs>(params))), ...);
    }(std::index_sequence_for<Params...>{});
    hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, argv, size_t(lds_bytes), stream);
    if (e != hipSuccess) return hip_fail(e, "kernel launch");
    return TCU_OK;
}

/// Adds which of the T step launches of an LSTM layer failed to the message (steps before it are enqueued).
int lstm_step_failed(int rc, int t, int T) {
    return fail(rc, g_last_error + " (LSTM step " + std::to_string(t) + " of " + std::to_string(T) +
                        "; the steps before it were enqueued)");
}

bool positive(std::initializer_list<int> v) {
    for (int x : v)
        if (x <= 0) return false;
    return true;
}

/// The kernels move 16 bytes per lane (vector loads, direct-to-LDS loads, vector stores): operands must start on a
/// 16-byte boundary (null = absent optional operand is fine here; required ones are checked for null separately).
bool aligned16(std::initializer_list<const void*> v) {
    for (const void* p : v)
        if (reinterpret_cast<uintptr_t>(p) % 16 != 0) return false;
    return true;
}

// ---------------------------------------------------------------------------- static scratch
// Device memory owned by the library for the entry point that may not allocate (tcu_lstm_f16_noalloc): every device
// the library runs on holds one copy of this array, at its own address, until the process ends. In host code the
// array's name is only a handle for hipGetSymbolAddress, never a device address.
constexpr unsigned long long kScratchBytes = 64ull << 20;
constexpr unsigned long long kPersistentSyncBytes = 4096;  // synchronisation words in front of the pre-activations
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

/// Device address of `scratch` on the current device, looked up once per device.
int scratch_address(void** out) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (device < 0 || device >= kMaxDevices) return fail(TCU_ERR_HIP, "device ordinal beyond the scratch table");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        if (!ptr || reinterpret_cast<uintptr_t>(ptr) % 256 != 0)
            return fail(TCU_ERR_HIP, "hipGetSymbolAddress(scratch) returned an unusable address");
        g_scratch_ptr[device] = ptr;
    }
    *out = g_scratch_ptr[device];
    return TCU_OK;
}

// ---------------------------------------------------------------------------- GEMM
template <typename OutType, int kM, int kN, int kK, int kTM, int kTN, int kChunkK, typename WarpLayout>
int launch_simple_gemm(const __half* A, const __half* B, OutType* C, hipStream_t stream) {
    using Shape = GemmShape<kM, kN, kK>;
    using Cfg = GemmTraits<__half, OutType, Shape, kTM, kTN, WarpLayout, kChunkK>;
    auto kernel = &simple_gemm<__half, OutType, kM, kN, kK, kTM, kTN, typename Cfg::IteratorA, typename Cfg::RegA,
                               typename Cfg::ALoader, typename Cfg::IteratorB, typename Cfg::RegB,
                               typename Cfg::BLoader, typename Cfg::GlobalC, typename Cfg::RegC,
                               typename Cfg::CStorer>;
    return launch(kernel, dim3(kM / kTM, kN / kTN), dim3(Cfg::kThreads), 0, stream, A, B, C);
}

template <typename OutType, int kM, int kN, int kK, int kTM, int kTN, int kTK, int kRK, typename WarpLayout>
int launch_all_mem_gemm(const __half* A, const __half* B, OutType* C, hipStream_t stream) {
    using Cfg = KeGemmTraits<__half, OutType, GemmShape<kM, kN, kK>, GemmShape<kTM, kTN, kTK>, kRK, WarpLayout>;
    auto kernel =
        &gemm<__half, OutType, kM, kN, kK, kTM, kTN, kTK, typename Cfg::GIteratorA, typename Cfg::SIteratorA,
              typename Cfg::SharedA, typename Cfg::RegA, typename Cfg::G2SLoaderA, typename Cfg::S2RLoaderA,
              typename Cfg::GIteratorB, typename Cfg::SIteratorB, typename Cfg::SharedB, typename Cfg::RegB,
              typename Cfg::G2SLoaderB, typename Cfg::S2RLoaderB, typename Cfg::GlobalC, typename Cfg::SharedC,
              typename Cfg::RegC, typename Cfg::R2SStorerC, typename Cfg::S2GStorerC>;
    return launch(kernel, dim3(kM / kTM, kN / kTN), dim3(Cfg::kThreads), Cfg::kShmBytes, stream, A, B, C);
}

using PipeLarge = PipelinedGemmTraits<256, 256, 64, 4, 2, 2>;  // 8 wavefronts, 2 per SIMD
using PipeMid = PipelinedGemmTraits<128, 128, 64, 2, 2, 2>;
using PipeSmall = PipelinedGemmTraits<64, 64, 64, 2, 2, 2>;
using PipeSmallRing = PipelinedGemmTraits<64, 64, 64, 2, 2, 4>;  // 4-stage ring, 64 KiB of LDS: 2 workgroups per CU

/// Which tile the pipelined kernel takes for a shape, and what the launch is expected to cost. A launch runs
/// ceil(tiles / capacity) rounds of workgroups, capacity = 256 CUs x the workgroups of that size a CU holds (1, 2, 4),
/// and a round costs K / 1024 x 25.5, 16 or 13 us for 256 x 256, 128 x 128 and 64 x 64 tiles (measured on full rounds at
/// K = 1024 .. 4096); the larger tile wins a tie. With few 64 x 64 tiles per CU there is no neighbour workgroup to hide
/// the latency of a tile's loads behind: then the same tile with a 4-stage ring (3 tiles in flight, 2 workgroups per
/// CU) is the choice: 4.2 us per K / 1024 with at most one workgroup per CU (1024^2 x 8192: 36.7 us), 5.8 with two, 7 per
/// round beyond.
enum PipeConfig { kPipeLarge, kPipeMid, kPipeSmall, kPipeSmallRing };
struct PipePlan {
    PipeConfig config;
    double us;
};
PipePlan pipelined_plan(int M, int N, int K) {
    const auto tiles = [&](int tile) { return (long)((M + tile - 1) / tile) * ((N + tile - 1) / tile); };
    const auto rounds = [&](int tile, int per_cu) { return double((tiles(tile) + 256l * per_cu - 1) / (256l * per_cu)); };
    const double large = rounds(256, 1) * 25.5, mid = rounds(128, 2) * 16.0, small = rounds(64, 4) * 13.0;
    const double ring = tiles(64) <= 256 ? 4.2 : tiles(64) <= 512 ? 5.8 : rounds(64, 2) * 7.0;
    const double least_small = small < ring ? small : ring;
    PipePlan plan;
    if (large <= mid && large <= least_small) plan = {kPipeLarge, large};
    else if (mid <= least_small) plan = {kPipeMid, mid};
    else if (small <= ring) plan = {kPipeSmall, small};
    else plan = {kPipeSmallRing, ring};
    plan.us = 2.5 + plan.us * K / 1024.0;
    return plan;
}

/// The pipelined kernel for M, N, K any multiples of 16, with the tile of pipelined_plan(). Edge tiles (rows clamped,
/// stores guarded, the K tail zeroed in LDS) are compiled in only where the shape is not a whole number of the chosen
/// tiles.
template <typename OutType>
int gemm_pipelined_dispatch(const __half* A, const __half* B, OutType* C, int M, int N, int K, hipStream_t stream,
                            int ldc = 0) {
    if (ldc == 0) ldc = N;
    if (M % 16 != 0 || N % 16 != 0 || K % 16 != 0)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "GEMM shapes are whole 16 x 16 tiles: M, N and K must be multiples of 16");
    if ((long)K * 512 >= (1l << 32))
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "pipelined GEMM addresses a tile's rows with 32-bit offsets: K < 2^23");
    auto go = [&](auto traits) {
        using Traits = decltype(traits);
        const long grid = (long)((M + Traits::kBM - 1) / Traits::kBM) * ((N + Traits::kBN - 1) / Traits::kBN);
        if (grid > INT_MAX) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "GEMM: too many tiles for one launch");
        if (M % Traits::kBM == 0 && N % Traits::kBN == 0 && K % Traits::kBK == 0)
            return launch(&gemm_pipelined<Traits, OutType, false>, dim3(unsigned(grid)), dim3(Traits::kThreads),
                          Traits::template lds_bytes<OutType>(), stream, A, B, C, M, N, K, ldc);
        return launch(&gemm_pipelined<Traits, OutType, true>, dim3(unsigned(grid)), dim3(Traits::kThreads),
                      Traits::template lds_bytes<OutType>(), stream, A, B, C, M, N, K, ldc);
    };
    switch (pipelined_plan(M, N, K).config) {
        case kPipeLarge: return go(PipeLarge{});
        case kPipeMid: return go(PipeMid{});
        case kPipeSmall: return go(PipeSmall{});
        default: return go(PipeSmallRing{});
    }
}

template <typename OutType>
int gemm_w128_dispatch(const __half* A, const __half* B, OutType* C, int M, int N, int K, hipStream_t stream,
                       int lda = 0, int ldb = 0, int ldc = 0, unsigned int* zero_words = nullptr, int zero_count = 0) {
    using T = GemmW128Traits;
    if (lda == 0) lda = K;
    if (ldb == 0) ldb = K;
    if (ldc == 0) ldc = N;
    if (M % 16 != 0 || N % 16 != 0 || K % 16 != 0)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the one-wavefront-per-SIMD GEMM needs M, N and K in multiples of 16");
    if ((long)std::max(lda, ldb) * 2 * T::kBM >= (1l << 32))
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the one-wavefront-per-SIMD GEMM addresses a 256-row panel with 32-bit offsets");
    if (M % T::kBM == 0 && N % T::kBN == 0 && K % T::kBK == 0)
        return launch(&gemm_w128<OutType>, dim3((M / T::kBM) * (N / T::kBN)), dim3(T::kThreads), T::kLdsBytes, stream, A, B,
                      C, M, N, K, lda, ldb, ldc, zero_words, zero_count);
    // edge tiles: rows beyond M or N loaded from the last valid row, stores guarded, a partial last tile of K zero-filled
    const long grid = (long)((M + T::kBM - 1) / T::kBM) * ((N + T::kBN - 1) / T::kBN);
    if (grid > INT_MAX) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "GEMM: too many tiles for one launch");
    return launch(&gemm_w128<OutType, T, true>, dim3(unsigned(grid)), dim3(T::kThreads), T::kLdsBytes, stream, A, B, C, M, N,
                  K, lda, ldb, ldc, zero_words, zero_count);
}

/// gemm_w128 with 256 x 128 workgroup tiles: for products with too few 256 x 256 tiles to fill the chip and too many
/// 128 x 128 tiles for one round of the K-splitting kernel.
template <typename OutType>
int gemm_w128_narrow_dispatch(const __half* A, const __half* B, OutType* C, int M, int N, int K, hipStream_t stream,
                              int ldc = 0) {
    using T = GemmW128TraitsN<4>;
    if (ldc == 0) ldc = N;
    if (M % 16 != 0 || N % 16 != 0 || K % T::kBK != 0)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the one-wavefront-per-SIMD GEMM with 256 x 128 tiles needs M and N in "
                                               "multiples of 16 and K % 64 == 0");
    if ((long)K * 2 * T::kBM >= (1l << 32))
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the one-wavefront-per-SIMD GEMM addresses a 256-row panel with 32-bit offsets");
    if (M % T::kBM == 0 && N % T::kBN == 0)
        return launch(&gemm_w128<OutType, T>, dim3((M / T::kBM) * (N / T::kBN)), dim3(T::kThreads), T::kLdsBytes, stream, A,
                      B, C, M, N, K, K, K, ldc, static_cast<unsigned int*>(nullptr), 0);
    // edge tiles: rows beyond M or N loaded from the last valid row, stores guarded
    const long grid = (long)((M + T::kBM - 1) / T::kBM) * ((N + T::kBN - 1) / T::kBN);
    if (grid > INT_MAX) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "GEMM: too many tiles for one launch");
    return launch(&gemm_w128<OutType, T, true>, dim3(unsigned(grid)), dim3(T::kThreads), T::kLdsBytes, stream, A, B, C, M, N,
                  K, K, K, ldc, static_cast<unsigned int*>(nullptr), 0);
}

template <typename OutType, typename T>
int launch_gemm_w128k(const __half* A, const __half* B, OutType* C, int M, int N, int K, hipStream_t stream, int ldc) {
    const long grid = (long)((M + T::kBM - 1) / T::kBM) * ((N + T::kBN - 1) / T::kBN);
    if (grid > INT_MAX) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "GEMM: too many tiles for one launch");
    if (M % T::kBM == 0 && N % T::kBN == 0)
        return launch(&gemm_w128k<OutType, false, T>, dim3(unsigned(grid)), dim3(T::kThreads), T::kLdsBytes, stream, A, B, C,
                      M, N, K, K, K, ldc);
    // edge tiles: rows beyond M or N loaded from the last valid row, stores guarded per 16 x 16 block
    return launch(&gemm_w128k<OutType, true, T>, dim3(unsigned(grid)), dim3(T::kThreads), T::kLdsBytes, stream, A, B, C, M,
                  N, K, K, K, ldc);
}

template <typename OutType>
int gemm_w128k_dispatch(const __half* A, const __half* B, OutType* C, int M, int N, int K, hipStream_t stream,
                        int ldc = 0) {
    using T = GemmW128kTraits;
    if (ldc == 0) ldc = N;
    if (M % 16 != 0 || N % 16 != 0 || K % T::kBK != 0)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the K-splitting one-wavefront-per-SIMD GEMM needs M and N in multiples of 16 "
                                               "and K in multiples of 128");
    if ((long)K * 2 * T::kBM >= (1l << 32))
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the K-splitting GEMM addresses a 128-row panel with 32-bit offsets");
    // All workgroups run at once (one per CU), so the launch takes as long as one tile: when 128 x 128 tiles would
    // leave a quarter of the CUs idle and 128 x 96 tiles still fit one round, the smaller tile is the shorter launch
    const long rows = (M + 127) / 128;
    const long tiles128 = rows * ((N + 127) / 128), tiles96 = rows * ((N + 95) / 96);
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
        cus = 0;
    if (cus > 0 && tiles128 <= (3l * cus) / 4 && tiles96 <= cus)
        return launch_gemm_w128k<OutType, GemmW128kTraitsN<6>>(A, B, C, M, N, K, stream, ldc);
    return launch_gemm_w128k<OutType, T>(A, B, C, M, N, K, stream, ldc);
}

template <typename OutType, int kM, int kN, int kK, int kTM, int kTN, typename WarpLayout>
int launch_tile_pipelined(const __half* A, const __half* B, OutType* C, hipStream_t stream) {
    using Traits = PipelinedGemmTileTraits<__half, OutType, GemmShape<kM, kN, kK>, kTM, kTN, WarpLayout>;
    auto kernel = &gemm_tile_pipelined<__half, OutType, Traits>;
    return launch(kernel, dim3((kM / kTM) * (kN / kTN)), dim3(Traits::kThreads), Traits::kShmBytes, stream, A, B, C);
}

/// The pipelined kernel composed from tile-library functors has compile-time shapes, like every kernel written against
/// the tile API: the instantiations below are the benchmark shape and the shapes its tests use.
template <typename OutType>
int gemm_tile_pipelined_dispatch(const __half* A, const __half* B, OutType* C, int M, int N, int K, hipStream_t stream) {
    using W42 = tl::RowMajor<4, 2>;
    using W22 = tl::RowMajor<2, 2>;
    if (M == 4096 && N == 4096 && K == 4096) return launch_tile_pipelined<OutType, 4096, 4096, 4096, 256, 256, W42>(A, B, C, stream);
    if (M == 1024 && N == 1024 && K == 1024) return launch_tile_pipelined<OutType, 1024, 1024, 1024, 256, 256, W42>(A, B, C, stream);
    if (M == 512 && N == 768 && K == 192) return launch_tile_pipelined<OutType, 512, 768, 192, 128, 128, W22>(A, B, C, stream);
    if (M == 256 && N == 256 && K == 64) return launch_tile_pipelined<OutType, 256, 256, 64, 64, 64, W22>(A, B, C, stream);
    return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the tile-API pipelined GEMM is instantiated for 4096^3, 1024^3, 512x768x192 "
                                           "and 256x256x64");
}

template <typename OutType, int kM, int kN, int kK>
int launch_tile_w128(const __half* A, const __half* B, OutType* C, hipStream_t stream) {
    using Traits = ScheduledGemmTileTraits<__half, OutType, GemmShape<kM, kN, kK>>;
    auto kernel = &gemm_tile_w128<__half, OutType, Traits>;
    return launch(kernel, dim3((kM / Traits::kTM) * (kN / Traits::kTN)), dim3(Traits::kThreads), Traits::kShmBytes, stream,
                  A, B, C);
}

/// The one-wavefront-per-SIMD kernel composed from tile-library functors: compile-time shapes, as above.
template <typename OutType>
int gemm_tile_w128_dispatch(const __half* A, const __half* B, OutType* C, int M, int N, int K, hipStream_t stream) {
    if (M == 4096 && N == 4096 && K == 4096) return launch_tile_w128<OutType, 4096, 4096, 4096>(A, B, C, stream);
    if (M == 1024 && N == 1024 && K == 1024) return launch_tile_w128<OutType, 1024, 1024, 1024>(A, B, C, stream);
    if (M == 512 && N == 768 && K == 192) return launch_tile_w128<OutType, 512, 768, 192>(A, B, C, stream);
    if (M == 256 && N == 256 && K == 64) return launch_tile_w128<OutType, 256, 256, 64>(A, B, C, stream);
    return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the tile-API one-wavefront-per-SIMD GEMM is instantiated for 4096^3, 1024^3, "
                                           "512x768x192 and 256x256x64");
}

/// M or N a little above a multiple of 256: edge tiles of 256 x 256 cost a whole extra round of workgroups for a
/// sliver of output. When the cost model says so, the product is computed as three launches on disjoint parts of C:
/// the leading block of whole 256 x 256 tiles by the one-wavefront-per-SIMD kernel, the columns beyond it (all rows)
/// and the rows beyond it (the leading columns) by the pipelined kernel with small tiles. Same order of the sum
/// everywhere, so the result is bit for bit that of one launch. Returns kPlanNotTaken when the plain launch is the
/// better plan.
constexpr int kPlanNotTaken = INT_MIN;
double gemm_w128_us(long tiles, int K);
template <typename OutType>
int gemm_main_and_strips(const __half* A, const __half* B, OutType* C, int M, int N, int K, hipStream_t stream,
                         double other_us) {
    using T = GemmW128Traits;
    const int Mm = M / T::kBM * T::kBM, Nm = N / T::kBN * T::kBN;
    if ((Mm == M && Nm == N) || K % T::kBK != 0 || (long)K * 512 >= (1l << 32)) return kPlanNotTaken;
    const long tiles = (long)(Mm / T::kBM) * (Nm / T::kBN);
    if (tiles < 128) return kPlanNotTaken;
    const double main_us = gemm_w128_us(tiles, K);
    const double right_us = N > Nm ? 2.0 + pipelined_plan(M, N - Nm, K).us : 0.0;
    const double bottom_us = M > Mm ? 2.0 + pipelined_plan(M - Mm, Nm, K).us : 0.0;
    if (main_us + right_us + bottom_us >= std::min(other_us, pipelined_plan(M, N, K).us)) return kPlanNotTaken;
    int rc = gemm_w128_dispatch<OutType>(A, B, C, Mm, Nm, K, stream, K, K, N);
    if (rc == TCU_OK && N > Nm) rc = gemm_pipelined_dispatch<OutType>(A, B + size_t(Nm) * K, C + Nm, M, N - Nm, K, stream, N);
    if (rc == TCU_OK && M > Mm)
        rc = gemm_pipelined_dispatch<OutType>(A + size_t(Mm) * K, B, C + size_t(Mm) * N, M - Mm, Nm, K, stream, N);
    return rc;
}

/// Whether AUTO sends an unsplit product to the kernel whose wavefronts split K: about one 128 x 128 tile per CU and a
/// long enough K (2048^3: 21.9 against 26.8 us for the LDS-bound 64 x 64-per-wavefront tilings, 1536 x 1536 x 4096: 26.6
/// against 38.5 us, 2048 x 2048 x 1536: 19.8 against 22.6 us); with a short K its reduction through LDS costs more than
/// it saves.
bool gemm_w128k_is_the_choice(int M, int N, int K) {
    if (M % 16 != 0 || N % 16 != 0 || K % 128 != 0 || K < 1024 || (long)K * 256 >= (1l << 32)) return false;
    const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
    // the fewer tiles, the longer K has to be (1408 x 1280 x 4096, 110 tiles: 24.7 against 26.1 us; 1536 x 1280 x 2048, 120:
    // 15.6 against 14.2; 1792^2 x 1024, 196: 11.8 against 13.2; 1536^2 x 1024, 144: 10.3 against 10.0)
    // (512 x 2304 x 8192, 72 tiles: 40.3 against 42.7; 2304 x 640 x 8192, 90: 41.3 against 46.8)
    return tiles >= (K >= 8192 ? 72 : K >= 4096 ? 100 : K >= 1536 ? 128 : 150) && tiles <= 256;
}

/// Whether AUTO sends an unsplit product to the 256 x 128 tile: at most 128 tiles of 256 x 256 (half of the chip or
/// more would idle), 128 x 128 tiles need two rounds of the K-splitting kernel, but 256 x 128 tiles fill one round
/// (2048 x 2560 x 4096: 45.9 against 59.1 us for the pipelined kernel, 3072 x 2560 x 4096: 57.0 against 67.3,
/// 4096 x 2048 x 8192: 106.5 against 134.7 us for 128 tiles of 256 x 256); a short K is left to the pipelined kernel's
/// ring.
bool gemm_narrow_is_the_choice(int M, int N, int K) {
    if (M % 16 != 0 || N % 16 != 0 || K % 64 != 0 || K < 1024 || (long)K * 512 >= (1l << 32)) return false;
    if (gemm_w128k_is_the_choice(M, N, K)) return false;
    const long narrow = (long)((M + 255) / 256) * ((N + 127) / 128);  // with edge tiles where M, N are not whole tiles
    return narrow > 128 && narrow <= 256;
}

/// Expected time of one launch, in us, of the kernels above where AUTO runs them (measured on whole-chip launches): the
/// K-splitting kernel 5 us + 0.95 us per 128 of K with 128 x 128 tiles, 0.75 us with 128 x 96 tiles; the 256 x 128 tile
/// 6 us + per 64 of K 0.70 us with up to 160 tiles, rising to 0.83 us with 256; 256 x 256 tiles 3 us + per 1024 of K
/// 23.5 us for every full round of 256 workgroups and, for a single round of t, 10.6 + 12.9 t / 256 us (the chip is
/// power-limited: fewer busy CUs run at a higher clock) but not below 17 us (what one workgroup needs by itself).
double gemm_w128k_us(int M, int N, int K) {
    const long rows = (M + 127) / 128;
    const long tiles128 = rows * ((N + 127) / 128), tiles96 = rows * ((N + 95) / 96);
    return 5.0 + (tiles128 <= 192 && tiles96 <= 256 ? 0.75 : 0.95) * (K / 128);
}

double gemm_narrow_us(int M, int N, int K) {
    const long narrow = (long)((M + 255) / 256) * ((N + 127) / 128);
    return 6.0 + (0.70 + 0.13 * (narrow > 160 ? double(narrow - 160) / 96.0 : 0.0)) * (K / 64);
}

double gemm_w128_us(long tiles, int K) {
    const long full = (tiles - 1) / 256, last = tiles - 256 * full;
    // a last round behind full ones starts unevenly (the XCDs differ by about 4 %) and runs beside their stragglers:
    // 13 to 23 us measured, rising with its fill (8192 x 8448, 7168^2, 6144^2, 2560 x 8192, 6976 x 8192)
    const double fill = last / 256.0;
    const double last_us = full == 0 ? std::max(17.0, 10.6 + 12.9 * fill) : std::min(23.5, 12.0 + 20.0 * fill);
    return 3.0 + (K / 1024.0) * (23.5 * full + last_us);
}

/// More than one round of 256 x 256 tiles, the last of them far from full (2560 x 8192: 320 tiles, the last 64 of which
/// cost as much again as the first 256): the leading rows (or columns) whose tiles fill whole rounds go to gemm_w128, the
/// rest of C to the kernel that fills the chip with smaller tiles - the K-splitting kernel (32 to 64 tiles of 256 x 256
/// left), the 256 x 128 tile (65 to 128 left), else the pipelined kernel. Two launches on disjoint parts of C
/// (2560 x 8192 x 4096: 134.6 against 166.3 us, 4352^2 x 4096: 127.8 against 164.1, 3072 x 6144 x 4096: 125.6 against
/// 160.9). M and N in multiples of 16: the split falls on a multiple of 256, every kernel involved has edge tiles.
/// The plan: the best split and what it is expected to cost (1e30: none).
struct GemmRoundsPlan {
    double us;
    int main_rows, main_cols;  // in tiles of 256; one of them is set
};

GemmRoundsPlan gemm_rounds_and_rest_plan(int M, int N, int K) {
    GemmRoundsPlan plan{1e30, 0, 0};
    if (M % 16 != 0 || N % 16 != 0 || K % 64 != 0 || (long)K * 512 >= (1l << 32)) return plan;
    const int tm = (M + 255) / 256, tn = (N + 255) / 256;
    const long tiles = (long)tm * tn;
    if (tiles <= 256 || tiles % 256 == 0) return plan;
    auto rest_us = [&](int Mr, int Nr) {
        if (gemm_w128k_is_the_choice(Mr, Nr, K)) return gemm_w128k_us(Mr, Nr, K);
        if (gemm_narrow_is_the_choice(Mr, Nr, K)) return gemm_narrow_us(Mr, Nr, K);
        return pipelined_plan(Mr, Nr, K).us;
    };
    for (int t = 1; t < tm; ++t) {
        const double us = gemm_w128_us((long)t * tn, K) + 2.0 + rest_us(M - 256 * t, N);
        if (us < plan.us) plan = {us, t, 0};
    }
    for (int t = 1; t < tn; ++t) {
        const double us = gemm_w128_us((long)t * tm, K) + 2.0 + rest_us(M, N - 256 * t);
        if (us < plan.us) plan = {us, 0, t};
    }
    return plan;
}

template <typename OutType>
int gemm_rounds_and_rest(const __half* A, const __half* B, OutType* C, int M, int N, int K, GemmRoundsPlan plan,
                         hipStream_t stream) {
    const int Mm = plan.main_rows ? 256 * plan.main_rows : M, Nm = plan.main_cols ? 256 * plan.main_cols : N;
    int rc = gemm_w128_dispatch<OutType>(A, B, C, Mm, Nm, K, stream, K, K, N);
    if (rc != TCU_OK) return rc;
    const __half* Ar = plan.main_rows ? A + size_t(Mm) * K : A;
    const __half* Br = plan.main_cols ? B + size_t(Nm) * K : B;
    OutType* Cr = plan.main_rows ? C + size_t(Mm) * N : C + Nm;
    const int Mr = plan.main_rows ? M - Mm : M, Nr = plan.main_cols ? N - Nm : N;
    if (gemm_w128k_is_the_choice(Mr, Nr, K)) return gemm_w128k_dispatch<OutType>(Ar, Br, Cr, Mr, Nr, K, stream, N);
    if (gemm_narrow_is_the_choice(Mr, Nr, K)) return gemm_w128_narrow_dispatch<OutType>(Ar, Br, Cr, Mr, Nr, K, stream, N);
    return gemm_pipelined_dispatch<OutType>(Ar, Br, Cr, Mr, Nr, K, stream, N);
}

/// How tcu_gemm_f16_ws runs a product: unsplit (splits == 1), or split over K into `splits` ranges whose f32 partial
/// products come from gemm_w128 (256 x 256 tiles) or from gemm_w128k (128 x 128 tiles: four times the workgroups per
/// range, so a quarter of the ranges - and of the partial products to write and add - fills the chip).
/// Split only if 256 x 256 tiles would leave at least half of the chip idle (at most 128 tiles), K gives every workgroup
/// at least 512 of it (1024 with 128 x 128 tiles), and the split is expected to beat the unsplit launch by 5 %. Expected
/// cost of s ranges (measured, one workgroup per CU at most): 10 us for the two launches and the epilogues + 1.4 us per
/// k-tile of a range + the partial products written and read once (2 x s x M x N x 4 bytes at 5.3 TB/s); of the unsplit
/// launch: pipelined_plan(), or the K-splitting kernel's time where AUTO would run it.
struct GemmSplitPlan {
    int splits;
    bool tiles128;
};

GemmSplitPlan gemm_split_plan(int M, int N, int K) {
    using T = GemmW128Traits;
    GemmSplitPlan plan{1, false};
    if (M % 16 != 0 || N % 16 != 0 || K % T::kBK != 0) return plan;
    const bool whole256 = M % T::kBM == 0 && N % T::kBN == 0;  // the 256 x 256 form splits whole tiles only
    const long tiles = (long)((M + T::kBM - 1) / T::kBM) * ((N + T::kBN - 1) / T::kBN);
    const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);  // (the 128 x 128 form has edge tiles)
    if (tiles > 128) return plan;
    double unsplit_us = pipelined_plan(M, N, K).us;
    // the kernels AUTO would run instead of the pipelined one
    if (gemm_w128k_is_the_choice(M, N, K)) unsplit_us = std::min(unsplit_us, gemm_w128k_us(M, N, K));
    if (gemm_narrow_is_the_choice(M, N, K)) unsplit_us = std::min(unsplit_us, gemm_narrow_us(M, N, K));
    double best_us = 0.95 * unsplit_us;
    const double plane_us = 2.0 * double(M) * N * 4 / 5.3e6;  // a plane of partial products written and read once
    for (int s = 2; whole256 && s * tiles <= 256 && K % (s * T::kBK) == 0 && K / s >= 512; s *= 2) {
        const double us = 10.0 + 1.4 * (K / s / T::kBK) + s * plane_us;
        if (us < best_us) {
            plan = {s, false};
            best_us = us;
        }
    }
    // partial products from the kernel whose wavefronts split K inside the workgroup: 8 us for the two launches, the
    // reduction through LDS and the epilogues + per 128 of a range 0.62 us with up to 128 workgroups, rising to 0.95 us
    // with 256 (their loads share the L2s) - measured on 256^2 x 8192 ... 1024 x 2048 x 16384 with 2 to 16 ranges
    if ((long)K * 256 < (1l << 32)) {
        for (int s = 2; s * tiles128 <= 256 && K % (s * 128) == 0 && K / s >= 512; s *= 2) {
            const long groups = s * tiles128;
            const double per_tile = 0.62 + 0.33 * (groups > 128 ? double(groups - 128) / 128.0 : 0.0);
            const double us = 8.0 + per_tile * (K / s / 128) + s * plane_us;
            if (us < best_us) {
                plan = {s, true};
                best_us = us;
            }
        }
    }
    return plan;
}

int gemm_split_count(int M, int N, int K) { return gemm_split_plan(M, N, K).splits; }

template <typename OutType>
int gemm_splitk(const __half* A, const __half* B, OutType* C, int M, int N, int K, GemmSplitPlan plan, float* partial,
                hipStream_t stream) {
    using T = GemmW128Traits;
    if ((long)K * 2 * T::kBM >= (1l << 32))
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the one-wavefront-per-SIMD GEMM addresses a 256-row panel with 32-bit offsets");
    int rc;
    if (plan.tiles128) {
        using Tk = GemmW128kTraits;
        const int tiles = ((M + Tk::kBM - 1) / Tk::kBM) * ((N + Tk::kBN - 1) / Tk::kBN);
        if (M % Tk::kBM == 0 && N % Tk::kBN == 0)
            rc = launch(&gemm_w128k<float, false, Tk>, dim3(tiles, plan.splits), dim3(Tk::kThreads), Tk::kLdsBytes, stream, A,
                        B, partial, M, N, K / plan.splits, K, K, N);
        else  // edge tiles: rows beyond M or N loaded from the last valid row, stores guarded
            rc = launch(&gemm_w128k<float, true, Tk>, dim3(tiles, plan.splits), dim3(Tk::kThreads), Tk::kLdsBytes, stream, A,
                        B, partial, M, N, K / plan.splits, K, K, N);
    } else {
        const int tiles = (M / T::kBM) * (N / T::kBN);
        rc = launch(&gemm_w128<float>, dim3(tiles, plan.splits), dim3(T::kThreads), T::kLdsBytes, stream, A, B, partial, M, N,
                    K / plan.splits, K, K, N, static_cast<unsigned int*>(nullptr), 0);
    }
    if (rc != TCU_OK) return rc;
    const size_t n = size_t(M) * N;
    return launch(&splitk_reduce<OutType>, dim3(unsigned((n / 4 + 255) / 256)), dim3(256), 0, stream,
                  static_cast<const float*>(partial), C, n, plan.splits);
}

template <typename OutType>
int gemm_ragged_dispatch(const __half* A, const __half* B, OutType* C, int M, int N, int K, hipStream_t stream) {
    using T = RaggedGemmTraits;
    if (M % 16 != 0 || N % 16 != 0 || K % 16 != 0)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "GEMM shapes are whole 16 x 16 tiles: M, N and K must be multiples of 16");
    const long grid = (long)((M + T::kBM - 1) / T::kBM) * ((N + T::kBN - 1) / T::kBN);
    if (grid > INT_MAX) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "GEMM: too many 64 x 64 blocks for one launch");
    return launch(&gemm_ragged<OutType>, dim3(unsigned(grid)), dim3(T::kThreads), 0, stream, A, B, C, M, N, K);
}

template <typename OutType>
int gemm_dispatch(const __half* A, const __half* B, OutType* C, int M, int N, int K, int algo, hipStream_t stream) {
    using W22 = tl::RowMajor<2, 2>;
    switch (algo) {
        case TCU_GEMM_TILE_PIPELINED:
            return gemm_tile_pipelined_dispatch<OutType>(A, B, C, M, N, K, stream);
        case TCU_GEMM_WAVE128:
            return gemm_w128_dispatch<OutType>(A, B, C, M, N, K, stream);
        case TCU_GEMM_TILE_WAVE128:
            return gemm_tile_w128_dispatch<OutType>(A, B, C, M, N, K, stream);
        case TCU_GEMM_WAVE128_KSPLIT:
            return gemm_w128k_dispatch<OutType>(A, B, C, M, N, K, stream);
        case TCU_GEMM_WAVE128_NARROW:
            return gemm_w128_narrow_dispatch<OutType>(A, B, C, M, N, K, stream);
        case TCU_GEMM_AUTO:
            // where the 256 x 256 tile is the choice anyway, the one-wavefront-per-SIMD kernel is the faster one
            if (M % 256 == 0 && N % 256 == 0 && K % 64 == 0 && (long)(M / 256) * (N / 256) > 128 &&
                (long)K * 512 < (1l << 32)) {
                // ... in one launch, or - where its last round would be far from full and the cost model expects 7 % -
                // on the leading rows or columns, with a second launch of smaller tiles on the rest of C
                const GemmRoundsPlan rounds = gemm_rounds_and_rest_plan(M, N, K);
                if (rounds.us < 0.93 * gemm_w128_us((long)(M / 256) * (N / 256), K))
                    return gemm_rounds_and_rest<OutType>(A, B, C, M, N, K, rounds, stream);
                return gemm_w128_dispatch<OutType>(A, B, C, M, N, K, stream);
            }
            // too few 256 x 256 tiles for the chip, but about one 128 x 128 tile per CU and a long enough K: the
            // kernel whose wavefronts split K (each owns the whole tile)
            if (gemm_w128k_is_the_choice(M, N, K)) return gemm_w128k_dispatch<OutType>(A, B, C, M, N, K, stream);
            // between the two: 256 x 128 tiles fill one round
            if (gemm_narrow_is_the_choice(M, N, K)) return gemm_w128_narrow_dispatch<OutType>(A, B, C, M, N, K, stream);
            if (M % 16 == 0 && N % 16 == 0) {
                // M or N not multiples of 256: the one-wavefront-per-SIMD kernel with edge tiles, that kernel on the
                // leading block of whole tiles plus the pipelined kernel on the strips beyond it, that kernel on the
                // rows or columns that fill whole rounds plus smaller tiles on the rest, or the pipelined kernel with the
                // tile its cost model picks - whichever is expected to be the shortest
                const long tiles_e = (long)((M + 255) / 256) * ((N + 255) / 256);
                const double edge_us = K % 16 == 0 && tiles_e >= 128 && (long)K * 512 < (1l << 32)
                                           ? gemm_w128_us(tiles_e, (K + 63) / 64 * 64) : 1e30;
                const GemmRoundsPlan rounds = gemm_rounds_and_rest_plan(M, N, K);
                const double rounds_us = rounds.us / 0.93;  // (two launches have to promise 7 % over the other plans)
                const int rc = gemm_main_and_strips<OutType>(A, B, C, M, N, K, stream, std::min(edge_us, rounds_us));
                if (rc != kPlanNotTaken) return rc;
                const double pipelined_us = pipelined_plan(M, N, K).us;
                if (rounds_us < edge_us && rounds_us < pipelined_us)
                    return gemm_rounds_and_rest<OutType>(A, B, C, M, N, K, rounds, stream);
                if (edge_us < pipelined_us) return gemm_w128_dispatch<OutType>(A, B, C, M, N, K, stream);
            }
            // tiny problems: the kernel that takes its operand tiles straight from global memory has the shorter start
            if ((long)M * N < 64 * 64) return gemm_ragged_dispatch<OutType>(A, B, C, M, N, K, stream);
            [[fallthrough]];
        case TCU_GEMM_PIPELINED:
            return gemm_pipelined_dispatch<OutType>(A, B, C, M, N, K, stream);
        case TCU_GEMM_RAGGED:
            return gemm_ragged_dispatch<OutType>(A, B, C, M, N, K, stream);
        case TCU_GEMM_GLOBAL_REG:
          if constexpr (std::is_same_v<OutType, float>) {
            if (M == 128 && N == 64 && K == 256)  // the README shape of the reference
                return launch_simple_gemm<OutType, 128, 64, 256, 128, 64, 32, W22>(A, B, C, stream);
            if (M == 1024 && N == 1024 && K == 2048)  // the driver shape of 01_gemm_global_reg/main.cu:105-106
                return launch_simple_gemm<OutType, 1024, 1024, 2048, 256, 128, 64, W22>(A, B, C, stream);
            return fail(TCU_ERR_UNSUPPORTED_SHAPE, "global->register GEMM is instantiated for 128x64x256 and "
                                                   "1024x1024x2048 only");
          }
          [[fallthrough]];
        case TCU_GEMM_ALL_MEM:
          if constexpr (std::is_same_v<OutType, float>) {
            if (algo == TCU_GEMM_ALL_MEM && M == 128 && N == 64 && K == 256)
                return launch_all_mem_gemm<OutType, 128, 64, 256, 64, 64, 64, 32, W22>(A, B, C, stream);
            if (algo == TCU_GEMM_ALL_MEM && M == 4096 && N == 4096 && K == 4096)  // the driver shape of 02_gemm_all_mem/main.cu:5-8
                return launch_all_mem_gemm<OutType, 4096, 4096, 4096, 64, 256, 32, 32, W22>(A, B, C, stream);
            return fail(TCU_ERR_UNSUPPORTED_SHAPE, "single-stage LDS GEMM is instantiated for 128x64x256 and "
                                                   "4096^3 only");
          }
          return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the reference-style GEMM kernels write f32 only");
        default:
            return fail(TCU_ERR_INVALID_ARGUMENT, "unknown GEMM algo");
    }
}

// ---------------------------------------------------------------------------- b2b GEMM
template <typename OutType, int kN, int kK, int kP, int kTM, int kTN, typename WarpLayout>
int launch_b2b(const __half* A, const __half* B, const __half* C, OutType* D, int M, int batch, hipStream_t stream) {
    using Traits = FusedGemmTraits<__half, float, OutType, FusedGemmShape<0, kN, kK, kP>,
                                   FusedGemmShape<kTM, kTN, kK, kP>, WarpLayout>;
    auto kernel = &KeFusedGemm<__half, OutType, Traits>;
    return launch(kernel, dim3(M / kTM, 1, batch), dim3(Traits::kThreads), Traits::kShmBytes, stream, A, B, C, D, M);
}

template <typename OutType, int kN, int kK = 128, int kP = 128, int kTN = 256, int kWaves = 8>
int launch_b2b_tile_resident(const __half* A, const __half* B, const __half* C, OutType* D, int M, int batch, hipStream_t stream) {
    using Traits = ResidentFusedGemmTraits<__half, OutType, kN, kK, kP, kTN, kWaves>;
    return launch(&b2b_gemm_tile_resident<__half, OutType, Traits>, dim3(M / Traits::kTM, batch), dim3(Traits::kThreads),
                  Traits::kShmBytes, stream, A, B, C, D, M);
}

template <typename OutType>
int b2b_dispatch(const __half* A, const __half* B, const __half* C, OutType* D, int M, int N, int K, int P, int batch,
                 int algo, hipStream_t stream) {
    if (algo != TCU_B2B_AUTO && algo != TCU_B2B_TILE_LIBRARY && algo != TCU_B2B_RESIDENT && algo != TCU_B2B_ROWS &&
        algo != TCU_B2B_TILE_RESIDENT)
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_b2b_gemm_f16: unknown algo");
    if (algo == TCU_B2B_TILE_RESIDENT) {
        // the LDS-resident kernel composed from tile-library functors: compile-time N, like every tile-API kernel
        if (K == 128 && P == 128 && M % 32 == 0) {
            if (N == 256) return launch_b2b_tile_resident<OutType, 256>(A, B, C, D, M, batch, stream);
            if (N == 1024) return launch_b2b_tile_resident<OutType, 1024>(A, B, C, D, M, batch, stream);
            if (N == 2048) return launch_b2b_tile_resident<OutType, 2048>(A, B, C, D, M, batch, stream);
        }
        if (K == 64 && P == 64 && M % 32 == 0) {
            if (N == 128) return launch_b2b_tile_resident<OutType, 128, 64, 64, 128, 4>(A, B, C, D, M, batch, stream);
            if (N == 256) return launch_b2b_tile_resident<OutType, 256, 64, 64, 128, 4>(A, B, C, D, M, batch, stream);
        }
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the tile-API LDS-resident b2b kernel is instantiated for K = P = 128 with N in "
                                               "{256, 1024, 2048} and for K = P = 64 with N in {128, 256}, M a multiple of 32");
    }
    // many rows: workgroups that keep both weight blocks for their whole life and walk over blocks of 256 rows
    if (algo == TCU_B2B_ROWS || (algo == TCU_B2B_AUTO && (long)M * batch >= 32768)) {
        if (N == 256 && K == 128 && P == 128 && M % 64 == 0) {
            using T = B2bRowsTraits;
            const int blocks = (M + T::kRowsPerBlock - 1) / T::kRowsPerBlock;
            const int per_item = std::max(1, 256 / batch);  // one workgroup per CU: about 256 in all
            return launch(&b2b_gemm_rows<OutType>, dim3(std::min(blocks, per_item), batch), dim3(T::kThreads), T::kLdsBytes,
                          stream, A, B, C, D, M);
        }
        if (algo == TCU_B2B_ROWS)
            return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the many-rows b2b kernel takes N = 256, K = P = 128 and M a multiple of 64");
    }
    if (algo != TCU_B2B_TILE_LIBRARY) {
        if (N % 256 == 0 && K == 128 && P == 128 && M % 32 == 0)
            return launch(&b2b_gemm_resident<OutType>, dim3(M / B2bResidentTraits::kTM, batch),
                          dim3(B2bResidentTraits::kThreads), B2bResidentTraits::kLdsBytes, stream, A, B, C, D, M, N);
        if (algo == TCU_B2B_RESIDENT)
            return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the LDS-resident b2b kernel takes K = P = 128, N a multiple of 256 "
                                                   "and M a multiple of 32");
    }
    // K = P = 64: the LDS-resident composition from tile-library functors is the fast kernel (direct-to-LDS loads, both
    // products split over the wavefronts): 2.2 against 3.0 us at the reference driver's (256, 128, 64, 64)
    if (algo == TCU_B2B_AUTO && K == 64 && P == 64 && M % 32 == 0) {
        if (N == 128) return launch_b2b_tile_resident<OutType, 128, 64, 64, 128, 4>(A, B, C, D, M, batch, stream);
        if (N == 256) return launch_b2b_tile_resident<OutType, 256, 64, 64, 128, 4>(A, B, C, D, M, batch, stream);
    }
    if (N == 256 && K == 128 && P == 128) {
        // 32-row tiles keep all 256 CUs busy up to M * batch = 8192; 64-row tiles beyond that
        if (M % 64 == 0 && (long)M * batch > 16384)
            return launch_b2b<OutType, 256, 128, 128, 64, 64, tl::RowMajor<4, 1>>(A, B, C, D, M, batch, stream);
        if (M % 32 == 0) return launch_b2b<OutType, 256, 128, 128, 32, 64, tl::RowMajor<2, 1>>(A, B, C, D, M, batch, stream);
    }
    if (N == 128 && K == 64 && P == 64 && M % 32 == 0)
        return launch_b2b<OutType, 128, 64, 64, 32, 64, tl::RowMajor<2, 1>>(A, B, C, D, M, batch, stream);
    if (N == 64 && K == 64 && P == 64 && M % 16 == 0)
        return launch_b2b<OutType, 64, 64, 64, 16, 32, tl::RowMajor<1, 1>>(A, B, C, D, M, batch, stream);
    // the rest of the shape list of the reference's driver (examples/cpp/02_fused_two_gemms/fused_gemm.cu:212-259),
    // with its tile shapes and warp layouts
    if (N == 16 && K == 16 && P == 16 && M % 16 == 0)
        return launch_b2b<OutType, 16, 16, 16, 16, 16, tl::RowMajor<1, 1>>(A, B, C, D, M, batch, stream);
    if (N == 32 && K == 16 && P == 32 && M % 16 == 0)
        return launch_b2b<OutType, 32, 16, 32, 16, 16, tl::RowMajor<1, 1>>(A, B, C, D, M, batch, stream);
    if (N == 64 && K == 32 && P == 64 && M % 32 == 0)
        return launch_b2b<OutType, 64, 32, 64, 32, 32, tl::RowMajor<2, 1>>(A, B, C, D, M, batch, stream);
    if (N == 1024 && K == 128 && P == 128 && M % 64 == 0)
        return launch_b2b<OutType, 1024, 128, 128, 64, 64, tl::RowMajor<4, 1>>(A, B, C, D, M, batch, stream);
    if (N == 2048 && K == 128 && P == 128 && M % 64 == 0)
        return launch_b2b<OutType, 2048, 128, 128, 64, 128, tl::RowMajor<4, 1>>(A, B, C, D, M, batch, stream);
    return fail(TCU_ERR_UNSUPPORTED_SHAPE,
                "the tile-library b2b GEMM is instantiated for (N, K, P) in {(16,16,16), (32,16,32), (64,32,64), (64,64,64), "
                "(128,64,64), (256,128,128), (1024,128,128), (2048,128,128)} with M a multiple of its row tile (16 ... 64); "
                "the LDS-resident kernel takes K = P = 128, N % 256 == 0, M % 32 == 0");
}

// ---------------------------------------------------------------------------- attention
template <int kNStatic, int kD, bool kVRowMajor, int kTM, int kTN, typename WarpLayout>
int launch_fa(const __half* Q, const __half* K, const __half* V, __half* O, int batch, int M, int N, float scale,
              hipStream_t stream) {
    using Traits = FlashAttentionTraits<__half, float, __half, FlashAttentionShape<0, kNStatic, kD, kD>,
                                        FlashAttentionShape<kTM, kTN, kD, kD>, kVRowMajor, WarpLayout>;
    auto kernel = &flash_attention<__half, __half, Traits>;
    return launch(kernel, dim3(M / kTM, 1, batch), dim3(Traits::kThreads), Traits::kShmBytes, stream, Q, K, V, O, M, N,
                  scale);
}

template <int kNStatic, int kD, bool kVRowMajor, int kTM, int kTN, typename WarpLayout>
int launch_fa_pipelined(const __half* Q, const __half* K, const __half* V, __half* O, int batch, int M, int N, float scale,
                        hipStream_t stream) {
    using Traits = FlashAttentionTraits<__half, float, __half, FlashAttentionShape<0, kNStatic, kD, kD>,
                                        FlashAttentionShape<kTM, kTN, kD, kD>, kVRowMajor, WarpLayout>;
    auto kernel = &flash_attention_pipelined<__half, __half, Traits>;
    return launch(kernel, dim3(M / kTM, 1, batch), dim3(Traits::kThreads), Traits::kShmBytesPipelined, stream, Q, K, V, O,
                  M, N, scale);
}

template <int kD, int kWaves, bool kFused>
int launch_fa_fwd(const __half* Q, const __half* K, const __half* V, __half* O, int batch, int M, int N, float scale,
                  hipStream_t stream) {
    using Traits = FlashFwdTraits<kD, kWaves, 64>;
    auto kernel = kFused ? &flash_attention_fwd_fused<Traits> : &flash_attention_fwd<Traits>;
    return launch(kernel, dim3((M / Traits::kBM) * batch), dim3(Traits::kThreads), Traits::kLdsBytes, stream, Q, K, V,
                  O, batch, M, N, scale);
}

template <bool kVColMajor>
int launch_fa_w64(const __half* Q, const __half* K, const __half* V, __half* O, int batch, int M, int N, float scale,
                  hipStream_t stream) {
    using Traits = FlashW64Traits<128>;
    if ((long)N * 256 >= (1l << 32))
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the one-wavefront-per-SIMD attention kernel addresses a V block with 32-bit offsets");
    return launch(&flash_attention_fwd_w64<Traits, kVColMajor>, dim3(((M + Traits::kBM - 1) / Traits::kBM) * batch),
                  dim3(Traits::kThreads), Traits::kLdsBytes, stream, Q, K, V, O, batch, M, N, scale);
}

template <int kM, int kN>
int launch_fa_tile_w64(const __half* Q, const __half* K, const __half* V, __half* O, int batch, float scale,
                       hipStream_t stream) {
    using Traits = FlashW64TileTraits<__half, kM, kN, 128>;
    return launch(&flash_attention_tile_w64<__half, Traits>, dim3((kM / Traits::kTM) * batch), dim3(Traits::kThreads),
                  Traits::kShmBytes, stream, Q, K, V, O, batch, scale);
}

/// The one-wavefront-per-SIMD kernel composed from tile-library functors: compile-time sequence lengths, like every
/// kernel written against the tile API (the benchmark shape and the shapes its tests use).
int fa_tile_w64_dispatch(const __half* Q, const __half* K, const __half* V, __half* O, int batch, int M, int N, int Kd,
                         float scale, int v_layout, hipStream_t stream) {
    if (Kd != 128 || v_layout != TCU_V_ROW_MAJOR)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the tile-API one-wavefront-per-SIMD attention kernel takes head size 128 and a row-major V");
    if (M == 2048 && N == 2048) return launch_fa_tile_w64<2048, 2048>(Q, K, V, O, batch, scale, stream);
    if (M == 512 && N == 1024) return launch_fa_tile_w64<512, 1024>(Q, K, V, O, batch, scale, stream);
    if (M == 256 && N == 640) return launch_fa_tile_w64<256, 640>(Q, K, V, O, batch, scale, stream);
    if (M == 256 && N == 320) return launch_fa_tile_w64<256, 320>(Q, K, V, O, batch, scale, stream);
    return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the tile-API one-wavefront-per-SIMD attention kernel is instantiated for "
                                           "(M, N) in {(2048, 2048), (512, 1024), (256, 640), (256, 320)}");
}

/// The one-wavefront-per-SIMD kernel on the 16x16x32 instruction (tile-library functors, run-time M and N, either V
/// layout).
template <int kD, bool kVColMajor>
int launch_fa_w64_k32(const __half* Q, const __half* K, const __half* V, __half* O, int batch, int M, int N, float scale,
                      hipStream_t stream) {
    using Traits = FlashW64K32Traits<__half, kD, kVColMajor>;
    // one workgroup per CU; a workgroup with more than one item fetches the next one's first operands under the last
    // steps of the current one. Items keep their XCD (item number modulo 8) only if the grid is a multiple of 8.
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus < 8)
        return fail(TCU_ERR_HIP, "attention: cannot read the number of compute units");
    const long items = (long)((M + Traits::kTM - 1) / Traits::kTM) * batch;
    const long grid = std::min<long>(items, cus - cus % 8);
    return launch(&flash_attention_w64_k32<__half, Traits>, dim3(unsigned(grid)), dim3(Traits::kThreads),
                  Traits::kShmBytes, stream, Q, K, V, O, batch, M, N, scale);
}

int fa_w64_k32_dispatch(const __half* Q, const __half* K, const __half* V, __half* O, int batch, int M, int N, int Kd,
                        float scale, int v_layout, hipStream_t stream) {
    using Traits = FlashW64K32Traits<__half, 128>;
    if (Kd != 128 && !(Kd == 64 && v_layout == TCU_V_ROW_MAJOR))
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the 16x16x32 one-wavefront-per-SIMD attention kernel is instantiated for head size "
                                               "128, and for head size 64 with a row-major V");
    if (N < Traits::kStages * Traits::kTN)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the 16x16x32 one-wavefront-per-SIMD attention kernel needs N >= 320");
    if ((long)N * 256 >= (1l << 32))
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the one-wavefront-per-SIMD attention kernel addresses a V block with 32-bit offsets");
    if (Kd == 64) return launch_fa_w64_k32<64, false>(Q, K, V, O, batch, M, N, scale, stream);
    return v_layout == TCU_V_ROW_MAJOR ? launch_fa_w64_k32<128, false>(Q, K, V, O, batch, M, N, scale, stream)
                                       : launch_fa_w64_k32<128, true>(Q, K, V, O, batch, M, N, scale, stream);
}

template <int kD, bool kFused>
int fa_fwd_by_rows(const __half* Q, const __half* K, const __half* V, __half* O, int batch, int M, int N, float scale,
                   hipStream_t stream) {
    if (M % 256 == 0) return launch_fa_fwd<kD, 8, kFused>(Q, K, V, O, batch, M, N, scale, stream);
    if (M % 128 == 0) return launch_fa_fwd<kD, 4, kFused>(Q, K, V, O, batch, M, N, scale, stream);
    return launch_fa_fwd<kD, 2, kFused>(Q, K, V, O, batch, M, N, scale, stream);
}

int fa_dispatch(const __half* Q, const __half* K, const __half* V, __half* O, int batch, int M, int N, int Kd, int P,
                float scale, int v_layout, int algo, hipStream_t stream) {
    using W41 = tl::RowMajor<4, 1>;
    if (Kd != P) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "attention needs the query and value head sizes equal");
    if (M % 64 != 0 || N % 64 != 0) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "attention needs M % 64 == 0 and N % 64 == 0");
    if (algo != TCU_ATTN_AUTO && algo != TCU_ATTN_TILE_LIBRARY && algo != TCU_ATTN_MFMA32 &&
        algo != TCU_ATTN_MFMA32_FUSED && algo != TCU_ATTN_WAVE64 && algo != TCU_ATTN_TILE_WAVE64 &&
        algo != TCU_ATTN_WAVE64_K32)
        return fail(TCU_ERR_INVALID_ARGUMENT, "unknown attention algo");
    if (v_layout != TCU_V_ROW_MAJOR && v_layout != TCU_V_COL_MAJOR) return fail(TCU_ERR_INVALID_ARGUMENT, "unknown v_layout");
    if (algo == TCU_ATTN_TILE_WAVE64) return fa_tile_w64_dispatch(Q, K, V, O, batch, M, N, Kd, scale, v_layout, stream);
    if (algo == TCU_ATTN_WAVE64_K32) return fa_w64_k32_dispatch(Q, K, V, O, batch, M, N, Kd, scale, v_layout, stream);
    if (algo == TCU_ATTN_WAVE64) {
        if (Kd != 128)
            return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the one-wavefront-per-SIMD attention kernel is instantiated for head size 128");
        return v_layout == TCU_V_ROW_MAJOR ? launch_fa_w64<false>(Q, K, V, O, batch, M, N, scale, stream)
                                           : launch_fa_w64<true>(Q, K, V, O, batch, M, N, scale, stream);
    }
    if (v_layout == TCU_V_ROW_MAJOR && algo != TCU_ATTN_TILE_LIBRARY) {
        if (Kd != 128 && Kd != 64) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "attention is instantiated for head sizes 64 and 128");
        // Enough query blocks to fill the chip: the kernels with 64 queries per wavefront. From one block of 256 queries
        // per CU on (counting a sequence's whole blocks; M is any multiple of 64) the chip runs at its power limit, where
        // the 16x16x32 instruction wins, at every sequence length that kernel takes (256 x 512 x 512 x 128: 45.6 against
        // 57.9 us for the 8-wavefront kernel, 1024 x 320 x 320: 117.7 against 203); a half-empty chip runs at full clock,
        // where the 32x32x16 kernel's fewer issue cycles do (long sequences, head size 128: 16 x 2048^2 45.7 against 48.8
        // us; with 192 blocks the 16x16x32 kernel is ahead again, 52.6 against 55.5).
        const long blocks = (long)batch * (M / 256);
        if (algo == TCU_ATTN_AUTO && N >= 320 && (blocks >= 256 || (blocks >= 192 && N >= 1024)))
            return fa_w64_k32_dispatch(Q, K, V, O, batch, M, N, Kd, scale, v_layout, stream);
        if (algo == TCU_ATTN_AUTO && Kd == 128 && N >= 1024 && blocks >= 128)
            return launch_fa_w64<false>(Q, K, V, O, batch, M, N, scale, stream);
        if (algo == TCU_ATTN_MFMA32)
            return Kd == 128 ? fa_fwd_by_rows<128, false>(Q, K, V, O, batch, M, N, scale, stream)
                             : fa_fwd_by_rows<64, false>(Q, K, V, O, batch, M, N, scale, stream);
        return Kd == 128 ? fa_fwd_by_rows<128, true>(Q, K, V, O, batch, M, N, scale, stream)
                         : fa_fwd_by_rows<64, true>(Q, K, V, O, batch, M, N, scale, stream);
    }
    if (algo == TCU_ATTN_MFMA32 || algo == TCU_ATTN_MFMA32_FUSED)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the 32x32x16 attention kernels take a row-major V");
    if (v_layout == TCU_V_ROW_MAJOR) {
        // row-major V: the double-buffered composition (direct-to-LDS ring); 32 query rows per wavefront where M allows
        if (Kd == 128 && M % 128 == 0) return launch_fa_pipelined<0, 128, true, 128, 64, W41>(Q, K, V, O, batch, M, N, scale, stream);
        if (Kd == 128) return launch_fa_pipelined<0, 128, true, 64, 64, W41>(Q, K, V, O, batch, M, N, scale, stream);
        if (Kd == 64) return launch_fa_pipelined<0, 64, true, 64, 64, W41>(Q, K, V, O, batch, M, N, scale, stream);
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "attention is instantiated for head sizes 64 and 128");
    }
    // column-major V (the reference op's convention), any N % 64 == 0
    if (Kd != 128) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "column-major V is instantiated for head size 128");
    if (algo == TCU_ATTN_AUTO) {
        // enough query blocks to fill the chip: the 16x16x32 kernel, as for a row-major V
        const long blocks = (long)batch * (M / 256);
        if (N >= 320 && (blocks >= 256 || (blocks >= 192 && N >= 1024)))
            return fa_w64_k32_dispatch(Q, K, V, O, batch, M, N, Kd, scale, v_layout, stream);
        return launch_fa_w64<true>(Q, K, V, O, batch, M, N, scale, stream);
    }
    // the kernel composed from tile primitives has the leading dimension of V (= N) as a compile-time constant, like
    // the reference op: one instantiation per N
    switch (N) {
        case 64: return launch_fa<64, 128, false, 64, 64, W41>(Q, K, V, O, batch, M, N, scale, stream);
        case 128: return launch_fa<128, 128, false, 64, 64, W41>(Q, K, V, O, batch, M, N, scale, stream);
        case 256: return launch_fa<256, 128, false, 64, 64, W41>(Q, K, V, O, batch, M, N, scale, stream);
        case 2048: return launch_fa<2048, 128, false, 64, 64, W41>(Q, K, V, O, batch, M, N, scale, stream);
        default:
            return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the tile-library attention kernel takes a column-major V for N in {64, 128, "
                                                   "256, 2048}");
    }
}

// ---------------------------------------------------------------------------- LSTM
template <int kI, int kH, int kTM, int kTH, int kTK, typename WarpLayout>
int launch_lstm(const __half* x, const __half* W, const __half* bias, const __half* h0, const float* c0,
                __half* h_all, float* c_out, int T, int B, hipStream_t stream) {
    using Traits = LstmCellTraits<__half, float, kI, kH, kTM, kTH, kTK, WarpLayout>;
    auto kernel = &lstm_cell<__half, Traits>;
    for (int t = 0; t < T; ++t) {
        const __half* x_t = x + size_t(t) * B * kI;
        const __half* h_in = t == 0 ? h0 : h_all + size_t(t - 1) * B * kH;
        const float* c_in = t == 0 ? c0 : c_out;
        __half* h_out = h_all + size_t(t) * B * kH;
        int rc = launch(kernel, dim3(B / kTM, kH / kTH), dim3(Traits::kThreads), Traits::kShmBytes, stream, x_t, h_in,
                        W, bias, c_in, c_out, h_out);
        if (rc != TCU_OK) return lstm_step_failed(rc, t, T);
    }
    return TCU_OK;
}

/// kI == kH == 0: the run-time-shape instantiation of the streaming kernel (I, H any multiples of 128).
template <int kI, int kH>
int launch_lstm_hoisted(const __half* x, const __half* W, const __half* bias, const __half* h0, const float* c0,
                        __half* h_all, float* c_out, int T, int B, int I, int H, float* pre, hipStream_t stream) {
    using Traits = LstmFwdTraits<kI, kH>;
    // pre[T * B, 4H] = x[T * B, I] . W[:, :I]^T: the stored [4H, I] operand is the first I columns of W's rows
    const long rows = long(T) * B;
    if (rows > INT_MAX) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "tcu_lstm_f16_ws: T * B exceeds the 32-bit row count");
    int rc = gemm_w128_dispatch<float>(x, W, pre, int(rows), 4 * H, I, stream, I, I + H);
    if (rc != TCU_OK) return rc;
    auto kernel = &lstm_cell_fwd<Traits, true>;
    const int grid = (B / Traits::kTM) * (H / Traits::kTH);
    for (int t = 0; t < T; ++t) {
        const __half* x_t = x + size_t(t) * B * I;
        const __half* h_in = t == 0 ? h0 : h_all + size_t(t - 1) * B * H;
        const float* c_in = t == 0 ? c0 : c_out;
        __half* h_out = h_all + size_t(t) * B * H;
        const float* pre_t = pre + size_t(t) * B * 4 * H;
        rc = launch(kernel, dim3(grid), dim3(Traits::kThreads), Traits::kLdsBytes, stream, x_t, h_in, W, bias, c_in,
                    c_out, h_out, B, pre_t, I, H);
        if (rc != TCU_OK) return lstm_step_failed(rc, t, T);
    }
    return TCU_OK;
}

int launch_lstm_ragged(const __half* x, const __half* W, const __half* bias, const __half* h0, const float* c0,
                       __half* h_all, float* c_out, int T, int B, int I, int H, hipStream_t stream) {
    using Traits = RaggedLstmTraits;
    const dim3 grid((H + Traits::kUnits - 1) / Traits::kUnits, B / Traits::kRows);
    for (int t = 0; t < T; ++t) {
        const __half* x_t = x + size_t(t) * B * I;
        const __half* h_in = t == 0 ? h0 : h_all + size_t(t - 1) * B * H;
        const float* c_in = t == 0 ? c0 : c_out;
        __half* h_out = h_all + size_t(t) * B * H;
        int rc = launch(&lstm_cell_ragged, grid, dim3(Traits::kThreads), 0, stream, x_t, h_in, W, bias, c_in, c_out, h_out,
                        B, I, H);
        if (rc != TCU_OK) return lstm_step_failed(rc, t, T);
    }
    return TCU_OK;
}

/// kI == kH == 0: the run-time-shape instantiation (I, H any multiples of 128).
template <int kI, int kH>
int launch_lstm_fwd(const __half* x, const __half* W, const __half* bias, const __half* h0, const float* c0,
                    __half* h_all, float* c_out, int T, int B, int I, int H, hipStream_t stream) {
    using Traits = LstmFwdTraits<kI, kH>;
    auto kernel = &lstm_cell_fwd<Traits>;
    const int grid = (B / Traits::kTM) * (H / Traits::kTH);
    for (int t = 0; t < T; ++t) {
        const __half* x_t = x + size_t(t) * B * I;
        const __half* h_in = t == 0 ? h0 : h_all + size_t(t - 1) * B * H;
        const float* c_in = t == 0 ? c0 : c_out;
        __half* h_out = h_all + size_t(t) * B * H;
        int rc = launch(kernel, dim3(grid), dim3(Traits::kThreads), Traits::kLdsBytes, stream, x_t, h_in, W, bias, c_in,
                        c_out, h_out, B, static_cast<const float*>(nullptr), I, H);
        if (rc != TCU_OK) return lstm_step_failed(rc, t, T);
    }
    return TCU_OK;
}

/// The weight-stationary recurrence for hidden size kH: 8 * kH / 32 workgroups, kH / 32 per XCD.
template <int kH>
int launch_lstm_recurrent_xcd(const __half* pre, const __half* W, const void* bias, const void* h0, const void* c0, void* h_all,
                              void* c_out, int T, int B, int I, unsigned int* sync, unsigned long long spin_us,
                              long peers_override, hipStream_t s) {
    using Traits = LstmRecurrentTraits<kH>;
    const unsigned int peers = peers_override >= 0 ? unsigned(peers_override) : unsigned(Traits::kCusPerXcd);
    return launch(&lstm_recurrent_xcd<Traits, __half>, dim3(Traits::kGrid), dim3(Traits::kThreads), Traits::kLdsBytes, s, pre,
                  W, I + kH, I, static_cast<const __half*>(bias), static_cast<const __half*>(h0),
                  static_cast<const float*>(c0), static_cast<__half*>(h_all), static_cast<float*>(c_out), T, B, sync,
                  spin_us * 100ull, peers);
}
}  // namespace

extern "C" {

int tcu_version(void) { return 100; }

const char* tcu_last_error(void) { return g_last_error.c_str(); }

int tcu_device_count(void) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) return fail(TCU_ERR_NO_DEVICE, std::string("hipGetDeviceCount: ") + hipGetErrorString(e));
    return n;
}

int tcu_gemm_f16(const void* A, const void* B, void* C, int M, int N, int K, int out_dtype, int algo, void* stream) {
    if (!A || !B || !C) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_gemm_f16: null pointer");
    if (!positive({M, N, K})) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_gemm_f16: sizes must be positive");
    if (!aligned16({A, B, C})) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_gemm_f16: operands must be 16-byte aligned");
    auto s = static_cast<hipStream_t>(stream);
    auto a = static_cast<const __half*>(A), b = static_cast<const __half*>(B);
    if (out_dtype == TCU_DTYPE_F32) return gemm_dispatch<float>(a, b, static_cast<float*>(C), M, N, K, algo, s);
    if (out_dtype == TCU_DTYPE_F16) {
        if (algo == TCU_GEMM_GLOBAL_REG || algo == TCU_GEMM_ALL_MEM)
            return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the reference-style GEMM kernels write f32 (their accumulator type)");
        return gemm_dispatch<__half>(a, b, static_cast<__half*>(C), M, N, K, algo, s);
    }
    return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_gemm_f16: out_dtype must be TCU_DTYPE_F32 or TCU_DTYPE_F16");
}

unsigned long long tcu_gemm_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const int splits = gemm_split_count(M, N, K);
    return splits > 1 ? (unsigned long long)splits * M * N * sizeof(float) : 0;
}

int tcu_gemm_f16_ws(const void* A, const void* B, void* C, int M, int N, int K, int out_dtype, void* workspace,
                    unsigned long long workspace_bytes, void* stream) {
    const unsigned long long need = (M > 0 && N > 0 && K > 0) ? tcu_gemm_workspace_bytes(M, N, K) : 0;
    if (need == 0 || !workspace) return tcu_gemm_f16(A, B, C, M, N, K, out_dtype, TCU_GEMM_AUTO, stream);
    if (!A || !B || !C) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_gemm_f16_ws: null pointer");
    if (!aligned16({A, B, C, workspace})) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_gemm_f16_ws: operands must be 16-byte aligned");
    if (workspace_bytes < need)
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_gemm_f16_ws: workspace smaller than tcu_gemm_workspace_bytes()");
    auto a = static_cast<const __half*>(A), b = static_cast<const __half*>(B);
    auto s = static_cast<hipStream_t>(stream);
    auto ws = static_cast<float*>(workspace);
    const GemmSplitPlan plan = gemm_split_plan(M, N, K);
    if (out_dtype == TCU_DTYPE_F32) return gemm_splitk<float>(a, b, static_cast<float*>(C), M, N, K, plan, ws, s);
    if (out_dtype == TCU_DTYPE_F16) return gemm_splitk<__half>(a, b, static_cast<__half*>(C), M, N, K, plan, ws, s);
    return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_gemm_f16_ws: out_dtype must be TCU_DTYPE_F32 or TCU_DTYPE_F16");
}

int tcu_b2b_gemm_f16(const void* A, const void* B, const void* C, void* D, int M, int N, int K, int P, int batch,
                     int out_dtype, void* stream) {
    return tcu_b2b_gemm_f16_algo(A, B, C, D, M, N, K, P, batch, out_dtype, TCU_B2B_AUTO, stream);
}

int tcu_b2b_gemm_f16_algo(const void* A, const void* B, const void* C, void* D, int M, int N, int K, int P, int batch,
                          int out_dtype, int algo, void* stream) {
    if (!A || !B || !C || !D) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_b2b_gemm_f16: null pointer");
    if (!positive({M, N, K, P, batch}))
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_b2b_gemm_f16: sizes must be positive");
    if (!aligned16({A, B, C, D}))
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_b2b_gemm_f16: operands must be 16-byte aligned");
    auto s = static_cast<hipStream_t>(stream);
    auto a = static_cast<const __half*>(A), b = static_cast<const __half*>(B), c = static_cast<const __half*>(C);
    if (out_dtype == TCU_DTYPE_F32) return b2b_dispatch<float>(a, b, c, static_cast<float*>(D), M, N, K, P, batch, algo, s);
    if (out_dtype == TCU_DTYPE_F16) return b2b_dispatch<__half>(a, b, c, static_cast<__half*>(D), M, N, K, P, batch, algo, s);
    return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_b2b_gemm_f16: out_dtype must be TCU_DTYPE_F32 or TCU_DTYPE_F16");
}

int tcu_flash_attn_fwd_f16_algo(const void* Q, const void* K, const void* V, void* O, int batch, int M, int N,
                                int Kdim, int P, float scale, int v_layout, int algo, void* stream) {
    if (!Q || !K || !V || !O) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_flash_attn_fwd_f16: null pointer");
    if (!positive({batch, M, N, Kdim, P}))
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_flash_attn_fwd_f16: sizes must be positive");
    if (!aligned16({Q, K, V, O}))
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_flash_attn_fwd_f16: operands must be 16-byte aligned");
    return fa_dispatch(static_cast<const __half*>(Q), static_cast<const __half*>(K), static_cast<const __half*>(V),
                       static_cast<__half*>(O), batch, M, N, Kdim, P, scale, v_layout, algo,
                       static_cast<hipStream_t>(stream));
}

int tcu_flash_attn_fwd_f16(const void* Q, const void* K, const void* V, void* O, int batch, int M, int N, int Kdim,
                           int P, float scale, int v_layout, void* stream) {
    return tcu_flash_attn_fwd_f16_algo(Q, K, V, O, batch, M, N, Kdim, P, scale, v_layout, TCU_ATTN_AUTO, stream);
}

int tcu_lstm_f16(const void* x, const void* W, const void* bias, const void* h0, const void* c0, void* h_all,
                 void* c_out, int T, int B, int I, int H, void* stream) {
    return tcu_lstm_f16_algo(x, W, bias, h0, c0, h_all, c_out, T, B, I, H, TCU_LSTM_AUTO, stream);
}

int tcu_lstm_f16_algo(const void* x, const void* W, const void* bias, const void* h0, const void* c0, void* h_all,
                      void* c_out, int T, int B, int I, int H, int algo, void* stream) {
    if (!x || !W || !bias || !h_all || !c_out) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16: null pointer");
    if (!positive({T, B, I, H})) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16: sizes must be positive");
    if (!aligned16({x, W, bias, h0, c0, h_all, c_out}))
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16: operands must be 16-byte aligned");
    auto s = static_cast<hipStream_t>(stream);
    auto xp = static_cast<const __half*>(x), wp = static_cast<const __half*>(W), bp = static_cast<const __half*>(bias);
    auto h0p = static_cast<const __half*>(h0);
    auto c0p = static_cast<const float*>(c0);
    auto hp = static_cast<__half*>(h_all);
    auto cp = static_cast<float*>(c_out);
    if (long(T) * B > INT_MAX) return fail(TCU_ERR_UNSUPPORTED_SHAPE, "tcu_lstm_f16: T * B exceeds the 32-bit row count");
    if (algo != TCU_LSTM_AUTO && algo != TCU_LSTM_TILE_LIBRARY && algo != TCU_LSTM_STREAMING && algo != TCU_LSTM_RAGGED)
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16: unknown algo");
    if (B % 16 != 0 || I % 16 != 0 || H % 16 != 0)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "tcu_lstm_f16: shapes are whole 16 x 16 tiles: B, I and H must be multiples of 16");
    if (algo == TCU_LSTM_RAGGED) return launch_lstm_ragged(xp, wp, bp, h0p, c0p, hp, cp, T, B, I, H, s);
    const bool b64 = B % 64 == 0;
    if (algo != TCU_LSTM_TILE_LIBRARY && b64 && I % 128 == 0 && H % 128 == 0) {
        // the benchmark shape with its sizes as constants; every other shape with the sizes as kernel arguments
        if (I == 1024 && H == 1024) return launch_lstm_fwd<1024, 1024>(xp, wp, bp, h0p, c0p, hp, cp, T, B, I, H, s);
        return launch_lstm_fwd<0, 0>(xp, wp, bp, h0p, c0p, hp, cp, T, B, I, H, s);
    }
    if (algo == TCU_LSTM_STREAMING)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "the streaming LSTM kernel needs I % 128 == 0, H % 128 == 0 and B % 64 == 0");
    if (b64) {
        if (I == 1024 && H == 1024)
            return launch_lstm<1024, 1024, 64, 16, 64, tl::RowMajor<4, 1>>(xp, wp, bp, h0p, c0p, hp, cp, T, B, s);
        if (I == 128 && H == 128)
            return launch_lstm<128, 128, 64, 16, 64, tl::RowMajor<4, 1>>(xp, wp, bp, h0p, c0p, hp, cp, T, B, s);
        if (I == 64 && H == 128)
            return launch_lstm<64, 128, 64, 16, 64, tl::RowMajor<4, 1>>(xp, wp, bp, h0p, c0p, hp, cp, T, B, s);
    }
    if (algo == TCU_LSTM_TILE_LIBRARY)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE,
                    "the tile-library LSTM kernel is instantiated for (I, H) in {(1024,1024), (128,128), (64,128)}, B % 64 == 0");
    // every other shape made of whole 16 x 16 tiles: the run-time-shape kernel
    return launch_lstm_ragged(xp, wp, bp, h0p, c0p, hp, cp, T, B, I, H, s);
}

unsigned long long tcu_lstm_workspace_bytes(int T, int B, int I, int H) {
    const bool shape_ok = I > 0 && H > 0 && I % 128 == 0 && H % 128 == 0 && (long)(I + H) * 512 < (1l << 32);
    if (!shape_ok || T <= 0 || B <= 0 || B % 64 != 0 || ((long)T * B) % 256 != 0) return 0;
    return (unsigned long long)T * B * 4 * H * sizeof(float);
}

int tcu_lstm_f16_ws(const void* x, const void* W, const void* bias, const void* h0, const void* c0, void* h_all,
                    void* c_out, int T, int B, int I, int H, void* workspace, unsigned long long workspace_bytes,
                    void* stream) {
    if (!x || !W || !bias || !h_all || !c_out || !workspace)
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_ws: null pointer");
    if (!positive({T, B, I, H})) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_ws: sizes must be positive");
    if (!aligned16({x, W, bias, h0, c0, h_all, c_out, workspace}))
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_ws: operands must be 16-byte aligned");
    const unsigned long long need = tcu_lstm_workspace_bytes(T, B, I, H);
    if (need == 0)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "tcu_lstm_f16_ws: needs I % 128 == 0, H % 128 == 0, B % 64 == 0 and "
                                               "T * B % 256 == 0");
    if (workspace_bytes < need)
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_ws: workspace smaller than tcu_lstm_workspace_bytes()");
    auto s = static_cast<hipStream_t>(stream);
    auto xp = static_cast<const __half*>(x), wp = static_cast<const __half*>(W), bp = static_cast<const __half*>(bias);
    auto h0p = static_cast<const __half*>(h0);
    auto c0p = static_cast<const float*>(c0);
    auto hp = static_cast<__half*>(h_all);
    auto cp = static_cast<float*>(c_out);
    auto pre = static_cast<float*>(workspace);
    if (I == 1024 && H == 1024) return launch_lstm_hoisted<1024, 1024>(xp, wp, bp, h0p, c0p, hp, cp, T, B, I, H, pre, s);
    return launch_lstm_hoisted<0, 0>(xp, wp, bp, h0p, c0p, hp, cp, T, B, I, H, pre, s);
}

unsigned long long tcu_lstm_persistent_workspace_bytes(int T, int B, int I, int H) {
    using Traits = LstmRecurrentTraits<1024>;
    if (T <= 0 || B <= 0 || I <= 0 || (H != 256 && H != 512 && H != 768 && H != 1024)) return 0;
    if (B % Traits::kRows != 0 || B > Traits::kRows * Traits::kXcds || I % 64 != 0) return 0;
    if ((long)T * B % 256 != 0 || (long)T * B > INT_MAX) return 0;
    // the pre-activations of all steps in f16: [T, B, 4H]
    return kPersistentSyncBytes + (unsigned long long)T * B * 4 * H * sizeof(__half);
}

int tcu_lstm_f16_persistent(const void* x, const void* W, const void* bias, const void* h0, const void* c0, void* h_all,
                            void* c_out, int T, int B, int I, int H, void* workspace, unsigned long long workspace_bytes,
                            void* stream) {
    using Traits = LstmRecurrentTraits<1024>;
    if (!x || !W || !bias || !h_all || !c_out || !workspace)
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_persistent: null pointer");
    if (!positive({T, B, I, H})) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_persistent: sizes must be positive");
    if (!aligned16({x, W, bias, h0, c0, h_all, c_out}) || reinterpret_cast<uintptr_t>(workspace) % 128 != 0)
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_persistent: operands must be 16-byte aligned, the workspace 128-byte aligned");
    const unsigned long long need = tcu_lstm_persistent_workspace_bytes(T, B, I, H);
    if (need == 0)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "tcu_lstm_f16_persistent: needs H in {256, 512, 768, 1024}, I % 64 == 0, B % 32 == 0, "
                                               "B <= 256 and T * B % 256 == 0");
    if (workspace_bytes < need)
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_persistent: workspace smaller than tcu_lstm_persistent_workspace_bytes()");
    // one workgroup per CU, all resident at once, H / 32 per XCD (dealt to the 8 XCDs in turn): at H = 1024 the grid is
    // the chip
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
        return fail(TCU_ERR_NO_DEVICE, "tcu_lstm_f16_persistent: no current HIP device");
    if (cus != Traits::kGrid)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "tcu_lstm_f16_persistent: written for a device of 256 CUs in 8 XCDs; this one has " +
                                                   std::to_string(cus) + " CUs");
    unsigned long long spin_us = 2000000;  // a wait is microseconds when every workgroup is resident
    long peers = -1;                       // (the number of workgroups per XCD)
    if (const char* e = std::getenv("TCU_LSTM_PERSISTENT_SPIN_US")) spin_us = std::strtoull(e, nullptr, 10);
    if (const char* e = std::getenv("TCU_LSTM_PERSISTENT_PEERS")) peers = long(std::strtoul(e, nullptr, 10));
    auto s = static_cast<hipStream_t>(stream);
    auto sync = static_cast<unsigned int*>(workspace);
    auto pre = reinterpret_cast<__half*>(static_cast<unsigned char*>(workspace) + kPersistentSyncBytes);
    auto xp = static_cast<const __half*>(x), wp = static_cast<const __half*>(W);
    // The projection GEMM writes the pre-activations as f16 (f32 sums rounded once: half the bytes written here and read
    // by the recurrence, where the f32 form of tcu_lstm_f16_ws is bound by the volume of that write) and clears the
    // synchronisation words on the side (its first workgroup): no launch of its own.
    int rc = gemm_w128_dispatch<__half>(xp, wp, pre, T * B, 4 * H, I, s, I, I + H, 0, sync, Traits::kSyncWords);
    if (rc != TCU_OK) return rc;
    switch (H) {
        case 256: return launch_lstm_recurrent_xcd<256>(pre, wp, bias, h0, c0, h_all, c_out, T, B, I, sync, spin_us, peers, s);
        case 512: return launch_lstm_recurrent_xcd<512>(pre, wp, bias, h0, c0, h_all, c_out, T, B, I, sync, spin_us, peers, s);
        case 768: return launch_lstm_recurrent_xcd<768>(pre, wp, bias, h0, c0, h_all, c_out, T, B, I, sync, spin_us, peers, s);
        default: return launch_lstm_recurrent_xcd<1024>(pre, wp, bias, h0, c0, h_all, c_out, T, B, I, sync, spin_us, peers, s);
    }
}

int tcu_lstm_persistent_status(const void* workspace, void* stream) {
    if (!workspace) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_persistent_status: null pointer");
    auto s = static_cast<hipStream_t>(stream);
    unsigned int word = 0;
    hipError_t e = hipStreamSynchronize(s);
    if (e == hipSuccess)
        e = hipMemcpy(&word, static_cast<const unsigned int*>(workspace) + LstmRecurrentTraits<1024>::kErrorWord, sizeof(word),
                      hipMemcpyDeviceToHost);
    if (e != hipSuccess) return fail(TCU_ERR_HIP, std::string("tcu_lstm_persistent_status: ") + hipGetErrorString(e));
    if (word == 1)
        return fail(TCU_ERR_INCOMPLETE, "tcu_lstm_f16_persistent: workgroups that exchange h through an L2 were placed on different XCDs; the outputs are invalid");
    if (word != 0)
        return fail(TCU_ERR_INCOMPLETE, "tcu_lstm_f16_persistent: a workgroup waited for its XCD longer than the limit (the grid "
                                    "was not resident at once); the outputs are invalid");
    return TCU_OK;
}

unsigned long long tcu_lstm_noalloc_max_bytes(void) { return kScratchBytes; }

int tcu_lstm_f16_noalloc(const void* x, const void* W, const void* bias, const void* h0, const void* c0, void* h_all,
                         void* c_out, int T, int B, int I, int H, void* stream) {
    if (!x || !W || !bias || !h_all || !c_out) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_noalloc: null pointer");
    if (!positive({T, B, I, H})) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_noalloc: sizes must be positive");
    if (!aligned16({x, W, bias, h0, c0, h_all, c_out}))
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_lstm_f16_noalloc: operands must be 16-byte aligned");
    const unsigned long long need = tcu_lstm_workspace_bytes(T, B, I, H);
    if (need == 0)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE, "tcu_lstm_f16_noalloc: needs I % 128 == 0, H % 128 == 0, B % 64 == 0 and "
                                               "T * B % 256 == 0");
    if (need > kScratchBytes)
        return fail(TCU_ERR_UNSUPPORTED_SHAPE,
                    "tcu_lstm_f16_noalloc: the gate pre-activations need " + std::to_string(need) +
                        " bytes, more than the library's static scratch buffer of " + std::to_string(kScratchBytes) +
                        " bytes (T * B * 4H * 4 must not exceed it); use tcu_lstm_f16_ws with a caller-owned workspace");
    void* ws = nullptr;
    if (int rc = scratch_address(&ws); rc != TCU_OK) return rc;
    return tcu_lstm_f16_ws(x, W, bias, h0, c0, h_all, c_out, T, B, I, H, ws, kScratchBytes, stream);
}

int tcu_scatter_nd(void* data, const void* updates, const void* indices, const long long* data_dims, int rank,
                   long long n, int k, int dtype, int mode, void* skipped_rows, void* stream) {
    using namespace tiledcuda::kernels;
    if (!data || !updates || !indices || !data_dims) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_scatter_nd: null pointer");
    if (rank <= 0 || rank > kScatterMaxRank || k <= 0 || k > rank)
        return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_scatter_nd: need 0 < k <= rank <= 8");
    if (n < 0) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_scatter_nd: negative row count");
    if (dtype != TCU_DTYPE_F32 && dtype != TCU_DTYPE_F16) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_scatter_nd: dtype must be f32 or f16");
    if (mode != TCU_SCATTER_ASSIGN && mode != TCU_SCATTER_ADD) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_scatter_nd: unknown mode");
    ScatterNdShape shape{};
    int64_t stride = 1;
    for (int d = rank - 1; d >= 0; --d) {
        if (data_dims[d] <= 0) return fail(TCU_ERR_INVALID_ARGUMENT, "tcu_scatter_nd: dimensions must be positive");
        if (d < k) {
            shape.strides[d] = stride;
            shape.dims[d] = data_dims[d];
        }
        stride *= data_dims[d];
    }
    shape.slice = 1;
    for (int d = k; d < rank; ++d) shape.slice *= data_dims[d];
    shape.n = n;
    shape.k = k;
    if (n == 0) return TCU_OK;
    auto s = static_cast<hipStream_t>(stream);
    auto idx = static_cast<const int64_t*>(indices);
    auto bad = static_cast<unsigned int*>(skipped_rows);
    const size_t elem = dtype == TCU_DTYPE_F32 ? 4 : 2;
    const int vec = int(16 / elem);
    const bool vec_ok = mode == TCU_SCATTER_ASSIGN && shape.slice % vec == 0 &&
                        reinterpret_cast<uintptr_t>(data) % 16 == 0 && reinterpret_cast<uintptr_t>(updates) % 16 == 0;
    const int64_t lanes = n * (vec_ok ? shape.slice / vec : shape.slice);
    // enough workgroups to fill the chip several times over; the kernel strides over the rest
    const int64_t want = (lanes + 255) / 256;
    const dim3 grid(static_cast<unsigned>(want < 1 ? 1 : (want > 256 * 64 ? 256 * 64 : want))), block(256);
    auto go = [&](auto* dptr, auto kernel) {
        using T = std::remove_pointer_t<decltype(dptr)>;
        return launch(kernel, grid, block, 0, s, dptr, static_cast<const T*>(updates), idx, shape, bad);
    };
    if (dtype == TCU_DTYPE_F32) {
        auto* d = static_cast<float*>(data);
        if (mode == TCU_SCATTER_ADD) return go(d, &scatter_nd_kernel<float, 1, ScatterMode::kAdd>);
        return vec_ok ? go(d, &scatter_nd_kernel<float, 4, ScatterMode::kAssign>)
                      : go(d, &scatter_nd_kernel<float, 1, ScatterMode::kAssign>);
    }
    auto* d = static_cast<__half*>(data);
    if (mode == TCU_SCATTER_ADD) return go(d, &scatter_nd_kernel<__half, 1, ScatterMode::kAdd>);
    return vec_ok ? go(d, &scatter_nd_kernel<__half, 8, ScatterMode::kAssign>)
                  : go(d, &scatter_nd_kernel<__half, 1, ScatterMode::kAssign>);
}

}  // extern "C"
