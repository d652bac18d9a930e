// A C++ host program on the C-ABI of the tile-kernel library (include/tcu_c_api.h): allocates device memory with the
// HIP runtime, launches a configuration through the library's extern "C" entry points, checks the GEMM-shaped ones
// against the vendor library (rocBLAS; the role cuBLAS plays in the reference's drivers), times warm-up + iterations
// with HIP events and prints vendor time, this library's time and their ratio.
// The counterpart of the reference's drivers examples/cpp/01_gemm/01_gemm_global_reg/main.cu:10-107,
// examples/cpp/01_gemm/02_gemm_all_mem/main.cu:10-116, examples/cpp/02_fused_two_gemms/fused_gemm.cu:17-262 and
// examples/cpp/03_flash_attention/main.cu; host code only (no kernels here: compiled by the host compiler).
//
//   host_driver <config> [--in DIR] [--out DIR] [--iters N] [--warmup N] [--no-vendor]
//   config: gemm_c1 | gemm_c2 | b2b_c3 | attn_c4 | lstm_c5 | all
//   --in DIR   read the operands from DIR/<config>.<operand>.bin (raw arrays, the layouts of tcu_c_api.h) instead of
//              generating them here
//   --out DIR  write the result of the first launch to DIR/<config>.<output>.bin
// Without --in the operands are pseudo-random (a 64-bit LCG; uniform[-1, 1] for the GEMMs, a sum of uniforms scaled
// to the stated deviation elsewhere): enough for timing and for the comparison with the vendor library.
#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <functional>
#include <iomanip>
#include <iostream>
#include <string>
#include <vector>

#include "tcu_c_api.h"

namespace {

struct Options {
    std::string in_dir, out_dir;
    int iters = 20, warmup = 10;  // the reference drivers' counts (02_gemm_all_mem/main.cu:91-99)
    bool vendor = true;
};

#define HIP_OK(expr)                                                                                   \
    do {                                                                                               \
        hipError_t e_ = (expr);                                                                        \
        if (e_ != hipSuccess) {                                                                        \
            std::fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); \
            std::exit(2);                                                                              \
        }                                                                                              \
    } while (0)

#define TCU_OK_OR_DIE(expr)                                                              \
    do {                                                                                 \
        int rc_ = (expr);                                                                \
        if (rc_ != TCU_OK) {                                                             \
            std::fprintf(stderr, "%s: status %d: %s\n", #expr, rc_, tcu_last_error());   \
            std::exit(3);                                                                \
        }                                                                                \
    } while (0)

#define ROCBLAS_OK(expr)                                                             \
    do {                                                                             \
        rocblas_status s_ = (expr);                                                  \
        if (s_ != rocblas_status_success) {                                          \
            std::fprintf(stderr, "%s: %s\n", #expr, rocblas_status_to_string(s_));   \
            std::exit(4);                                                            \
        }                                                                            \
    } while (0)

// ---- host-side f16 (the host compiler has no arithmetic on __half; the conversions below are exact / round to nearest even)
uint16_t f32_to_f16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return uint16_t(sign | 0x7e00u);   // NaN
    if (ax >= 0x47800000u) return uint16_t(sign | 0x7c00u);  // 65536 and beyond, infinity
    if (ax >= 0x38800000u) {
        // normal f16 range: round the 13 dropped bits to nearest even, re-bias the exponent (a carry out of the
        // mantissa moves to the next exponent, up to infinity, which is the correct result)
        ax += ((ax >> 13) & 1u) + 0xfffu;
        return uint16_t(sign | ((ax - (112u << 23)) >> 13));
    }
    // subnormal f16 range: adding 0.5 aligns the mantissa's last bit with 2^-24, the addition itself rounds
    float a;
    std::memcpy(&a, &ax, 4);
    a += 0.5f;
    uint32_t bits;
    std::memcpy(&bits, &a, 4);
    return uint16_t(sign | (bits - 0x3f000000u));
}

float f16_to_f32(uint16_t h) {
    const uint32_t sign = uint32_t(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else {
            int e = -1;
            do {
                ++e;
                man <<= 1;
            } while (!(man & 0x400u));
            x = sign | uint32_t(127 - 15 - e) << 23 | (man & 0x3ffu) << 13;
        }
    } else if (exp == 31) {
        x = sign | 0x7f800000u | man << 13;
    } else {
        x = sign | (exp + 112) << 23 | man << 13;
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

struct Lcg {
    uint64_t s;
    explicit Lcg(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 1) {}
    double uniform() {  // [0, 1)
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        return double(s >> 11) * (1.0 / 9007199254740992.0);
    }
};

std::vector<uint16_t> fill_uniform_f16(size_t n, uint64_t seed) {
    Lcg g(seed);
    std::vector<uint16_t> v(n);
    for (auto& x : v) x = f32_to_f16(float(2.0 * g.uniform() - 1.0));
    return v;
}

/// Approximately normal (sum of 12 uniforms), mean 0.
std::vector<uint16_t> fill_normal_f16(size_t n, uint64_t seed, double sigma) {
    Lcg g(seed);
    std::vector<uint16_t> v(n);
    for (auto& x : v) {
        double s = -6.0;
        for (int i = 0; i < 12; ++i) s += g.uniform();
        x = f32_to_f16(float(s * sigma));
    }
    return v;
}

bool read_file(const std::string& path, void* dst, size_t bytes) {
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    f.read(static_cast<char*>(dst), std::streamsize(bytes));
    return size_t(f.gcount()) == bytes;
}

void write_file(const std::string& path, const void* src, size_t bytes) {
    std::ofstream f(path, std::ios::binary);
    f.write(static_cast<const char*>(src), std::streamsize(bytes));
    if (!f) {
        std::fprintf(stderr, "cannot write %s\n", path.c_str());
        std::exit(5);
    }
}

/// An operand: generated here, or read from <in_dir>/<config>.<name>.bin when --in is given.
std::vector<uint16_t> operand(const Options& opt, const std::string& config, const std::string& name, size_t n,
                              const std::function<std::vector<uint16_t>()>& generate) {
    if (opt.in_dir.empty()) return generate();
    std::vector<uint16_t> v(n);
    const std::string path = opt.in_dir + "/" + config + "." + name + ".bin";
    if (!read_file(path, v.data(), n * 2)) {
        std::fprintf(stderr, "cannot read %zu bytes from %s\n", n * 2, path.c_str());
        std::exit(5);
    }
    return v;
}

template <typename T>
struct DeviceBuffer {
    T* ptr = nullptr;
    size_t n = 0;
    explicit DeviceBuffer(size_t count) : n(count) { HIP_OK(hipMalloc(reinterpret_cast<void**>(&ptr), count * sizeof(T))); }
    explicit DeviceBuffer(const std::vector<T>& host) : DeviceBuffer(host.size()) {
        HIP_OK(hipMemcpy(ptr, host.data(), n * sizeof(T), hipMemcpyHostToDevice));
    }
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    ~DeviceBuffer() { (void)hipFree(ptr); }
    std::vector<T> to_host() const {
        std::vector<T> h(n);
        HIP_OK(hipMemcpy(h.data(), ptr, n * sizeof(T), hipMemcpyDeviceToHost));
        return h;
    }
};

/// Average milliseconds per call of `launch` over `iters` calls after `warmup` calls, by HIP events on `stream`.
float time_ms(const Options& opt, hipStream_t stream, const std::function<void()>& launch) {
    for (int i = 0; i < opt.warmup; ++i) launch();
    HIP_OK(hipStreamSynchronize(stream));
    hipEvent_t start, stop;
    HIP_OK(hipEventCreate(&start));
    HIP_OK(hipEventCreate(&stop));
    HIP_OK(hipEventRecord(start, stream));
    for (int i = 0; i < opt.iters; ++i) launch();
    HIP_OK(hipEventRecord(stop, stream));
    HIP_OK(hipEventSynchronize(stop));
    float ms = 0.f;
    HIP_OK(hipEventElapsedTime(&ms, start, stop));
    HIP_OK(hipEventDestroy(start));
    HIP_OK(hipEventDestroy(stop));
    return ms / float(opt.iters);
}

void report(const std::string& config, double flop, double bytes, float vendor_ms, float ours_ms) {
    std::cout << std::setprecision(4);
    if (vendor_ms > 0.f) {
        std::cout << "rocBLAS(ms)\ttiledcuda_amd(ms)\tRatio\n" << vendor_ms << "\t" << ours_ms << "\t" << ours_ms / vendor_ms << "\n";
    } else {
        std::cout << "tiledcuda_amd(ms)\n" << ours_ms << "\n";
    }
    std::cout << config << ": " << flop / (ours_ms * 1e-3) * 1e-12 << " TFLOP/s, " << bytes / (ours_ms * 1e-3) * 1e-9
              << " GB/s of algorithmic bytes" << std::endl;
}

/// max |x - ref| / max(|ref|, eps * rms(ref)): elementwise relative error with a floor, so that outputs that happen to
/// lie next to zero do not dominate.
double max_rel_err(const std::vector<float>& x, const std::vector<float>& ref, double eps) {
    double ss = 0.0;
    for (float r : ref) ss += double(r) * r;
    const double floor_v = eps * std::sqrt(ss / double(ref.size()));
    double worst = 0.0;
    for (size_t i = 0; i < ref.size(); ++i) {
        const double d = std::fabs(double(x[i]) - ref[i]) / std::max(std::fabs(double(ref[i])), floor_v);
        if (!(d <= worst)) worst = d;  // NaN propagates
    }
    return worst;
}

std::vector<float> widen(const std::vector<uint16_t>& h) {
    std::vector<float> f(h.size());
    for (size_t i = 0; i < h.size(); ++i) f[i] = f16_to_f32(h[i]);
    return f;
}

/// C[M, N] (row-major, f16 or f32) = A[M, K] (row-major) x B (column-major, stored [N, K]) with rocBLAS: in its
/// column-major terms C^T[N, M] = op_T(B_stored as K x N, ld K) x (A_stored as K x M, ld K).
void vendor_gemm(rocblas_handle handle, const void* A, const void* B, void* C, int M, int N, int K, bool f16_out,
                 int batch = 1, long stride_a = 0, long stride_b = 0, long stride_c = 0) {
    const float alpha = 1.f, beta = 0.f;
    const rocblas_datatype out = f16_out ? rocblas_datatype_f16_r : rocblas_datatype_f32_r;
    if (batch == 1) {
        ROCBLAS_OK(rocblas_gemm_ex(handle, rocblas_operation_transpose, rocblas_operation_none, N, M, K, &alpha, B,
                                   rocblas_datatype_f16_r, K, A, rocblas_datatype_f16_r, K, &beta, C, out, N, C, out, N,
                                   rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0));
    } else {
        ROCBLAS_OK(rocblas_gemm_strided_batched_ex(handle, rocblas_operation_transpose, rocblas_operation_none, N, M, K,
                                                   &alpha, B, rocblas_datatype_f16_r, K, stride_b, A, rocblas_datatype_f16_r,
                                                   K, stride_a, &beta, C, out, N, stride_c, C, out, N, stride_c, batch,
                                                   rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0));
    }
}

// ---------------------------------------------------------------------------- configurations
int run_gemm(const Options& opt, const std::string& config, int M, int N, int K, bool f16_out, rocblas_handle handle,
             hipStream_t stream) {
    std::cout << "== " << config << ": C[" << M << ", " << N << "] = A[" << M << ", " << K << "] . B[" << K << ", " << N
              << "], f16 in, " << (f16_out ? "f16" : "f32") << " out" << std::endl;
    const auto hA = operand(opt, config, "A", size_t(M) * K, [&] { return fill_uniform_f16(size_t(M) * K, 1); });
    const auto hB = operand(opt, config, "B", size_t(N) * K, [&] { return fill_uniform_f16(size_t(N) * K, 2); });
    DeviceBuffer<uint16_t> dA(hA), dB(hB);
    const size_t out_bytes = size_t(M) * N * (f16_out ? 2 : 4);
    DeviceBuffer<unsigned char> dC(out_bytes), dC2(out_bytes);
    const int dtype = f16_out ? TCU_DTYPE_F16 : TCU_DTYPE_F32;
    auto ours = [&] { TCU_OK_OR_DIE(tcu_gemm_f16(dA.ptr, dB.ptr, dC.ptr, M, N, K, dtype, TCU_GEMM_AUTO, stream)); };
    ours();
    HIP_OK(hipStreamSynchronize(stream));
    const auto hC = dC.to_host();
    if (!opt.out_dir.empty()) write_file(opt.out_dir + "/" + config + ".C.bin", hC.data(), out_bytes);
    bool passed = true;
    float vendor_ms = 0.f;
    if (opt.vendor) {
        auto theirs = [&] { vendor_gemm(handle, dA.ptr, dB.ptr, dC2.ptr, M, N, K, f16_out); };
        theirs();
        HIP_OK(hipStreamSynchronize(stream));
        const auto hC2 = dC2.to_host();
        std::vector<float> x(size_t(M) * N), ref(size_t(M) * N);
        for (size_t i = 0; i < x.size(); ++i) {
            if (f16_out) {
                x[i] = f16_to_f32(reinterpret_cast<const uint16_t*>(hC.data())[i]);
                ref[i] = f16_to_f32(reinterpret_cast<const uint16_t*>(hC2.data())[i]);
            } else {
                x[i] = reinterpret_cast<const float*>(hC.data())[i];
                ref[i] = reinterpret_cast<const float*>(hC2.data())[i];
            }
        }
        // both sides round an f32 sum to f16 (2^-11 each) and sum in different orders
        const double err = max_rel_err(x, ref, 0.01), tol = f16_out ? 2e-3 : 1e-3;
        passed = err <= tol;
        std::cout << "max rel err vs rocBLAS " << err << (passed ? ": Test passed." : ": Test failed.") << std::endl;
        if (passed) vendor_ms = time_ms(opt, stream, theirs);
    }
    if (!passed) return 1;
    const float ours_ms = time_ms(opt, stream, ours);
    report(config, 2.0 * M * N * K, 2.0 * (double(M) * K + double(N) * K) + double(out_bytes), vendor_ms, ours_ms);
    return 0;
}

int run_b2b(const Options& opt, const std::string& config, int M, int N, int K, int P, int batch, rocblas_handle handle,
            hipStream_t stream) {
    std::cout << "== " << config << ": D[" << M << ", " << P << "] = (A[" << M << ", " << K << "] . B[" << K << ", " << N
              << "]) . C[" << N << ", " << P << "], batch " << batch << ", f16" << std::endl;
    const size_t nA = size_t(batch) * M * K, nB = size_t(batch) * N * K, nC = size_t(batch) * P * N, nD = size_t(batch) * M * P;
    const auto hA = operand(opt, config, "A", nA, [&] { return fill_normal_f16(nA, 11, 0.1); });
    const auto hB = operand(opt, config, "B", nB, [&] { return fill_normal_f16(nB, 12, 0.1); });
    const auto hC = operand(opt, config, "C", nC, [&] { return fill_normal_f16(nC, 13, 0.1); });
    DeviceBuffer<uint16_t> dA(hA), dB(hB), dC(hC), dD(nD), dD2(nD), dAcc(size_t(batch) * M * N);
    auto ours = [&] {
        TCU_OK_OR_DIE(tcu_b2b_gemm_f16(dA.ptr, dB.ptr, dC.ptr, dD.ptr, M, N, K, P, batch, TCU_DTYPE_F16, stream));
    };
    ours();
    HIP_OK(hipStreamSynchronize(stream));
    const auto hD = dD.to_host();
    if (!opt.out_dir.empty()) write_file(opt.out_dir + "/" + config + ".D.bin", hD.data(), nD * 2);
    bool passed = true;
    float vendor_ms = 0.f;
    if (opt.vendor) {
        // two vendor GEMMs with the intermediate rounded to f16 in memory (the reference's cublas_two_gemms,
        // examples/cpp/02_fused_two_gemms/util.hpp:31-75)
        auto theirs = [&] {
            vendor_gemm(handle, dA.ptr, dB.ptr, dAcc.ptr, M, N, K, true, batch, long(M) * K, long(N) * K, long(M) * N);
            vendor_gemm(handle, dAcc.ptr, dC.ptr, dD2.ptr, M, P, N, true, batch, long(M) * N, long(P) * N, long(M) * P);
        };
        theirs();
        HIP_OK(hipStreamSynchronize(stream));
        const double err = max_rel_err(widen(hD), widen(dD2.to_host()), 1.0);
        passed = err <= 2e-3;
        std::cout << "max err vs two rocBLAS GEMMs (relative to rms) " << err << (passed ? ": passed." : ": failed.") << std::endl;
        if (passed) vendor_ms = time_ms(opt, stream, theirs);
    }
    if (!passed) return 1;
    const float ours_ms = time_ms(opt, stream, ours);
    report(config, 2.0 * batch * M * N * (double(K) + P), 2.0 * double(nA + nB + nC + nD), vendor_ms, ours_ms);
    return 0;
}

int run_attention(const Options& opt, const std::string& config, int batch, int S, int D, hipStream_t stream) {
    std::cout << "== " << config << ": softmax(Q K^T / sqrt(" << D << ")) V, " << batch << " heads of [" << S << ", " << D
              << "], f16, row-major V" << std::endl;
    const size_t n = size_t(batch) * S * D;
    const auto hQ = operand(opt, config, "Q", n, [&] { return fill_normal_f16(n, 21, 1.0); });
    const auto hK = operand(opt, config, "K", n, [&] { return fill_normal_f16(n, 22, 1.0); });
    const auto hV = operand(opt, config, "V", n, [&] { return fill_normal_f16(n, 23, 1.0); });
    DeviceBuffer<uint16_t> dQ(hQ), dK(hK), dV(hV), dO(n);
    const float scale = 1.0f / std::sqrt(float(D));
    auto ours = [&] {
        TCU_OK_OR_DIE(tcu_flash_attn_fwd_f16(dQ.ptr, dK.ptr, dV.ptr, dO.ptr, batch, S, S, D, D, scale, TCU_V_ROW_MAJOR, stream));
    };
    ours();
    HIP_OK(hipStreamSynchronize(stream));
    const auto hO = dO.to_host();
    if (!opt.out_dir.empty()) write_file(opt.out_dir + "/" + config + ".O.bin", hO.data(), n * 2);
    // a property the host can check without a second implementation: every output row is a convex combination of V
    // rows, so it lies inside the per-column range of that head's V
    int bad = 0;
    for (int b = 0; b < batch && bad == 0; ++b) {
        std::vector<float> lo(D, 1e30f), hi(D, -1e30f);
        for (int r = 0; r < S; ++r)
            for (int d = 0; d < D; ++d) {
                const float v = f16_to_f32(hV[(size_t(b) * S + r) * D + d]);
                lo[d] = std::min(lo[d], v);
                hi[d] = std::max(hi[d], v);
            }
        for (int r = 0; r < S; ++r)
            for (int d = 0; d < D; ++d) {
                const float o = f16_to_f32(hO[(size_t(b) * S + r) * D + d]);
                if (!(o >= lo[d] - 1e-2f && o <= hi[d] + 1e-2f)) ++bad;
            }
    }
    std::cout << (bad == 0 ? "outputs inside the range of V: passed." : "outputs outside the range of V: failed.") << std::endl;
    if (bad != 0) return 1;
    const float ours_ms = time_ms(opt, stream, ours);
    report(config, 4.0 * batch * double(S) * S * D, 8.0 * double(n), 0.f, ours_ms);
    return 0;
}

int run_lstm(const Options& opt, const std::string& config, int T, int B, int I, int H, hipStream_t stream) {
    std::cout << "== " << config << ": LSTM layer, " << T << " steps, batch " << B << ", input " << I << ", hidden " << H
              << ", hoisted input projection" << std::endl;
    const size_t nx = size_t(T) * B * I, nW = size_t(4) * H * (I + H);
    const auto hx = operand(opt, config, "x", nx, [&] { return fill_normal_f16(nx, 31, 0.05); });
    const auto hW = operand(opt, config, "W", nW, [&] { return fill_normal_f16(nW, 32, 0.05); });
    const auto hb = operand(opt, config, "b", size_t(4) * H, [&] { return fill_normal_f16(size_t(4) * H, 33, 0.05); });
    DeviceBuffer<uint16_t> dx(hx), dW(hW), db(hb), dh(size_t(T) * B * H);
    DeviceBuffer<float> dc(size_t(B) * H);
    const unsigned long long ws_bytes = tcu_lstm_workspace_bytes(T, B, I, H);
    DeviceBuffer<unsigned char> ws(ws_bytes ? ws_bytes : 16);
    auto ours = [&] {
        if (ws_bytes)
            TCU_OK_OR_DIE(tcu_lstm_f16_ws(dx.ptr, dW.ptr, db.ptr, nullptr, nullptr, dh.ptr, dc.ptr, T, B, I, H, ws.ptr, ws_bytes, stream));
        else
            TCU_OK_OR_DIE(tcu_lstm_f16(dx.ptr, dW.ptr, db.ptr, nullptr, nullptr, dh.ptr, dc.ptr, T, B, I, H, stream));
    };
    ours();
    HIP_OK(hipStreamSynchronize(stream));
    const auto hh = dh.to_host();
    const auto hc = dc.to_host();
    if (!opt.out_dir.empty()) {
        write_file(opt.out_dir + "/" + config + ".h_all.bin", hh.data(), hh.size() * 2);
        write_file(opt.out_dir + "/" + config + ".c_T.bin", hc.data(), hc.size() * 4);
    }
    // |h| < 1 always (o * tanh(c) with o in (0, 1))
    int bad = 0;
    for (uint16_t v : hh) bad += !(std::fabs(f16_to_f32(v)) < 1.0f);
    std::cout << (bad == 0 ? "|h| < 1 everywhere: passed." : "|h| >= 1 or not a number somewhere: failed.") << std::endl;
    if (bad != 0) return 1;
    const float ours_ms = time_ms(opt, stream, ours);
    const double step_bytes = 2.0 * 4 * H * (I + H) + 2.0 * 4 * H + 2.0 * B * I + 2.0 * 2 * B * H + 4.0 * 2 * B * H;
    report(config, 2.0 * T * B * double(I + H) * 4 * H, T * step_bytes, 0.f, ours_ms);
    std::cout << config << ": " << ours_ms * 1e3 / T << " us per step" << std::endl;
    return 0;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc < 2) {
        std::fprintf(stderr, "usage: %s gemm_c1|gemm_c2|b2b_c3|attn_c4|lstm_c5|all [--in DIR] [--out DIR] [--iters N] "
                             "[--warmup N] [--no-vendor]\n", argv[0]);
        return 64;
    }
    const std::string which = argv[1];
    Options opt;
    for (int i = 2; i < argc; ++i) {
        const std::string a = argv[i];
        auto value = [&]() -> const char* {
            if (i + 1 >= argc) {
                std::fprintf(stderr, "%s needs a value\n", a.c_str());
                std::exit(64);
            }
            return argv[++i];
        };
        if (a == "--in") opt.in_dir = value();
        else if (a == "--out") opt.out_dir = value();
        else if (a == "--iters") opt.iters = std::atoi(value());
        else if (a == "--warmup") opt.warmup = std::atoi(value());
        else if (a == "--no-vendor") opt.vendor = false;
        else {
            std::fprintf(stderr, "unknown option %s\n", a.c_str());
            return 64;
        }
    }
    if (opt.iters <= 0 || opt.warmup < 0) {
        std::fprintf(stderr, "--iters must be positive, --warmup non-negative\n");
        return 64;
    }
    if (tcu_device_count() <= 0) {
        std::fprintf(stderr, "no HIP device: %s\n", tcu_last_error());
        return 2;
    }
    std::cout << "tiledcuda_amd C-ABI version " << tcu_version() << std::endl;
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    rocblas_handle handle = nullptr;
    if (opt.vendor) {
        ROCBLAS_OK(rocblas_create_handle(&handle));
        ROCBLAS_OK(rocblas_set_stream(handle, stream));
    }
    int failures = 0;
    bool known = false;
    auto selected = [&](const char* name) {
        const bool yes = which == "all" || which == name;
        known |= yes;
        return yes;
    };
    if (selected("gemm_c1")) failures += run_gemm(opt, "gemm_c1", 128, 64, 256, false, handle, stream);
    if (selected("gemm_c2")) failures += run_gemm(opt, "gemm_c2", 4096, 4096, 4096, true, handle, stream);
    if (selected("b2b_c3")) failures += run_b2b(opt, "b2b_c3", 8192, 256, 128, 128, 1, handle, stream);
    if (selected("attn_c4")) failures += run_attention(opt, "attn_c4", 64, 2048, 128, stream);
    if (selected("lstm_c5")) failures += run_lstm(opt, "lstm_c5", 16, 256, 1024, 1024, stream);
    if (!known) {
        std::fprintf(stderr, "unknown configuration %s\n", which.c_str());
        failures = 64;
    }
    if (handle) ROCBLAS_OK(rocblas_destroy_handle(handle));
    HIP_OK(hipStreamDestroy(stream));
    return failures;
}
