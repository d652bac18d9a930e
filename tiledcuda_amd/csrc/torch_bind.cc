// torch.ops.tiledcuda.* registered from C++: the counterpart of the reference's src/torch_bind.cc:8-11
// (TORCH_LIBRARY(tiledcuda, t) with scatter_nd and flash_attention_fwd), built against PyTorch-ROCm, so that a C++
// program (or Python, through torch.ops.load_library) gets the operators without the Python mirror.
// Same two operators with the same names, argument order and in-place outputs, plus gemm, b2b_gemm and lstm for the
// other kernel entries. Every implementation checks dtype, device, contiguity and shapes (TORCH_CHECK; the reference
// checks nothing), then calls the C-ABI (include/tcu_c_api.h) on torch's current stream of the operands' device.
// Nothing synchronises the device (the reference op launches on stream 0 and calls cudaDeviceSynchronize(),
// src/kernels/flash_attn.cu:418-421). Unsupported shapes raise (c10::Error -> RuntimeError in Python), as the
// reference's std::runtime_error does (:453-455). There is no CPU implementation.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <tuple>
#include <vector>

#include "tcu_c_api.h"

namespace {

void* current_stream(const at::Tensor& t) {
    return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

void check_status(int status, const char* op) {
    TORCH_CHECK(status == TCU_OK, "tiledcuda::", op, ": ", tcu_last_error(), " (status ", status, ")");
}

void check_operand(const at::Tensor& t, const char* name, at::ScalarType dtype, const at::Tensor& like) {
    TORCH_CHECK(t.is_cuda(), name, " must live in device memory");
    TORCH_CHECK(t.scalar_type() == dtype, name, " must be ", dtype, ", got ", t.scalar_type());
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    TORCH_CHECK(t.device() == like.device(), name, " must be on the same device as the first operand");
}

int out_code(const at::Tensor& t, const char* name) {
    if (t.scalar_type() == at::kFloat) return TCU_DTYPE_F32;
    if (t.scalar_type() == at::kHalf) return TCU_DTYPE_F16;
    TORCH_CHECK(false, name, " must be float32 or float16");
}

// data[indices[i, 0], ..., indices[i, k-1], ...] = updates[i, ...]; argument order of the reference op
void scatter_nd(at::Tensor& data, const at::Tensor& updates, const at::Tensor& indices) {
    TORCH_CHECK(indices.dim() >= 1, "indices must be [..., k]");
    const int64_t k = indices.size(-1), rank = data.dim();
    TORCH_CHECK(k >= 1 && k <= rank && rank <= 8, "scatter_nd needs 1 <= k <= rank(data) <= 8");
    const int dtype = out_code(data, "data");
    check_operand(data, "data", data.scalar_type(), data);
    check_operand(updates, "updates", data.scalar_type(), data);
    check_operand(indices, "indices", at::kLong, data);
    const int64_t n = indices.numel() / k;
    int64_t slice = 1;
    for (int64_t d = k; d < rank; ++d) slice *= data.size(d);
    TORCH_CHECK(updates.numel() == n * slice, "updates must have one slice data.shape[k:] per index row");
    std::vector<long long> dims(data.sizes().begin(), data.sizes().end());
    c10::hip::HIPGuardMasqueradingAsCUDA guard(data.device());
    check_status(tcu_scatter_nd(data.data_ptr(), updates.data_ptr(), indices.data_ptr(), dims.data(), int(rank), n, int(k),
                                dtype, TCU_SCATTER_ASSIGN, nullptr, current_stream(data)),
                 "scatter_nd");
}

// flattened f16 tensors: Q [m, k], K stored [n, k], V stored [p, n] (column-major V), O [m, p]; scale 1 (the reference's)
void flash_attention_fwd(const at::Tensor& Q, const at::Tensor& K, const at::Tensor& V, at::Tensor& O, int64_t m,
                         int64_t n, int64_t k, int64_t p) {
    TORCH_CHECK(m > 0 && n > 0 && k > 0 && p > 0, "m, n, k and p must be positive");
    check_operand(Q, "Q", at::kHalf, Q);
    check_operand(K, "K", at::kHalf, Q);
    check_operand(V, "V", at::kHalf, Q);
    check_operand(O, "O", at::kHalf, Q);
    TORCH_CHECK(Q.numel() == m * k, "Q must hold m * k elements");
    TORCH_CHECK(K.numel() == n * k, "K must hold n * k elements");
    TORCH_CHECK(V.numel() == p * n, "V must hold p * n elements");
    TORCH_CHECK(O.numel() == m * p, "O must hold m * p elements");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(Q.device());
    check_status(tcu_flash_attn_fwd_f16(Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), 1, int(m), int(n), int(k),
                                        int(p), 1.0f, TCU_V_COL_MAJOR, current_stream(Q)),
                 "flash_attention_fwd");
}

// C[M, N] = A[M, K] . B with B column-major, stored [N, K]
void gemm(const at::Tensor& A, const at::Tensor& B, at::Tensor& C) {
    TORCH_CHECK(A.dim() == 2 && B.dim() == 2 && C.dim() == 2, "A [M, K], B [N, K] and C [M, N] must be matrices");
    check_operand(A, "A", at::kHalf, A);
    check_operand(B, "B", at::kHalf, A);
    const int code = out_code(C, "C");
    check_operand(C, "C", C.scalar_type(), A);
    TORCH_CHECK(A.size(1) == B.size(1), "mismatched K dimension");
    TORCH_CHECK(C.size(0) == A.size(0) && C.size(1) == B.size(0), "C must be [M, N]");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(A.device());
    const int M = int(A.size(0)), N = int(B.size(0)), K = int(A.size(1));
    // few output tiles and a long K: split over K through a workspace from torch's caching allocator (stream-ordered:
    // the block goes back to the allocator when `ws` dies and is reused on this stream only after the work enqueued here)
    const unsigned long long need = tcu_gemm_workspace_bytes(M, N, K);
    if (need > 0) {
        at::Tensor ws = at::empty({static_cast<int64_t>(need)}, A.options().dtype(at::kByte));
        check_status(tcu_gemm_f16_ws(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, code, ws.data_ptr(), need,
                                     current_stream(A)),
                     "gemm");
        return;
    }
    check_status(tcu_gemm_f16(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, code, TCU_GEMM_AUTO, current_stream(A)),
                 "gemm");
}

// D = f16(A . B) . C per batch item: A [b, M, K], B stored [b, N, K], C stored [b, P, N], D [b, M, P] (or all 2-D)
void b2b_gemm(const at::Tensor& A, const at::Tensor& B, const at::Tensor& C, at::Tensor& D) {
    const bool batched = A.dim() == 3;
    TORCH_CHECK((A.dim() == 2 || batched) && B.dim() == A.dim() && C.dim() == A.dim(),
                "operands must all be 2-D or all be 3-D (batched)");
    check_operand(A, "A", at::kHalf, A);
    check_operand(B, "B", at::kHalf, A);
    check_operand(C, "C", at::kHalf, A);
    const int code = out_code(D, "D");
    check_operand(D, "D", D.scalar_type(), A);
    const int64_t o = batched ? 1 : 0, batch = batched ? A.size(0) : 1;
    const int64_t M = A.size(o), K = A.size(o + 1), N = B.size(o), P = C.size(o);
    TORCH_CHECK(B.size(o + 1) == K && C.size(o + 1) == N && (!batched || (B.size(0) == batch && C.size(0) == batch)),
                "operand shapes do not chain: A [b, M, K], B [b, N, K], C [b, P, N]");
    TORCH_CHECK(D.numel() == batch * M * P && D.size(-1) == P && D.size(-2) == M, "D must be [b, M, P]");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(A.device());
    check_status(tcu_b2b_gemm_f16(A.data_ptr(), B.data_ptr(), C.data_ptr(), D.data_ptr(), int(M), int(N), int(K), int(P),
                                  int(batch), code, current_stream(A)),
                 "b2b_gemm");
}

// x [T, B, I], W [4H, I + H] (gate rows i, f, g, o), bias [4H], h0 [B, H] f16 / c0 [B, H] f32 or None -> (h_all, c_T)
std::tuple<at::Tensor, at::Tensor> lstm(const at::Tensor& x, const at::Tensor& W, const at::Tensor& bias,
                                        const std::optional<at::Tensor>& h0, const std::optional<at::Tensor>& c0) {
    TORCH_CHECK(x.dim() == 3 && W.dim() == 2 && bias.dim() == 1, "x must be [T, B, I], W [4H, I+H] and bias [4H]");
    check_operand(x, "x", at::kHalf, x);
    check_operand(W, "W", at::kHalf, x);
    check_operand(bias, "bias", at::kHalf, x);
    const int64_t T = x.size(0), B = x.size(1), I = x.size(2), H = W.size(0) / 4;
    TORCH_CHECK(W.size(0) == 4 * H && W.size(1) == I + H && bias.size(0) == 4 * H, "W must be [4H, I+H] and bias [4H]");
    const void* h0p = nullptr;
    const void* c0p = nullptr;
    if (h0.has_value()) {
        check_operand(*h0, "h0", at::kHalf, x);
        TORCH_CHECK(h0->dim() == 2 && h0->size(0) == B && h0->size(1) == H, "h0 must be [B, H]");
        h0p = h0->data_ptr();
    }
    if (c0.has_value()) {
        check_operand(*c0, "c0", at::kFloat, x);
        TORCH_CHECK(c0->dim() == 2 && c0->size(0) == B && c0->size(1) == H, "c0 must be [B, H]");
        c0p = c0->data_ptr();
    }
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    at::Tensor h_all = at::empty({T, B, H}, x.options());
    at::Tensor c_out = at::empty({B, H}, x.options().dtype(at::kFloat));
    // with a long input size the input half of the gates is cheaper as one GEMM over all steps; its [T, B, 4H] f32
    // result lives in a block from torch's caching allocator (stream-ordered, returned when `ws` dies)
    const unsigned long long need = tcu_lstm_workspace_bytes(int(T), int(B), int(I), int(H));
    if (need > 0 && I >= 512 && T >= 4) {
        at::Tensor ws = at::empty({static_cast<int64_t>(need)}, x.options().dtype(at::kByte));
        check_status(tcu_lstm_f16_ws(x.data_ptr(), W.data_ptr(), bias.data_ptr(), h0p, c0p, h_all.data_ptr(), c_out.data_ptr(),
                                     int(T), int(B), int(I), int(H), ws.data_ptr(), need, current_stream(x)),
                     "lstm");
        return {h_all, c_out};
    }
    check_status(tcu_lstm_f16(x.data_ptr(), W.data_ptr(), bias.data_ptr(), h0p, c0p, h_all.data_ptr(), c_out.data_ptr(),
                              int(T), int(B), int(I), int(H), current_stream(x)),
                 "lstm");
    return {h_all, c_out};
}

}  // namespace

TORCH_LIBRARY(tiledcuda, m) {
    m.def("scatter_nd(Tensor(a!) data, Tensor updates, Tensor indices) -> ()");
    m.def("flash_attention_fwd(Tensor Q, Tensor K, Tensor V, Tensor(a!) O, int m, int n, int k, int p) -> ()");
    m.def("gemm(Tensor A, Tensor B, Tensor(a!) C) -> ()");
    m.def("b2b_gemm(Tensor A, Tensor B, Tensor C, Tensor(a!) D) -> ()");
    m.def("lstm(Tensor x, Tensor W, Tensor bias, Tensor? h0, Tensor? c0) -> (Tensor, Tensor)");
}

TORCH_LIBRARY_IMPL(tiledcuda, CUDA, m) {
    m.impl("scatter_nd", &scatter_nd);
    m.impl("flash_attention_fwd", &flash_attention_fwd);
    m.impl("gemm", &gemm);
    m.impl("b2b_gemm", &b2b_gemm);
    m.impl("lstm", &lstm);
}
