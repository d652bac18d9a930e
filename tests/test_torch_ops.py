"""torch.ops.tiledcuda.* : the reference's operator library (src/torch_bind.cc:8-11) on PyTorch-ROCm.
CPU part: the ops exist with the reference's names and argument order and have no CPU implementation.
GPU part: the reference's Python tests restated (tests/python/test_flash_attn.py:113-161 shapes through
TiledFlashAttention-style operands; tests/python/test_scatter_nd.py:22-56), results checked against the oracle."""
import random

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def ops(tcu):
    import tiledcuda_amd.torch_ops as torch_ops  # noqa: F401  (registers the library)

    return torch.ops.tiledcuda


def test_ops_are_registered_with_the_reference_schemas(ops):
    assert str(ops.scatter_nd.default._schema) == \
        "tiledcuda::scatter_nd(Tensor(a!) data, Tensor updates, Tensor indices) -> ()"
    assert str(ops.flash_attention_fwd.default._schema) == \
        "tiledcuda::flash_attention_fwd(Tensor Q, Tensor K, Tensor V, Tensor(a!) O, int m, int n, int k, int p) -> ()"
    for name in ("gemm", "b2b_gemm", "lstm"):
        assert hasattr(ops, name)


def test_ops_come_from_the_cpp_library(ops):
    """The registrations live in a shared library built from C++ (csrc/torch_bind.cc, the counterpart of the reference's
    src/torch_bind.cc), loaded with torch.ops.load_library, as the reference's Python package does."""
    import os

    import tiledcuda_amd.torch_ops as torch_ops

    path = torch_ops.library_path()
    assert os.path.basename(path) == "libtiledcuda_torch.so" and os.path.exists(path)
    assert path in torch.ops.loaded_libraries
    blob = open(path, "rb").read()
    assert b"tcu_flash_attn_fwd_f16" in blob and b"tcu_scatter_nd" in blob  # it calls the C-ABI, nothing else


def test_ops_have_no_cpu_fallback(ops):
    with pytest.raises(NotImplementedError):
        ops.gemm(torch.zeros(64, 64, dtype=torch.float16), torch.zeros(64, 64, dtype=torch.float16),
                 torch.zeros(64, 64, dtype=torch.float16))
    with pytest.raises(NotImplementedError):
        ops.scatter_nd(torch.zeros(4, 4), torch.zeros(1, 4), torch.zeros(1, 1, dtype=torch.int64))


@pytest.mark.gpu
@pytest.mark.parametrize("n", [64, 128, 256])
def test_flash_attention_fwd_op_reference_shapes(ops, oracle, device, n):
    """m = 64, k = p = 128, n in {64, 128, 256}: Q [m, k], K [k, n], V [n, p] drawn as the reference test draws
    them, handed to the op the way pytiledcuda.TiledFlashAttention does (K and V transposed, flattened); scale 1.
    Tolerance: the reference's own 8e-2 is far too loose; 1e-2 absolute against fp32 attention."""
    torch.manual_seed(1234)
    m, k, p = 64, 128, 128
    Q, Kmat, V = torch.randn(m, k), torch.randn(k, n), torch.randn(n, p)
    q = Q.half().flatten().to(device)
    key = Kmat.half().t().contiguous().flatten().to(device)
    val = V.half().t().contiguous().flatten().to(device)
    out = torch.empty(m * p, dtype=torch.half, device=device)
    ops.flash_attention_fwd(q, key, val, out, m, n, k, p)
    ref = oracle.attention(Q.half().numpy(), Kmat.half().t().contiguous().numpy(), V.half().numpy(), 1.0)
    assert oracle.max_abs_err(out.view(m, p).float().cpu().numpy(), ref) <= 1e-2


@pytest.mark.gpu
def test_cpp_ops_check_their_operands(ops, device):
    """dtype / shape / contiguity mistakes are refused by the C++ layer (TORCH_CHECK -> RuntimeError) before any
    pointer reaches a kernel; the reference op checks nothing."""
    h = dict(dtype=torch.half, device=device)
    a = torch.zeros(64, 64, **h)
    with pytest.raises(RuntimeError, match="must be"):
        ops.gemm(a.float(), a, torch.zeros(64, 64, **h))
    with pytest.raises(RuntimeError, match="mismatched K"):
        ops.gemm(a, torch.zeros(64, 32, **h), torch.zeros(64, 64, **h))
    with pytest.raises(RuntimeError, match=r"C must be \[M, N\]"):
        ops.gemm(a, a, torch.zeros(64, 32, **h))
    with pytest.raises(RuntimeError, match="contiguous"):
        ops.gemm(a.t(), a, torch.zeros(64, 64, **h))
    q = torch.zeros(64 * 128, **h)
    with pytest.raises(RuntimeError, match="K must hold"):
        ops.flash_attention_fwd(q, q[:-128], q, q, 64, 64, 128, 128)
    with pytest.raises(RuntimeError, match="h0 must be"):
        ops.lstm(torch.zeros(2, 64, 128, **h), torch.zeros(512, 256, **h), torch.zeros(512, **h),
                 torch.zeros(32, 128, **h), None)
    with pytest.raises(RuntimeError, match="one slice"):
        ops.scatter_nd(torch.zeros(8, 4, device=device), torch.zeros(3, 4, device=device),
                       torch.zeros(2, 1, dtype=torch.int64, device=device))


@pytest.mark.gpu
def test_flash_attention_fwd_op_unsupported_shape_raises(ops, device):
    t = torch.zeros(64 * 96, dtype=torch.half, device=device)
    with pytest.raises(RuntimeError):
        ops.flash_attention_fwd(t, t, t, t, 64, 64, 96, 96)


@pytest.mark.gpu
def test_scatter_nd_op_reference_test(ops, tcu, oracle, device):
    """The reference's test_scatter_nd: data [7, 8, 9, 10] filled with 5, five random (i, j) rows, updates filled
    with 10; expected = data[indices[:, 0], indices[:, 1]] = updates. Bit-exact."""
    random.seed(1234)
    data_shape = [7, 8, 9, 10]
    data = torch.full(data_shape, 5.0, dtype=torch.float32, device=device)
    indices = torch.tensor([[random.randint(0, 6), random.randint(0, 7)] for _ in range(5)], dtype=torch.int64,
                           device=device)
    updates = torch.full([5, 9, 10], 10.0, dtype=torch.float32, device=device)
    expect = data.clone()
    expect[indices[:, 0], indices[:, 1]] = updates
    ops.scatter_nd(data, updates, indices)
    assert torch.equal(data, expect)
    # and through the pytiledcuda-style wrapper (data, indices, updates)
    data2 = torch.full(data_shape, 5.0, dtype=torch.float32, device=device)
    tcu.scatter_nd(data2, indices, updates)
    assert torch.equal(data2, expect)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("shape,k", [((7, 8, 9, 10), 2), ((33, 5), 1), ((6, 4, 3), 3), ((128, 64), 1), ((5, 3, 7), 2)])
def test_scatter_nd_assign_against_oracle(tcu, oracle, device, dtype, shape, k):
    """Distinct index rows (a permutation prefix), random data: bit-exact against the oracle; covers the 16-byte
    vector path (slices that are multiples of 16 bytes), the per-element path (odd slices) and k == rank."""
    rng = np.random.default_rng(7 + k + len(shape))
    np_dtype = np.float32 if dtype == torch.float32 else np.float16
    data = rng.standard_normal(shape).astype(np_dtype)
    lead = int(np.prod(shape[:k]))
    n = max(1, lead // 2)
    flat_rows = rng.permutation(lead)[:n]
    idx = np.stack(np.unravel_index(flat_rows, shape[:k]), axis=1).astype(np.int64)
    upd = rng.standard_normal((n,) + tuple(shape[k:])).astype(np_dtype)
    d = torch.from_numpy(data).to(device)
    tcu.scatter_nd(d, torch.from_numpy(idx).to(device), torch.from_numpy(upd).to(device))
    assert np.array_equal(d.cpu().numpy(), oracle.scatter_nd(data, idx, upd))


@pytest.mark.gpu
def test_scatter_nd_add_with_duplicates_and_skipped_rows(tcu, oracle, device):
    """Atomic-add mode with repeated rows: integer-valued floats make the sum order-independent, so the result is
    exact. Out-of-range rows are skipped and counted."""
    rng = np.random.default_rng(11)
    data = rng.integers(-8, 8, size=(16, 12)).astype(np.float32)
    idx = rng.integers(0, 16, size=(200, 1)).astype(np.int64)
    idx[17, 0] = 16
    idx[101, 0] = -1
    upd = rng.integers(-4, 4, size=(200, 12)).astype(np.float32)
    d = torch.from_numpy(data).to(device)
    skipped = torch.zeros(1, dtype=torch.int32, device=device)
    tcu.scatter_nd(d, torch.from_numpy(idx).to(device), torch.from_numpy(upd).to(device), mode="add",
                   skipped_rows=skipped)
    assert np.array_equal(d.cpu().numpy(), oracle.scatter_nd(data, idx, upd, mode="add"))
    assert int(skipped.item()) == 2
    # fp16 accumulate: small integers stay exact in fp16
    data16 = rng.integers(-8, 8, size=(9, 5)).astype(np.float16)
    idx16 = rng.integers(0, 9, size=(64, 1)).astype(np.int64)
    upd16 = rng.integers(-2, 3, size=(64, 5)).astype(np.float16)
    d16 = torch.from_numpy(data16).to(device)
    tcu.scatter_nd(d16, torch.from_numpy(idx16).to(device), torch.from_numpy(upd16).to(device), mode="add")
    assert np.array_equal(d16.cpu().numpy(), oracle.scatter_nd(data16, idx16, upd16, mode="add"))


@pytest.mark.gpu
def test_scatter_nd_large_round_trip(tcu, device):
    """Full-size property check: scattering the rows of X to a random permutation and gathering them back is the
    identity (64 Mi elements, 256 MiB each way)."""
    rows, width = 65536, 1024
    g = torch.Generator(device="cpu").manual_seed(5)
    perm = torch.randperm(rows, generator=g).to(device)
    x = torch.randn(rows, width, device=device)
    y = torch.zeros_like(x)
    tcu.scatter_nd(y, perm.view(rows, 1), x)
    assert torch.equal(y[perm], x)


@pytest.mark.gpu
def test_gemm_b2b_lstm_ops(ops, tcu, oracle, device):
    A = oracle.fill_uniform(128 * 256, 1235).reshape(128, 256)
    Bt = oracle.fill_uniform(64 * 256, 2235).reshape(64, 256)
    C = torch.empty(128, 64, dtype=torch.float32, device=device)
    ops.gemm(torch.from_numpy(A).to(device), torch.from_numpy(Bt).to(device), C)
    assert oracle.max_rel_err(C.cpu().numpy(), oracle.gemm(A, Bt)) <= 1e-3

    # few output tiles and a long K: the op splits over K through a workspace it takes from torch's allocator
    A2 = oracle.fill_uniform(256 * 8192, 1236).reshape(256, 8192)
    Bt2 = oracle.fill_uniform(256 * 8192, 2236).reshape(256, 8192)
    assert tcu.gemm_workspace_bytes(256, 256, 8192) > 0
    C2 = torch.empty(256, 256, dtype=torch.float16, device=device)
    for _ in range(3):  # the workspace block is reused between calls
        ops.gemm(torch.from_numpy(A2).to(device), torch.from_numpy(Bt2).to(device), C2)
    assert oracle.max_rel_err(C2.float().cpu().numpy(), oracle.gemm(A2, Bt2)) <= 1e-3

    M, N, K, P = 64, 64, 64, 64
    A3 = oracle.fill_normal(M * K, 1, 0, 0.1).reshape(M, K)
    B3 = oracle.fill_normal(N * K, 2, 0, 0.1).reshape(N, K)
    C3 = oracle.fill_normal(P * N, 3, 0, 0.1).reshape(P, N)
    D = torch.empty(1, M, P, dtype=torch.float32, device=device)
    ops.b2b_gemm(*(torch.from_numpy(t).to(device) for t in (A3, B3, C3)), D)
    assert oracle.max_rel_err(D[0].cpu().numpy(), oracle.b2b_gemm(A3, B3, C3), eps=1.0) <= 1e-3

    T, Bb, I, H = 2, 64, 128, 128
    x = oracle.fill_normal(T * Bb * I, 4, 0, 0.5).reshape(T, Bb, I)
    W = oracle.fill_normal(4 * H * (I + H), 5, 0, 0.05).reshape(4 * H, I + H)
    b = oracle.fill_normal(4 * H, 6, 0, 0.05)
    h, c = ops.lstm(torch.from_numpy(x).to(device), torch.from_numpy(W).to(device), torch.from_numpy(b).to(device),
                    None, None)
    h_ref, c_ref = oracle.lstm(x, W, b)
    assert oracle.max_abs_err(h.float().cpu().numpy(), h_ref) <= 1e-2
    assert oracle.max_abs_err(c.cpu().numpy(), c_ref) <= 1e-2
