"""The C++ host program on the C-ABI (examples/cpp/host_driver.cc, built by __graft_entry__.build()): run as a child
process on operands written from the oracle's seeded generators; the results it dumps are checked here against the
oracle (the checker stays in the test, the program only launches, times and dumps). The counterpart of running the
reference's example drivers (examples/cpp/01_gemm/02_gemm_all_mem/main.cu:10-116,
examples/cpp/02_fused_two_gemms/fused_gemm.cu:17-262)."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "examples", "cpp", "_build", "host_driver")


def test_host_driver_is_built_and_links_the_c_abi():
    """No GPU needed: the binary exists, and its dynamic section names the C-ABI library (not a static copy of kernels)."""
    assert os.path.isfile(DRIVER), "run __graft_entry__.build() first"
    out = subprocess.run(["readelf", "-d", DRIVER], capture_output=True, text=True, check=True).stdout
    assert "libtiledcuda_amd.so" in out
    assert "librocblas.so" in out
    usage = subprocess.run([DRIVER], capture_output=True, text=True)
    assert usage.returncode == 64 and "usage:" in usage.stderr


def _run(args, tmp_path):
    print("host_driver " + " ".join(args), flush=True)
    proc = subprocess.run([DRIVER, *args, "--in", str(tmp_path), "--out", str(tmp_path), "--iters", "5", "--warmup", "2"],
                          capture_output=True, text=True, timeout=300)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    return proc.stdout


@pytest.mark.gpu
def test_host_driver_gemm_configs(oracle, device, tmp_path):
    # C1 in full, C2 on sampled rows
    A = oracle.fill_uniform(128 * 256, 1235).reshape(128, 256)
    Bt = oracle.fill_uniform(64 * 256, 2235).reshape(64, 256)
    A.tofile(tmp_path / "gemm_c1.A.bin")
    Bt.tofile(tmp_path / "gemm_c1.B.bin")
    out = _run(["gemm_c1"], tmp_path)
    assert "Test passed." in out and "Ratio" in out
    C = np.fromfile(tmp_path / "gemm_c1.C.bin", dtype=np.float32).reshape(128, 64)
    assert oracle.max_rel_err(C, oracle.gemm(A, Bt)) <= 1e-3

    n = 4096
    A = oracle.fill_uniform(n * n, 1236).reshape(n, n)
    Bt = oracle.fill_uniform(n * n, 2236).reshape(n, n)
    A.tofile(tmp_path / "gemm_c2.A.bin")
    Bt.tofile(tmp_path / "gemm_c2.B.bin")
    out = _run(["gemm_c2"], tmp_path)
    assert "Test passed." in out and "TFLOP/s" in out
    C = np.fromfile(tmp_path / "gemm_c2.C.bin", dtype=np.float16).reshape(n, n).astype(np.float32)
    for rows in [(0, 64), (2040, 2104), (4032, 4096)]:
        ref = oracle.gemm(A, Bt, rows=rows)
        assert oracle.max_rel_err(C[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= 1e-3


@pytest.mark.gpu
def test_host_driver_b2b_config3(oracle, device, tmp_path):
    M, N, K, P = 8192, 256, 128, 128
    A = oracle.fill_normal(M * K, 1237, 0, 0.1).reshape(1, M, K)
    Bt = oracle.fill_normal(N * K, 2237, 0, 0.1).reshape(1, N, K)
    Ct = oracle.fill_normal(P * N, 3237, 0, 0.1).reshape(1, P, N)
    for name, a in (("A", A), ("B", Bt), ("C", Ct)):
        a.tofile(tmp_path / f"b2b_c3.{name}.bin")
    out = _run(["b2b_c3"], tmp_path)
    assert "passed." in out
    D = np.fromfile(tmp_path / "b2b_c3.D.bin", dtype=np.float16).reshape(1, M, P).astype(np.float32)
    assert oracle.max_rel_err(D, oracle.b2b_gemm(A, Bt, Ct), eps=1.0) <= 1e-3


@pytest.mark.gpu
def test_host_driver_attention_config4(oracle, device, tmp_path):
    batch, S, D = 64, 2048, 128
    n = batch * S * D
    q = oracle.fill_normal(n, 1238).reshape(batch, S, D)
    k = oracle.fill_normal(n, 2238).reshape(batch, S, D)
    v = oracle.fill_normal(n, 3238).reshape(batch, S, D)
    for name, a in (("Q", q), ("K", k), ("V", v)):
        a.tofile(tmp_path / f"attn_c4.{name}.bin")
    out = _run(["attn_c4"], tmp_path)
    assert "passed." in out and "TFLOP/s" in out
    O = np.fromfile(tmp_path / "attn_c4.O.bin", dtype=np.float16).reshape(batch, S, D).astype(np.float32)
    scale = 1.0 / np.sqrt(D)
    for head, r0 in ((0, 0), (31, 960), (63, 1920)):
        ref = oracle.attention(np.ascontiguousarray(q[head:head + 1, r0:r0 + 128]), k[head:head + 1], v[head:head + 1], scale)
        assert oracle.max_abs_err(O[head:head + 1, r0:r0 + 128], ref) <= 1e-2
