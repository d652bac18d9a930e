"""Parity tests of the kernel entries, through the C-ABI (ctypes), against the CPU oracle on
the same seeded inputs.

Tolerances of the benchmark specification: GEMM / back-to-back GEMM max relative error <= 1e-3 against the
f32-accumulated oracle, where "relative" is |x - ref| / max(|ref|, eps * rms(ref)) (outputs of a
K-long dot product land arbitrarily close to zero, so a plain elementwise ratio is meaningless).
eps = 0.01 for the single GEMM. eps = 1 for the back-to-back GEMM: its f16-rounded
intermediate is part of the specification, and two correct f32 accumulations that differ in
the last bit round a few intermediates to neighbouring f16 values, which moves outputs by
about 3e-4 * rms (the oracle itself sits 9e-4 * rms away from the unrounded product), so
errors can only be judged against the output scale. Attention and LSTM: max absolute error
<= 1e-2.
Seeds: 1234 + configuration index, as the CPU-baseline plan fixes them.
"""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3
ABS_TOL = 1e-2


def dev(a, device):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def host(t):
    return t.float().cpu().numpy() if t.dtype != __import__("torch").float32 else t.cpu().numpy()


# ------------------------------------------------------------------------------ GEMM
@pytest.mark.parametrize("algo", ["global_reg", "all_mem", "pipelined", "auto"])
def test_gemm_config1_readme_shape(tcu, oracle, device, algo):
    """C1: M=128 N=64 K=256, U[-1,1], f32 out, every GEMM kernel."""
    import torch

    print(f"gemm C1 algo={algo}", flush=True)
    A = oracle.fill_uniform(128 * 256, 1235).reshape(128, 256)
    Bt = oracle.fill_uniform(64 * 256, 1235 + 1000).reshape(64, 256)
    C = tcu.gemm(dev(A, device), dev(Bt, device), out_dtype=torch.float32, algo=algo)
    torch.cuda.synchronize()
    assert oracle.max_rel_err(host(C), oracle.gemm(A, Bt)) <= REL_TOL


def test_gemm_golden_ramp(tcu, oracle, device):
    import os

    import torch

    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "golden_small.npz"))
    A, Bt, C = gold["gemm_128x64x256_A"], gold["gemm_128x64x256_Bt"], gold["gemm_128x64x256_C"]
    for algo in ("global_reg", "all_mem", "pipelined"):
        got = tcu.gemm(dev(A, device), dev(Bt, device), out_dtype=torch.float32, algo=algo)
        assert oracle.max_rel_err(host(got), C) <= REL_TOL


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (64, 128, 192), (128, 128, 64), (256, 128, 512), (256, 256, 128),
                                   (512, 1024, 256), (1024, 768, 320), (2048, 2048, 1024)])
@pytest.mark.parametrize("out_dtype", ["f32", "f16"])
def test_gemm_pipelined_shapes(tcu, oracle, device, M, N, K, out_dtype):
    """Run-time shapes across all three tile configurations, one- and many-k-tile loops."""
    import torch

    print(f"gemm pipelined {M}x{N}x{K} {out_dtype}", flush=True)
    A = oracle.fill_uniform(M * K, 7 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 9 + N).reshape(N, K)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    C = tcu.gemm(dev(A, device), dev(Bt, device), out_dtype=dt, algo="pipelined")
    torch.cuda.synchronize()
    assert oracle.max_rel_err(host(C), oracle.gemm(A, Bt)) <= REL_TOL


@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (256, 256, 128), (256, 512, 192), (512, 256, 256), (768, 1024, 320),
                                   (2048, 2048, 1024)])
@pytest.mark.parametrize("out_dtype", ["f32", "f16"])
def test_gemm_wave128_shapes(tcu, oracle, device, M, N, K, out_dtype):
    """The one-wavefront-per-SIMD kernel: one, two, three and many k-tiles (its last two tiles are peeled), one and many
    workgroups, both output types; against the oracle and bit for bit against the pipelined kernel, whose arithmetic
    (MFMA shape, order of the k-substeps) it shares."""
    import torch

    print(f"gemm wave128 {M}x{N}x{K} {out_dtype}", flush=True)
    A = oracle.fill_uniform(M * K, 17 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 19 + N).reshape(N, K)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    dA, dB = dev(A, device), dev(Bt, device)
    C = tcu.gemm(dA, dB, out_dtype=dt, algo="wave128")
    torch.cuda.synchronize()
    assert oracle.max_rel_err(host(C), oracle.gemm(A, Bt)) <= REL_TOL
    assert torch.equal(C, tcu.gemm(dA, dB, out_dtype=dt, algo="pipelined"))


@pytest.mark.parametrize("M,N,K", [(16, 16, 16), (16, 48, 32), (80, 16, 48), (48, 112, 80), (144, 208, 16), (64, 64, 64),
                                   (1040, 528, 272), (4096, 16, 4096)])
@pytest.mark.parametrize("out_dtype", ["f32", "f16"])
def test_gemm_ragged_shapes(tcu, oracle, device, M, N, K, out_dtype):
    """Every shape made of whole 16 x 16 BaseTiles (the granularity of the reference's tile types,
    include/types/register.hpp:108-112) runs: blocks that hang over the edge in M, in N and in both, a last k-step of
    16, one tile, a thin N; through AUTO (which must route them to the run-time-shape kernel) and by name. The output is
    surrounded by a guard band that must stay untouched."""
    import torch

    print(f"gemm ragged {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    A = oracle.fill_uniform(M * K, 31 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 37 + N).reshape(N, K)
    want = oracle.gemm(A, Bt)
    dA, dB = dev(A, device), dev(Bt, device)
    for algo in ("ragged", "auto"):
        guard = torch.full((M + 2, N), -7.0, dtype=dt, device=device)
        out = guard[1:M + 1]
        tcu.gemm(dA, dB, out=out, algo=algo)
        torch.cuda.synchronize()
        assert oracle.max_rel_err(host(out), want) <= REL_TOL
        assert torch.all(guard[0] == -7.0) and torch.all(guard[M + 1] == -7.0)


@pytest.mark.parametrize("M,N,K,splits", [(256, 256, 8192, 16), (512, 512, 16384, 8), (1024, 1024, 16384, 4),
                                          (1024, 2048, 16384, 2), (2048, 2048, 32768, 4), (2048, 2048, 8192, 1),
                                          (2048, 4096, 2048, 1),
                                          (1536, 1536, 4096, 1), (1024, 1024, 8192, 4), (1024, 1024, 4096, 1), (256, 512, 512, 1),
                                          (752, 1808, 8192, 2), (528, 512, 8192, 8), (272, 400, 8192, 16),
                                          (2048, 2048, 2048, 1)])
@pytest.mark.parametrize("out_dtype", ["f32", "f16"])
def test_gemm_split_k_with_workspace(tcu, oracle, device, M, N, K, splits, out_dtype):
    """tcu_gemm_f16_ws: few output tiles and a long K are split over K (f32 partial products in the caller's workspace,
    then a reduction) where that is expected to beat the unsplit launch - the partial products from the kernel with
    128 x 128 tiles whose wavefronts split K once more (first four cases, 1024 x 1024 x 8192, and - with edge tiles - the
    three shapes that are not whole tiles) or, where those tiles alone fill the chip, from
    the one with 256 x 256 tiles (2048 x 2048 x 32768); against the oracle and against the unsplit kernel; the workspace size is splits * M * N * 4, bytes past it stay untouched; shapes that are not split (last six
    cases: among them 2048 x 2048 x 8192 and 1536 x 1536 x 4096, where the kernel whose wavefronts split K inside the
    workgroup is the faster plan) take the ordinary path and need no workspace."""
    import torch

    print(f"gemm split-K {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    need = tcu.gemm_workspace_bytes(M, N, K)
    assert need == (splits * M * N * 4 if splits > 1 else 0)
    A = oracle.fill_uniform(M * K, 131 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 137 + N).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    ws = torch.full((need + 4096,), 0xFF, dtype=torch.uint8, device=device)
    C = tcu.gemm(dA, dB, out_dtype=dt, workspace=ws)
    torch.cuda.synchronize()
    rows = slice(0, min(M, 192 if N * K <= 2 ** 24 else 48))
    want = oracle.gemm(A[rows], Bt)
    assert oracle.max_rel_err(host(C)[rows], want) <= REL_TOL
    plain = tcu.gemm(dA, dB, out_dtype=dt, workspace=False)
    assert oracle.max_rel_err(host(C), host(plain)) <= REL_TOL
    assert bool((ws[need:] == 0xFF).all())
    if splits > 1:
        with pytest.raises(RuntimeError):
            tcu.gemm(dA, dB, out_dtype=dt, workspace=ws[:need // 2])


@pytest.mark.parametrize("M,N,K", [(80, 144, 64), (1040, 528, 256), (272, 4112, 128), (2064, 4080, 192), (4112, 4112, 64),
                                   (1040, 528, 272), (2064, 1040, 1072), (256, 256, 48), (4096, 4096, 144), (144, 208, 16)])
@pytest.mark.parametrize("out_dtype", ["f32", "f16"])
def test_gemm_edge_tiles(tcu, oracle, device, M, N, K, out_dtype):
    """M, N, K multiples of 16 but not all of 64: AUTO runs the pipelined kernel with edge tiles (rows beyond the edge
    loaded from the last valid row, stores guarded, the pieces of the last k-tile beyond K zeroed in LDS) in all three
    tile sizes, with k tails of 16, 32 and 48 and a single partial k-tile; against the oracle on sampled rows including
    the last ones, against the run-time-shape kernel everywhere, with guard bands around the output."""
    import torch

    print(f"gemm edge tiles {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    A = oracle.fill_uniform(M * K, 231 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 237 + N).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    guard = torch.full((M + 2, N), -7.0, dtype=dt, device=device)
    out = guard[1:M + 1]
    tcu.gemm(dA, dB, out=out, algo="auto")
    torch.cuda.synchronize()
    assert torch.all(guard[0] == -7.0) and torch.all(guard[M + 1] == -7.0)
    rows = sorted(set(list(range(0, min(M, 48))) + list(range(max(0, M - 48), M))))
    want = oracle.gemm(A[rows], Bt)
    assert oracle.max_rel_err(host(out)[rows], want) <= REL_TOL
    plain = tcu.gemm(dA, dB, out_dtype=dt, algo="ragged")
    assert oracle.max_rel_err(host(out), host(plain)) <= REL_TOL


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (256, 256, 64), (128, 192, 128), (256, 256, 192), (192, 320, 256),
                                   (256, 320, 320), (512, 512, 384), (1024, 1024, 2048), (80, 112, 48), (208, 400, 112), (144, 272, 1040)])
@pytest.mark.parametrize("out_dtype", ["f32", "f16"])
def test_gemm_ring_of_small_tiles(tcu, oracle, device, M, N, K, out_dtype):
    """Few 64 x 64 tiles per CU: the pipelined kernel runs them with a 4-stage ring (three tiles in flight behind the
    one being multiplied). Loops of 1 .. 6 and 32 k-tiles (shorter than, equal to and longer than the ring), whole and
    edge tiles with a k tail; against the oracle and, for the order of the sum, bit for bit against the two-stage kernel
    of the tile library where that is instantiated."""
    import torch

    print(f"gemm ring {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    A = oracle.fill_uniform(M * K, 331 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 337 + N).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    guard = torch.full((M + 2, N), -7.0, dtype=dt, device=device)
    out = guard[1:M + 1]
    tcu.gemm(dA, dB, out=out, algo="pipelined")
    torch.cuda.synchronize()
    assert torch.all(guard[0] == -7.0) and torch.all(guard[M + 1] == -7.0)
    assert oracle.max_rel_err(host(out), oracle.gemm(A, Bt)) <= REL_TOL
    if (M, N, K) == (256, 256, 64):
        assert torch.equal(out, tcu.gemm(dA, dB, out_dtype=dt, algo="tile_pipelined"))


def test_gemm_wave128_rotated_k_order(tcu, oracle, device):
    """K = 16384 (rows 32 KiB apart): each XCD's workgroups start their walk over K at a different eighth and wrap
    around. 8 tiles = one workgroup on every XCD, so every start is exercised; the oracle on 16 rows of each tile row."""
    import torch

    M, N, K = 512, 1024, 16384
    print(f"gemm wave128 rotated k {M}x{N}x{K}", flush=True)
    A = oracle.fill_uniform(M * K, 401).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 402).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    for dt in (torch.float32, torch.float16):
        C = tcu.gemm(dA, dB, out_dtype=dt, algo="wave128")
        torch.cuda.synchronize()
        got = host(C)
        for r0 in (0, 240, 256, 496):
            want = oracle.gemm(A[r0:r0 + 16], Bt)
            assert oracle.max_rel_err(got[r0:r0 + 16], want) <= REL_TOL
        # the same sums in the plain order, everywhere
        assert oracle.max_rel_err(got, host(tcu.gemm(dA, dB, out_dtype=dt, algo="pipelined"))) <= REL_TOL
        assert torch.equal(C, tcu.gemm(dA, dB, out_dtype=dt, algo="wave128"))  # the same on every run


@pytest.mark.parametrize("M,N,K", [(4112, 4112, 1024), (4112, 4096, 512), (4096, 4112, 512), (4144, 4128, 192)])
@pytest.mark.parametrize("out_dtype", ["f32", "f16"])
def test_gemm_main_block_and_strips(tcu, oracle, device, M, N, K, out_dtype):
    """M or N a little above a multiple of 256: AUTO computes the leading block of whole 256 x 256 tiles with the
    one-wavefront-per-SIMD kernel and the remaining columns / rows with small tiles (three launches on disjoint parts
    of C) instead of paying a whole extra round of 256 x 256 edge tiles. Against the oracle on the first and last rows
    (the last ones lie in the bottom strip, every row crosses into the right strip), bit for bit against the
    single-launch pipelined kernel everywhere, with guard rows around the output."""
    import torch

    print(f"gemm main block + strips {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    A = oracle.fill_uniform(M * K, 431 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 437 + N).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    guard = torch.full((M + 2, N), -7.0, dtype=dt, device=device)
    out = guard[1:M + 1]
    tcu.gemm(dA, dB, out=out, algo="auto")
    torch.cuda.synchronize()
    assert torch.all(guard[0] == -7.0) and torch.all(guard[M + 1] == -7.0)
    rows = list(range(0, 24)) + list(range(M - 24, M))
    assert oracle.max_rel_err(host(out)[rows], oracle.gemm(A[rows], Bt)) <= REL_TOL
    assert torch.equal(out, tcu.gemm(dA, dB, out_dtype=dt, algo="pipelined"))


def test_gemm_wave128_rejects_other_shapes(tcu, device):
    import torch

    A = torch.zeros(128, 40, dtype=torch.float16, device=device)  # K must be a multiple of 16
    with pytest.raises(RuntimeError):
        tcu.gemm(A, A, algo="wave128")


@pytest.mark.parametrize("M,N,K", [(16, 16, 64), (272, 400, 128), (1040, 528, 192), (4112, 272, 64), (240, 4112, 320),
                                   (3088, 3088, 256), (256, 256, 48), (256, 512, 80), (512, 768, 144), (1040, 528, 272),
                                   (272, 400, 16), (2064, 2320, 1072), (3600, 3600, 1200)])
@pytest.mark.parametrize("out_dtype", ["f16", "f32"])
def test_gemm_wave128_edge_tiles(tcu, oracle, device, M, N, K, out_dtype):
    """The one-wavefront-per-SIMD kernel on shapes that are not whole 256 x 256 tiles (M, N in multiples of 16): rows
    beyond the edge are fetched from the last valid row and their results dropped, the stores are guarded - a single
    partial tile, edges in M, in N and in both, a tile row and a tile column that are 16 wide; against the oracle, bit
    for bit against the pipelined kernel, with guard rows around C. 3088 x 3088 is a shape AUTO sends to it (169 tiles in one
    round). The last seven shapes have a K that is not whole tiles of 64 (tails of 16, 32 and 48 behind 0, 1, 2, 4, 16 and 18
    whole tiles): the pieces of the last tile beyond K are fetched from inside the row and zeroed in LDS; 3600 x 3600 x 1200
    is such a shape that AUTO sends here."""
    import torch

    print(f"gemm wave128 edge tiles {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float16 if out_dtype == "f16" else torch.float32
    A = oracle.fill_uniform(M * K, 6100 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 6200 + N).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    guard = torch.full((M + 2, N), -7.0, dtype=dt, device=device)
    out = guard[1:M + 1]
    tcu.gemm(dA, dB, out=out, algo="wave128")
    torch.cuda.synchronize()
    assert torch.all(guard[0] == -7.0) and torch.all(guard[M + 1] == -7.0)
    rows = (0, M) if M * N * K <= 2 ** 28 else (M - 64, M)
    ref = oracle.gemm(A, Bt, rows=rows)
    assert oracle.max_rel_err(host(out)[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= REL_TOL
    assert torch.equal(out, tcu.gemm(dA, dB, out_dtype=dt, algo="pipelined"))
    if M == 3088 or M == 3600:
        auto = tcu.gemm(dA, dB, out_dtype=dt, workspace=False)
        assert torch.equal(out, auto)


@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (512, 768, 192), (1024, 1024, 1024), (4096, 4096, 4096)])
@pytest.mark.parametrize("out_dtype", ["f16", "f32"])
def test_gemm_tile_api_pipelined_is_the_pipelined_kernel(tcu, oracle, device, M, N, K, out_dtype):
    """The multi-stage kernel written with tile-library functors only (GlobalToSharedDirectLoader into a SharedRing,
    SharedToRegLoader on 16 x 32 / 32 x 16 MFMA operand tiles, gemm()) against the oracle and, bit for bit, against
    the hand-indexed pipelined kernel, whose arithmetic it performs in the same order (1, 3, 16 and 64 k-tiles)."""
    import torch

    print(f"gemm tile_pipelined {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float16 if out_dtype == "f16" else torch.float32
    A = oracle.fill_uniform(M * K, 7000 + K).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 8000 + K).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    C = tcu.gemm(dA, dB, out_dtype=dt, algo="tile_pipelined")
    torch.cuda.synchronize()
    rows = (0, M) if M <= 1024 else (M - 192, M)
    ref = oracle.gemm(A, Bt, rows=rows)
    assert oracle.max_rel_err(host(C)[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= REL_TOL
    assert torch.equal(C, tcu.gemm(dA, dB, out_dtype=dt, algo="pipelined"))


@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (512, 768, 192), (1024, 1024, 1024), (4096, 4096, 4096)])
@pytest.mark.parametrize("out_dtype", ["f16", "f32"])
def test_gemm_tile_api_wave128_is_the_wave128_kernel(tcu, oracle, device, M, N, K, out_dtype):
    """The one-wavefront-per-SIMD kernel written with tile-library functors only (GlobalToSharedDirectPieces,
    SharedToRegLoader::load_one, gemm_scheduled with AGPR-pinned accumulators) against the oracle and, bit for bit,
    against the hand-indexed kernel whose schedule it reproduces (1, 3, 16 and 64 k-tiles: every peeled form of the
    loop over k)."""
    import torch

    print(f"gemm tile_wave128 {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float16 if out_dtype == "f16" else torch.float32
    A = oracle.fill_uniform(M * K, 7100 + K).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 8100 + K).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    C = tcu.gemm(dA, dB, out_dtype=dt, algo="tile_wave128")
    torch.cuda.synchronize()
    rows = (0, M) if M <= 1024 else (M - 192, M)
    ref = oracle.gemm(A, Bt, rows=rows)
    assert oracle.max_rel_err(host(C)[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= REL_TOL
    assert torch.equal(C, tcu.gemm(dA, dB, out_dtype=dt, algo="wave128"))


@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (256, 128, 256), (128, 384, 384), (512, 512, 512), (256, 256, 640),
                                   (2048, 2048, 2048)])
@pytest.mark.parametrize("out_dtype", ["f16", "f32"])
def test_gemm_wave128_ksplit(tcu, oracle, device, M, N, K, out_dtype):
    """The kernel whose four wavefronts each own the whole 128 x 128 tile over a quarter of K and add their partial
    tiles through LDS: 1 to 5 tiles of K (odd and even counts: the fragment buffers alternate) against the oracle,
    guard rows around C; 2048^3 is the shape AUTO sends to it, so AUTO must give the same bits there."""
    import torch

    print(f"gemm wave128_ksplit {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float16 if out_dtype == "f16" else torch.float32
    A = oracle.fill_uniform(M * K, 7200 + K).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 8200 + K).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    guard = torch.full((M + 2, N), -7.0, dtype=dt, device=device)
    out = guard[1:M + 1]
    tcu.gemm(dA, dB, out=out, algo="wave128_ksplit")
    torch.cuda.synchronize()
    assert torch.all(guard[0] == -7.0) and torch.all(guard[M + 1] == -7.0)
    rows = (0, M) if M <= 1024 else (M - 192, M)
    ref = oracle.gemm(A, Bt, rows=rows)
    assert oracle.max_rel_err(host(out)[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= REL_TOL
    if M == 2048:
        assert torch.equal(out, tcu.gemm(dA, dB, out_dtype=dt))
        # every row of the product, through the column sums: C^T 1 = B (A^T 1)
        col = A.astype(np.float64).sum(axis=0)
        want = Bt.astype(np.float64) @ col
        got = host(out).astype(np.float64).sum(axis=0)
        # entries are ~N(0, 15^2); f16 rounding (<= 2^-11 |c| each) of 2048 of them adds up to about a unit
        assert np.max(np.abs(got - want)) <= (5.0 if out_dtype == "f16" else 0.1)


@pytest.mark.parametrize("M,N,K", [(256, 128, 64), (256, 384, 128), (512, 640, 320), (1024, 1152, 1984), (2048, 2560, 4096),
                                   (2048, 4096, 1024), (16, 16, 64), (272, 400, 128), (1040, 528, 192), (1552, 3088, 1024)])
@pytest.mark.parametrize("out_dtype", ["f16", "f32"])
def test_gemm_wave128_narrow(tcu, oracle, device, M, N, K, out_dtype):
    """The one-wavefront-per-SIMD kernel with 256 x 128 workgroup tiles (a wavefront owns 128 x 64): 1 to 64 tiles of K,
    odd and even counts, against the oracle and bit for bit against the pipelined kernel (same order of the sum), guard
    rows around C; 2048 x 2560 x 4096 (160 tiles: more than half a round of 256 x 256 tiles would idle, 128 x 128 tiles
    need two rounds) and 2048 x 4096 x 1024 (exactly 128 tiles of 256 x 256, half of the chip) are shapes AUTO sends to it,
    and so is 1552 x 3088 x 1024 (175 tiles, with edge tiles: the last four shapes are not whole tiles - rows beyond the edge
    are fetched from the last valid row, the stores are guarded)."""
    import torch

    print(f"gemm wave128_narrow {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float16 if out_dtype == "f16" else torch.float32
    A = oracle.fill_uniform(M * K, 7300 + K).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 8300 + K).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    guard = torch.full((M + 2, N), -7.0, dtype=dt, device=device)
    out = guard[1:M + 1]
    tcu.gemm(dA, dB, out=out, algo="wave128_narrow")
    torch.cuda.synchronize()
    assert torch.all(guard[0] == -7.0) and torch.all(guard[M + 1] == -7.0)
    rows = (0, M) if M <= 1024 else (M - 192, M)
    ref = oracle.gemm(A, Bt, rows=rows)
    assert oracle.max_rel_err(host(out)[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= REL_TOL
    assert torch.equal(out, tcu.gemm(dA, dB, out_dtype=dt, algo="pipelined"))
    if M == 2048 or M == 1552:
        assert torch.equal(out, tcu.gemm(dA, dB, out_dtype=dt, workspace=False))  # AUTO takes this kernel here


@pytest.mark.parametrize("M,N,K,main,rest_algo", [(2560, 8192, 2048, (2048, 8192), "wave128_ksplit"),
                                                  (8192, 2560, 2048, (8192, 2048), "wave128_ksplit"),
                                                  (4608, 4608, 4096, None, "wave128_narrow"),
                                                  (2688, 6912, 2048, (2304, 6912), "wave128_ksplit")])
@pytest.mark.parametrize("out_dtype", ["f16", "f32"])
def test_gemm_full_rounds_and_rest(tcu, oracle, device, M, N, K, main, rest_algo, out_dtype):
    """More than 256 tiles of 256 x 256 with a last round that is far from full (320 = 256 + 64, 324 = 252 + 72): AUTO
    gives the leading rows (first and third case) or columns (second case) to the one-wavefront-per-SIMD kernel and the
    rest of C to a kernel with smaller tiles, as a second launch; the last case is not whole tiles (10.5 x 27 tiles: both
    launches have edge tiles). Against the oracle on rows of both parts; the main
    part bit for bit what the one-wavefront-per-SIMD kernel writes there in one launch, the rest bit for bit what the
    named kernel gives on that sub-problem (the kernel with 256 x 128 tiles sums in the same order as the one with
    256 x 256, so there all of C is compared with the single launch); guard rows around C."""
    import torch

    print(f"gemm rounds and rest {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float16 if out_dtype == "f16" else torch.float32
    A = oracle.fill_uniform(M * K, 9100 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 9200 + N).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    guard = torch.full((M + 2, N), -7.0, dtype=dt, device=device)
    out = guard[1:M + 1]
    tcu.gemm(dA, dB, out=out, workspace=False)
    torch.cuda.synchronize()
    assert torch.all(guard[0] == -7.0) and torch.all(guard[M + 1] == -7.0)
    for rows in ((0, 32), (M - 32, M)):
        ref = oracle.gemm(A, Bt, rows=rows)
        assert oracle.max_rel_err(host(out)[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= REL_TOL
    whole = tcu.gemm(dA, dB, out_dtype=dt, algo="wave128")
    if main is None:
        assert torch.equal(out, whole)
        return
    Mm, Nm = main
    assert torch.equal(out[:Mm, :Nm], whole[:Mm, :Nm])
    if Mm < M:
        assert torch.equal(out[Mm:], tcu.gemm(dA[Mm:], dB, out_dtype=dt, algo=rest_algo))
    else:
        assert torch.equal(out[:, Nm:], tcu.gemm(dA, dB[Nm:], out_dtype=dt, algo=rest_algo))


@pytest.mark.parametrize("M,N,K", [(16, 16, 128), (144, 112, 256), (272, 400, 384), (1552, 1552, 4096), (1536, 1616, 2048),
                                   (1808, 1936, 256), (1536, 1536, 512)])
@pytest.mark.parametrize("out_dtype", ["f16", "f32"])
def test_gemm_wave128_ksplit_edge_tiles(tcu, oracle, device, M, N, K, out_dtype):
    """The K-splitting kernel on shapes that are not whole tiles (M, N in multiples of 16): rows beyond the edge are
    fetched from the last valid row and their results dropped, the stores are guarded - nothing outside C is written
    (guard rows and guard columns around it) and every element of C matches the oracle. Both tile widths: 128 x 96
    where 128 x 128 tiles would leave a quarter of the CUs idle (1552 x 1552 x 4096: 221 instead of 169 workgroups, a
    shape AUTO sends to this kernel; 1536 x 1536: whole 128 x 96 tiles), 128 x 128 otherwise (1808 x 1936: 240 tiles
    with edges)."""
    import torch

    print(f"gemm wave128_ksplit edges {M}x{N}x{K} {out_dtype}", flush=True)
    dt = torch.float16 if out_dtype == "f16" else torch.float32
    A = oracle.fill_uniform(M * K, 9200 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 9300 + N).reshape(N, K)
    dA, dB = dev(A, device), dev(Bt, device)
    guard = torch.full((M + 2, N), -7.0, dtype=dt, device=device)
    out = guard[1:M + 1]
    tcu.gemm(dA, dB, out=out, algo="wave128_ksplit")
    torch.cuda.synchronize()
    assert torch.all(guard[0] == -7.0) and torch.all(guard[M + 1] == -7.0)
    got = host(out)
    assert np.isfinite(got).all()
    rows = (0, M) if M <= 512 else (M - 160, M)  # the last rows include the edge tiles
    ref = oracle.gemm(A, Bt, rows=rows)
    assert oracle.max_rel_err(got[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= REL_TOL
    if M > 512:
        # every element, through row and column sums in float64
        a64, b64 = A.astype(np.float64), Bt.astype(np.float64)
        tol = 5.0 if out_dtype == "f16" else 0.2
        assert np.max(np.abs(got.astype(np.float64).sum(axis=0) - b64 @ a64.sum(axis=0))) <= tol
        assert np.max(np.abs(got.astype(np.float64).sum(axis=1) - a64 @ b64.sum(axis=0))) <= tol
    if (M, N, K) == (1552, 1552, 4096):
        assert torch.equal(out, tcu.gemm(dA, dB, out_dtype=dt, workspace=False))  # AUTO takes this kernel here


@pytest.mark.parametrize("algo", ["pipelined", "wave128"])
def test_gemm_one_hot_index_probe(tcu, device, algo):
    """C[m, n] = A[m, k] * Bt[n, k] for one-hot operands: pins rows/cols/transposition exactly."""
    import torch

    M = N = K = 256
    A = torch.zeros(M, K, dtype=torch.float16, device=device)
    Bt = torch.zeros(N, K, dtype=torch.float16, device=device)
    picks = [(0, 0, 0), (37, 201, 99), (255, 3, 255), (128, 64, 32), (200, 255, 1)]
    for i, (m, n, k) in enumerate(picks):
        A[m, k] = 1.0 + i
        Bt[n, k] = 2.0
    C = tcu.gemm(A, Bt, out_dtype=torch.float32, algo=algo).cpu().numpy()
    want = A.float().cpu().numpy() @ Bt.float().cpu().numpy().T
    assert np.array_equal(C, want)


def test_gemm_reference_driver_shapes(tcu, oracle, device):
    """The driver shapes of the reference's two GEMM examples (1024x1024x2048 global->register,
    4096^3 single-stage LDS): checked on a window of rows."""
    import torch

    for (M, N, K, algo) in [(1024, 1024, 2048, "global_reg"), (4096, 4096, 4096, "all_mem")]:
        print(f"gemm reference driver {M}x{N}x{K} {algo}", flush=True)
        A = oracle.fill_uniform(M * K, 1236).reshape(M, K)
        Bt = oracle.fill_uniform(N * K, 2236).reshape(N, K)
        C = host(tcu.gemm(dev(A, device), dev(Bt, device), out_dtype=torch.float32, algo=algo))
        rows = (M // 2 - 32, M // 2 + 32)
        ref = oracle.gemm(A, Bt, rows=rows)
        assert oracle.max_rel_err(C[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= REL_TOL
        first = oracle.gemm(A, Bt, rows=(0, 16))
        assert oracle.max_rel_err(C[:16], first[:16]) <= REL_TOL


def test_gemm_config2_4096_cubed(tcu, oracle, device):
    """C2: M=N=K=4096, U[-1,1], f16 out. Oracle on 768 sampled rows (first/middle/last tiles)
    plus size-independent properties over the full output."""
    import torch

    print("gemm C2 4096^3", flush=True)
    n = 4096
    A = oracle.fill_uniform(n * n, 1236).reshape(n, n)
    Bt = oracle.fill_uniform(n * n, 2236).reshape(n, n)
    dA, dB = dev(A, device), dev(Bt, device)
    C = tcu.gemm(dA, dB, out_dtype=torch.float16)
    torch.cuda.synchronize()
    Ch = host(C)
    assert np.isfinite(Ch).all()
    for rows in [(0, 256), (1920, 2176), (3840, 4096)]:
        ref = oracle.gemm(A, Bt, rows=rows)
        assert oracle.max_rel_err(Ch[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= REL_TOL
    # column sums: ones^T (A B) = (ones^T A) B, computed in float64 on the host
    colsum = A.astype(np.float64).sum(0) @ Bt.astype(np.float64).T
    got = Ch.astype(np.float64).sum(0)
    # entries are ~N(0, 37^2) rounded to f16 (error <= 2^-11 |c|); 4096 of them add up to an error of a few units
    assert np.max(np.abs(got - colsum)) <= 10.0
    # linearity in A: gemm(2A) == 2 gemm(A) (power-of-two scaling commutes with rounding, except for
    # the handful of outputs that land in the f16 subnormal range, where the spacing is absolute)
    C2 = tcu.gemm((dA * 2).contiguous(), dB, out_dtype=torch.float16)
    assert float((C2.float() - 2 * C.float()).abs().max()) <= 2.0 ** -23
    # f32 output agrees with the f16 output to f16 rounding
    C32 = tcu.gemm(dA, dB, out_dtype=torch.float32)
    assert torch.equal(C32.half(), C)
    # the two tuned kernels share their arithmetic: identical bit for bit
    assert torch.equal(tcu.gemm(dA, dB, out_dtype=torch.float16, algo="pipelined"), C)
    assert torch.equal(tcu.gemm(dA, dB, out_dtype=torch.float16, algo="wave128"), C)


# ------------------------------------------------------------------------------ back-to-back GEMM
@pytest.mark.parametrize("M,N,K,P,batch", [(64, 64, 64, 64, 1), (48, 64, 64, 64, 3), (128, 128, 64, 64, 2),
                                           (256, 256, 128, 128, 1), (1024, 256, 128, 128, 2)])
@pytest.mark.parametrize("out_dtype", ["f32", "f16"])
def test_b2b_gemm_shapes(tcu, oracle, device, M, N, K, P, batch, out_dtype):
    import torch

    print(f"b2b {M}x{N}x{K}x{P} b{batch} {out_dtype}", flush=True)
    A = oracle.fill_normal(batch * M * K, 11, 0, 0.1).reshape(batch, M, K)
    Bt = oracle.fill_normal(batch * N * K, 12, 0, 0.1).reshape(batch, N, K)
    Ct = oracle.fill_normal(batch * P * N, 13, 0, 0.1).reshape(batch, P, N)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    D = tcu.b2b_gemm(dev(A, device), dev(Bt, device), dev(Ct, device), out_dtype=dt)
    torch.cuda.synchronize()
    ref = oracle.b2b_gemm(A, Bt, Ct)
    # the f16-rounded intermediate may round differently where the f32 sums differ in the last
    # bit (different accumulation order); that moves an output by at most 2^-11 * |acc| * |C|
    assert oracle.max_rel_err(host(D), ref, eps=1.0) <= REL_TOL


# every uncommented run<...> of the reference's driver, examples/cpp/02_fused_two_gemms/fused_gemm.cu:212-259
REFERENCE_B2B_SHAPES = [(16, 16, 16, 16, 1), (16, 32, 16, 32, 1), (32, 64, 32, 64, 1), (64, 64, 32, 64, 1),
                        (256, 128, 64, 64, 1), (1024, 1024, 128, 128, 1), (16, 16, 16, 16, 2),
                        (1024, 1024, 128, 128, 5), (64, 256, 128, 128, 1), (2048, 1024, 128, 128, 1),
                        (1024, 2048, 128, 128, 1)]


@pytest.mark.parametrize("M,N,K,P,batch", REFERENCE_B2B_SHAPES)
@pytest.mark.parametrize("algo", ["tile_library", "auto"])
def test_b2b_gemm_reference_shape_list(tcu, oracle, device, M, N, K, P, batch, algo):
    """The shapes the reference's fused two-GEMM example runs, on the kernel composed from tile primitives and on
    whatever AUTO picks (the LDS-resident kernel, streaming blocks of N, where K = P = 128 and N % 256 == 0)."""
    import torch

    print(f"b2b reference shape {M}x{N}x{K}x{P} batch {batch} {algo}", flush=True)
    A = oracle.fill_normal(batch * M * K, 811, 0, 0.1).reshape(batch, M, K)
    Bt = oracle.fill_normal(batch * N * K, 812, 0, 0.1).reshape(batch, N, K)
    Ct = oracle.fill_normal(batch * P * N, 813, 0, 0.1).reshape(batch, P, N)
    D = tcu.b2b_gemm(dev(A, device), dev(Bt, device), dev(Ct, device), out_dtype=torch.float32, algo=algo)
    torch.cuda.synchronize()
    got = host(D)
    for b in range(batch):
        assert oracle.max_rel_err(got[b], oracle.b2b_gemm(A[b], Bt[b], Ct[b]), eps=1.0) <= REL_TOL


@pytest.mark.parametrize("M,N,batch,out_dtype", [(32, 256, 1, "f32"), (96, 256, 3, "f16"), (8192, 256, 1, "f16"),
                                                 (64, 1024, 2, "f16"), (2048, 2048, 1, "f32")])
def test_b2b_gemm_tile_resident_is_resident(tcu, oracle, device, M, N, batch, out_dtype):
    """The LDS-resident kernel composed from tile-library functors (tile_resident) sums in the order of the
    hand-indexed one: bit-identical outputs, for one block of N and for several (B and C refilled under the products),
    and within tolerance of the oracle."""
    import torch

    print(f"b2b tile_resident M{M} N{N} b{batch} {out_dtype}", flush=True)
    K, P = 128, 128
    A = oracle.fill_normal(batch * M * K, 171, 0, 0.1).reshape(batch, M, K)
    Bt = oracle.fill_normal(batch * N * K, 172, 0, 0.1).reshape(batch, N, K)
    Ct = oracle.fill_normal(batch * P * N, 173, 0, 0.1).reshape(batch, P, N)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    dA, dB, dC = dev(A, device), dev(Bt, device), dev(Ct, device)
    want = tcu.b2b_gemm(dA, dB, dC, out_dtype=dt, algo="resident")
    got = torch.full_like(want, float("nan"))
    tcu.b2b_gemm(dA, dB, dC, out=got, out_dtype=dt, algo="tile_resident")
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    rows = slice(0, min(M, 64))
    ref = oracle.b2b_gemm(np.ascontiguousarray(A[:, rows]), Bt, Ct)
    assert oracle.max_rel_err(host(got)[:, rows], ref, eps=1.0) <= REL_TOL


@pytest.mark.parametrize("M,N,batch,out_dtype", [(256, 128, 1, "f32"), (96, 256, 3, "f16"), (8192, 128, 2, "f16")])
def test_b2b_gemm_inner_size_64(tcu, oracle, device, M, N, batch, out_dtype):
    """K = P = 64 (the reference driver's (256, 128, 64, 64), examples/cpp/02_fused_two_gemms/fused_gemm.cu:212-259, and
    larger M / N): the LDS-resident composition from tile-library functors, which is what AUTO runs there, against the
    oracle; AUTO gives the same bits."""
    import torch

    print(f"b2b K=P=64 M{M} N{N} b{batch} {out_dtype}", flush=True)
    K, P = 64, 64
    A = oracle.fill_normal(batch * M * K, 271, 0, 0.1).reshape(batch, M, K)
    Bt = oracle.fill_normal(batch * N * K, 272, 0, 0.1).reshape(batch, N, K)
    Ct = oracle.fill_normal(batch * P * N, 273, 0, 0.1).reshape(batch, P, N)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    dA, dB, dC = dev(A, device), dev(Bt, device), dev(Ct, device)
    got = tcu.b2b_gemm(dA, dB, dC, out_dtype=dt, algo="tile_resident")
    auto = tcu.b2b_gemm(dA, dB, dC, out_dtype=dt)
    torch.cuda.synchronize()
    assert torch.equal(got, auto)
    rows = slice(0, min(M, 128))
    ref = oracle.b2b_gemm(np.ascontiguousarray(A[:, rows]), Bt, Ct)
    assert oracle.max_rel_err(host(got)[:, rows], ref, eps=1.0) <= REL_TOL
    if N == 128:
        tile = tcu.b2b_gemm(dA, dB, dC, out_dtype=dt, algo="tile_library")
        assert oracle.max_rel_err(host(tile)[:, rows], ref, eps=1.0) <= REL_TOL


@pytest.mark.parametrize("algo", ["tile_library", "resident"])
@pytest.mark.parametrize("M,batch,out_dtype", [(32, 1, "f32"), (96, 3, "f16"), (8192, 1, "f16"), (16384, 2, "f32")])
def test_b2b_gemm_both_kernels_at_256x128x128(tcu, oracle, device, algo, M, batch, out_dtype):
    """(N, K, P) = (256, 128, 128): the tile-library kernel and the LDS-resident kernel against the oracle, one
    workgroup, ragged workgroup counts, the C3 size and a two-item batch; plus a one-hot probe of the index maps."""
    import torch

    print(f"b2b {algo} M{M} b{batch} {out_dtype}", flush=True)
    N, K, P = 256, 128, 128
    A = oracle.fill_normal(batch * M * K, 71, 0, 0.1).reshape(batch, M, K)
    Bt = oracle.fill_normal(batch * N * K, 72, 0, 0.1).reshape(batch, N, K)
    Ct = oracle.fill_normal(batch * P * N, 73, 0, 0.1).reshape(batch, P, N)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    D = tcu.b2b_gemm(dev(A, device), dev(Bt, device), dev(Ct, device), out_dtype=dt, algo=algo)
    torch.cuda.synchronize()
    rows = slice(0, M) if M <= 256 else slice(M // 2 - 48, M // 2 + 48)
    ref = oracle.b2b_gemm(np.ascontiguousarray(A[:, rows]), Bt, Ct)
    assert oracle.max_rel_err(host(D)[:, rows], ref, eps=1.0) <= REL_TOL
    if M == 96:
        # D[m, p] = A[m, k] B[k, n] C[n, p] with one-hot operands: exact, and wrong if any index is permuted
        A1 = torch.zeros(1, 96, K, dtype=torch.float16, device=device)
        B1 = torch.zeros(1, N, K, dtype=torch.float16, device=device)
        C1 = torch.zeros(1, P, N, dtype=torch.float16, device=device)
        for i, (m, k, n, p) in enumerate([(0, 0, 0, 0), (95, 127, 255, 127), (37, 5, 200, 66), (64, 77, 13, 1)]):
            A1[0, m, k] = 1.0 + i
            B1[0, n, k] = 2.0
            C1[0, p, n] = 0.5
        D1 = tcu.b2b_gemm(A1, B1, C1, out_dtype=torch.float32, algo=algo)
        want = (A1[0].float() @ B1[0].float().T) @ C1[0].float().T
        assert torch.equal(D1[0], want)


@pytest.mark.parametrize("M,batch,out_dtype", [(64, 1, "f32"), (192, 3, "f16"), (320, 2, "f32"), (8192, 1, "f16"),
                                               (65536, 1, "f16"), (4096, 40, "f32")])
def test_b2b_gemm_many_rows_kernel(tcu, oracle, device, M, batch, out_dtype):
    """(N, K, P) = (256, 128, 128) with the kernel for many rows: workgroups that keep both weight blocks and walk over
    blocks of 256 rows, a wavefront owning 64 rows (its intermediate never leaves its registers). One wavefront, partly
    filled blocks, several blocks per workgroup, batches with more items than workgroups per item; against the oracle on
    rows from the first, a middle and the last block, against the LDS-resident kernel everywhere, a one-hot probe of the
    index maps; AUTO takes this kernel from 32768 rows."""
    import torch

    print(f"b2b rows M{M} b{batch} {out_dtype}", flush=True)
    N, K, P = 256, 128, 128
    A = oracle.fill_normal(batch * M * K, 171, 0, 0.1).reshape(batch, M, K)
    Bt = oracle.fill_normal(batch * N * K, 172, 0, 0.1).reshape(batch, N, K)
    Ct = oracle.fill_normal(batch * P * N, 173, 0, 0.1).reshape(batch, P, N)
    dt = torch.float32 if out_dtype == "f32" else torch.float16
    dA, dB, dC = dev(A, device), dev(Bt, device), dev(Ct, device)
    D = tcu.b2b_gemm(dA, dB, dC, out_dtype=dt, algo="rows")
    torch.cuda.synchronize()
    rows = sorted(set(list(range(0, min(M, 64))) + list(range(M // 2, min(M, M // 2 + 32))) + list(range(M - 32, M))))
    items = sorted({0, batch - 1})
    ref = oracle.b2b_gemm(np.ascontiguousarray(A[items][:, rows]), Bt[items], Ct[items])
    assert oracle.max_rel_err(host(D)[items][:, rows], ref, eps=1.0) <= REL_TOL
    other = tcu.b2b_gemm(dA, dB, dC, out_dtype=dt, algo="resident")
    assert oracle.max_rel_err(host(D), host(other), eps=1.0) <= REL_TOL
    if (long_enough := M * batch >= 32768):
        assert torch.equal(D, tcu.b2b_gemm(dA, dB, dC, out_dtype=dt, algo="auto"))
    if M == 192:
        A1 = torch.zeros(1, 192, K, dtype=torch.float16, device=device)
        B1 = torch.zeros(1, N, K, dtype=torch.float16, device=device)
        C1 = torch.zeros(1, P, N, dtype=torch.float16, device=device)
        for i, (m, k, n, p) in enumerate([(0, 0, 0, 0), (191, 127, 255, 127), (37, 5, 200, 66), (64, 77, 13, 1),
                                          (130, 40, 147, 93)]):
            A1[0, m, k] = 1.0 + i
            B1[0, n, k] = 2.0
            C1[0, p, n] = 0.5
        D1 = tcu.b2b_gemm(A1, B1, C1, out_dtype=torch.float32, algo="rows")
        want = (A1[0].float() @ B1[0].float().T) @ C1[0].float().T
        assert torch.equal(D1[0], want)
    with pytest.raises(RuntimeError):
        tcu.b2b_gemm(dA[:, :32].contiguous(), dB, dC, algo="rows")  # M must be a multiple of 64


def test_kernels_in_a_hip_graph_replay_like_eager(tcu, oracle, device):
    """Launch-bound callers capture these entry points in HIP graphs: several replays, with eager work and
    synchronisations in between, each give the eager result (operands changed between replays)."""
    import torch

    M, N, K, P = 1024, 256, 128, 128
    A = dev(oracle.fill_normal(M * K, 81, 0, 0.1).reshape(1, M, K), device)
    Bt = dev(oracle.fill_normal(N * K, 82, 0, 0.1).reshape(1, N, K), device)
    Ct = dev(oracle.fill_normal(P * N, 83, 0, 0.1).reshape(1, P, N), device)
    D = torch.empty(1, M, P, dtype=torch.float16, device=device)
    G = torch.empty(M, N, dtype=torch.float16, device=device)
    tcu.b2b_gemm(A, Bt, Ct, out=D)
    tcu.gemm(A[0], Bt[0], out=G)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            tcu.b2b_gemm(A, Bt, Ct, out=D)
            tcu.gemm(A[0], Bt[0], out=G)
    torch.cuda.synchronize()
    for rep in range(4):
        A.mul_(-0.5 if rep % 2 else 1.5)  # eager work between the replays
        torch.cuda.synchronize()
        D.zero_()
        G.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(D, tcu.b2b_gemm(A, Bt, Ct)), f"replay {rep}"
        assert torch.equal(G, tcu.gemm(A[0], Bt[0])), f"replay {rep}"


def test_b2b_gemm_config3(tcu, oracle, device):
    """C3: A [8192x128], B [128x256], C [256x128], N(0, 0.1), f16 D."""
    import torch

    print("b2b C3", flush=True)
    M, N, K, P = 8192, 256, 128, 128
    A = oracle.fill_normal(M * K, 1237, 0, 0.1).reshape(M, K)
    Bt = oracle.fill_normal(N * K, 2237, 0, 0.1).reshape(N, K)
    Ct = oracle.fill_normal(P * N, 3237, 0, 0.1).reshape(P, N)
    D = tcu.b2b_gemm(dev(A, device), dev(Bt, device), dev(Ct, device), out_dtype=torch.float16)
    torch.cuda.synchronize()
    assert oracle.max_rel_err(host(D), oracle.b2b_gemm(A, Bt, Ct), eps=1.0) <= REL_TOL
    # identity second operand: D = f16(A B)
    eye = np.eye(N, dtype=np.float16)[:P].copy()  # C[n, p] = delta(n, p), stored [P, N]
    D2 = tcu.b2b_gemm(dev(A, device), dev(Bt, device), dev(eye, device), out_dtype=torch.float32)
    want = oracle.gemm(A, Bt)[:, :P]
    assert oracle.max_rel_err(host(D2), want.astype(np.float16).astype(np.float32), eps=1.0) <= REL_TOL


# ------------------------------------------------------------------------------ attention
@pytest.mark.parametrize("n", [64, 128, 256])
def test_flash_attention_reference_shapes(tcu, oracle, device, n):
    """The three shapes of the reference's tests/python/test_flash_attn.py (m=64, k=p=128), driven
    through the mirror of its TiledFlashAttention wrapper (K as [k, n], V as [n, p], scale 1).
    The reference accepts 8e-2; the bar here is 1e-2."""
    import torch

    print(f"attention reference shape n={n}", flush=True)
    m, k, p = 64, 128, 128
    Q = oracle.fill_normal(m * k, 1234).reshape(m, k)
    Kmat = oracle.fill_normal(k * n, 1235).reshape(k, n)
    V = oracle.fill_normal(n * p, 1236).reshape(n, p)
    op = tcu.TiledFlashAttention(dev(Q, device), dev(Kmat, device), dev(V, device))
    O = op.forward()
    torch.cuda.synchronize()
    assert tuple(O.shape) == (m, p) and O.dtype == torch.float16
    ref = oracle.attention(Q, np.ascontiguousarray(Kmat.T), V, 1.0)
    assert oracle.max_abs_err(host(O), ref) <= ABS_TOL


@pytest.mark.parametrize("algo", ["tile_library", "mfma32", "mfma32_fused", "wave64", "wave64_k32"])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("q_gain,k_growth,tol", [(2.0, 3.0, ABS_TOL), (4.0, 8.0, 5e-2)])
def test_flash_attention_growing_maxima(tcu, oracle, device, algo, D, q_gain, k_growth, tol):
    """Keys whose norm grows along the sequence and large queries: the row maxima move in many key blocks, so the
    rescale path of mfma32 and the failed-speculation path of mfma32_fused run all the time; also a block of
    keys far *below* the maximum (probabilities that underflow) and one query row of zeros (uniform weights); in the
    one-wavefront kernels (wave64, wave64_k32) the re-basing path runs in many steps.
    First setting: logits up to about +-30, the usual tolerance. Second setting: logits up to about +-150, where
    near-ties between the top keys are decided by the rounding of the scores themselves (the tuned kernels take
    Q pre-multiplied by scale * log2(e) in f16: relative error 2^-11 per product term), hence the looser bound."""
    import torch

    if algo == "wave64" and D != 128:
        pytest.skip("the wave64 kernel is instantiated for head size 128")
    batch, M, N = 2, 256, 1024
    q = oracle.fill_normal(batch * M * D, 51).reshape(batch, M, D).astype(np.float32) * q_gain
    k = oracle.fill_normal(batch * N * D, 52).reshape(batch, N, D).astype(np.float32)
    k *= (1.0 + k_growth * np.arange(N, dtype=np.float32) / N)[None, :, None]
    k[:, 512:576] *= 0.01
    q[:, 7] = 0.0
    v = oracle.fill_normal(batch * N * D, 53).reshape(batch, N, D)
    q, k = q.astype(np.float16), k.astype(np.float16)
    O = tcu.flash_attention(dev(q, device), dev(k, device), dev(v, device), algo=algo)
    torch.cuda.synchronize()
    ref = oracle.attention(q, k, v, 1.0 / math.sqrt(D))
    assert np.isfinite(host(O)).all()
    assert oracle.max_abs_err(host(O), ref) <= tol


@pytest.mark.parametrize("q_gain,bound_tile,bound_tuned", [(1.0, 3e-4, 3e-4), (3.0, 1.5e-3, 3e-3), (6.0, 1.5e-3, 7e-3)])
def test_flash_attention_prescaled_q_precision(tcu, oracle, device, q_gain, bound_tile, bound_tuned):
    """The tuned kernels multiply Q by scale * log2(e) and round it to f16 *before* the score MFMAs (a relative error
    of 2^-11 on every product term, so the error of a logit grows with its magnitude); the tile-library kernel, like
    the reference, scales the f32 scores. Each path gets its own bound (about 1.6 x what is measured), at logits up to
    about +-5, +-14 and +-29, so that a regression of either is visible: measured 1.4e-4 / 1.2e-4, 9.6e-4 / 1.7e-3,
    9.9e-4 / 4.4e-3 (tile library / tuned)."""
    import torch

    batch, M, N, D = 2, 256, 1024, 128
    q = (oracle.fill_normal(batch * M * D, 71).reshape(batch, M, D).astype(np.float32) * q_gain).astype(np.float16)
    k = oracle.fill_normal(batch * N * D, 72).reshape(batch, N, D)
    v = oracle.fill_normal(batch * N * D, 73).reshape(batch, N, D)
    ref = oracle.attention(q, k, v, 1.0 / math.sqrt(D))
    for algo in ("tile_library", "mfma32", "mfma32_fused", "wave64", "wave64_k32"):
        O = tcu.flash_attention(dev(q, device), dev(k, device), dev(v, device), algo=algo)
        torch.cuda.synchronize()
        err = oracle.max_abs_err(host(O), ref)
        assert err <= (bound_tile if algo == "tile_library" else bound_tuned), (algo, err)


@pytest.mark.parametrize("algo", ["tile_library", "mfma32", "mfma32_fused"])
@pytest.mark.parametrize("batch,M,N,D", [(1, 64, 64, 128), (3, 128, 192, 128), (2, 256, 512, 128), (2, 128, 256, 64),
                                         (1, 512, 1024, 128), (2, 192, 64, 64)])
def test_flash_attention_row_major_v(tcu, oracle, device, batch, M, N, D, algo):
    import torch

    print(f"attention {algo} b{batch} {M}x{N}x{D}", flush=True)
    q = oracle.fill_normal(batch * M * D, 21).reshape(batch, M, D)
    k = oracle.fill_normal(batch * N * D, 22).reshape(batch, N, D)
    v = oracle.fill_normal(batch * N * D, 23).reshape(batch, N, D)
    O = tcu.flash_attention(dev(q, device), dev(k, device), dev(v, device), algo=algo)
    torch.cuda.synchronize()
    ref = oracle.attention(q, k, v, 1.0 / math.sqrt(D))
    assert oracle.max_abs_err(host(O), ref) <= ABS_TOL


@pytest.mark.parametrize("batch,M,N", [(1, 256, 64), (3, 256, 128), (2, 512, 192), (1, 256, 256), (2, 256, 320),
                                       (1, 512, 384), (2, 256, 448), (1, 256, 576), (8, 512, 1024), (3, 768, 2112)])
def test_flash_attention_wave64_sequence_lengths(tcu, oracle, device, batch, M, N):
    """The kernel with 64 queries per wavefront, at every count of 64-key blocks that takes a different way through
    its prologue, its ring of five LDS stages and its peeled last block-iterations (1 ... 7, 9, 16, 33 blocks)."""
    import torch

    print(f"attention wave64 b{batch} {M}x{N}", flush=True)
    D = 128
    q = oracle.fill_normal(batch * M * D, 61).reshape(batch, M, D)
    k = oracle.fill_normal(batch * N * D, 62).reshape(batch, N, D)
    v = oracle.fill_normal(batch * N * D, 63).reshape(batch, N, D)
    O = tcu.flash_attention(dev(q, device), dev(k, device), dev(v, device), algo="wave64")
    torch.cuda.synchronize()
    ref = oracle.attention(q, k, v, 1.0 / math.sqrt(D))
    assert np.isfinite(host(O)).all()
    assert oracle.max_abs_err(host(O), ref) <= ABS_TOL


@pytest.mark.parametrize("batch,m,n", [(1, 64, 64), (1, 64, 192), (2, 128, 448), (3, 320, 256), (1, 256, 1088),
                                       (8, 512, 2048), (64, 2048, 2048)])
def test_flash_attention_fwd_op_convention_any_key_count(tcu, oracle, device, batch, m, n):
    """The reference op's call shape (flattened tensors, K as [n, k], V column-major = stored [p, n], scale 1) at key
    counts the reference op does not dispatch (it knows n in {64, 128, 256} at batch 1): the kernel with 64 queries per
    wavefront in its column-major-V form (keys re-ordered inside the score tiles, plain 16-byte reads of V), also with
    query counts that leave wavefronts of the last workgroup idle, up to the C4 problem in this layout."""
    import torch

    print(f"attention op convention b{batch} m{m} n{n}", flush=True)
    k = p = 128
    Q = oracle.fill_normal(batch * m * k, 81).reshape(batch, m, k) * np.float16(0.3)
    Kn = oracle.fill_normal(batch * n * k, 82).reshape(batch, n, k) * np.float16(0.3)
    V = oracle.fill_normal(batch * n * p, 83).reshape(batch, n, p)
    Vt = np.ascontiguousarray(V.transpose(0, 2, 1))
    O = torch.full((batch * m * p,), float("nan"), dtype=torch.float16, device=device)
    tcu.flash_attention_fwd(dev(Q, device).flatten(), dev(Kn, device).flatten(), dev(Vt, device).flatten(), O, m, n, k, p,
                            batch=batch)
    torch.cuda.synchronize()
    got = host(O).reshape(batch, m, p)
    assert np.isfinite(got).all()
    items = range(batch) if batch <= 8 else (0, 21, batch - 1)
    for b in items:
        rows = (0, m) if m <= 512 else (m - 160, m - 32)
        ref = oracle.attention(Q[b], Kn[b], V[b], 1.0, rows=rows)
        assert oracle.max_abs_err(got[b, rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= ABS_TOL


@pytest.mark.parametrize("batch,M,N", [(2, 64, 128), (1, 192, 384), (3, 320, 64), (2, 448, 704)])
def test_flash_attention_wave64_partial_workgroups(tcu, oracle, device, batch, M, N):
    """Query counts that are multiples of 64 but not of 256: wavefronts of the last workgroup beyond M take part in the
    loads and barriers and write nothing (the output buffer is followed by a guard region that must stay untouched)."""
    import torch

    D = 128
    q = oracle.fill_normal(batch * M * D, 91).reshape(batch, M, D)
    k = oracle.fill_normal(batch * N * D, 92).reshape(batch, N, D)
    v = oracle.fill_normal(batch * N * D, 93).reshape(batch, N, D)
    buf = torch.full((batch * M * D + 256 * D,), 7.0, dtype=torch.float16, device=device)
    out = buf[:batch * M * D].view(batch, M, D)
    tcu.flash_attention(dev(q, device), dev(k, device), dev(v, device), out=out, algo="wave64")
    torch.cuda.synchronize()
    assert oracle.max_abs_err(host(out), oracle.attention(q, k, v, 1.0 / math.sqrt(D))) <= ABS_TOL
    assert bool((buf[batch * M * D:] == 7.0).all())


def test_flash_attention_wave64_maximum_jumps_late(tcu, oracle, device):
    """One key far above everything before it, placed in each half of a 64-key block and in the last block: the
    check on the sum of a 32-key half fails there, and the reference maxima, the output accumulators, the running
    sums and the scores already computed for the following half are all re-based. Also a key of +inf-like weight at
    the very first position (nothing to rescale yet)."""
    import torch

    batch, M, N, D = 2, 256, 640, 128
    q = oracle.fill_normal(batch * M * D, 71).reshape(batch, M, D).astype(np.float32)
    k = oracle.fill_normal(batch * N * D, 72).reshape(batch, N, D).astype(np.float32)
    v = oracle.fill_normal(batch * N * D, 73).reshape(batch, N, D)
    qdir = q / np.linalg.norm(q, axis=-1, keepdims=True)
    for pos, gain in ((0, 30.0), (200, 60.0), (225, 120.0), (300, 200.0), (639, 400.0)):
        # key `pos` points along a different query each time: for that query its logit exceeds all earlier ones by far
        k[:, pos] = qdir[:, pos % M] * gain
    q, k = q.astype(np.float16), k.astype(np.float16)
    O = tcu.flash_attention(dev(q, device), dev(k, device), dev(v, device), algo="wave64")
    torch.cuda.synchronize()
    ref = oracle.attention(q, k, v, 1.0 / math.sqrt(D))
    assert np.isfinite(host(O)).all()
    assert oracle.max_abs_err(host(O), ref) <= 2e-2  # logits of several hundred: see test_flash_attention_growing_maxima


@pytest.mark.parametrize("batch,M,N", [(3, 256, 320), (8, 256, 640), (2, 512, 1024), (64, 2048, 2048)])
def test_flash_attention_tile_wave64_is_wave64(tcu, oracle, device, batch, M, N):
    """The one-wavefront-per-SIMD kernel composed from tile-library functors (tile_wave64) does the arithmetic of the
    hand-indexed one in the same order: bit-identical outputs, at 5 key blocks (the minimum), at sizes with one and two
    rounds of workgroups, and with keys that force the rare re-basing path; and within tolerance of the oracle."""
    import torch

    D = 128
    print(f"attention tile_wave64 b{batch} {M}x{N}", flush=True)
    q = oracle.fill_normal(batch * M * D, 81).reshape(batch, M, D).astype(np.float32)
    k = oracle.fill_normal(batch * N * D, 82).reshape(batch, N, D).astype(np.float32)
    v = oracle.fill_normal(batch * N * D, 83).reshape(batch, N, D)
    if N == 640:
        qdir = q / np.linalg.norm(q, axis=-1, keepdims=True)
        for pos, gain in ((0, 30.0), (200, 60.0), (225, 120.0), (300, 200.0), (639, 400.0)):
            k[:, pos] = qdir[:, pos % M] * gain
    q, k = q.astype(np.float16), k.astype(np.float16)
    dq, dk, dv = dev(q, device), dev(k, device), dev(v, device)
    ref_kernel = tcu.flash_attention(dq, dk, dv, algo="wave64")
    out = torch.full_like(ref_kernel, float("nan"))
    tcu.flash_attention(dq, dk, dv, out=out, algo="tile_wave64")
    torch.cuda.synchronize()
    assert torch.equal(out, ref_kernel)
    heads = [0, batch - 1]
    ref = oracle.attention(np.ascontiguousarray(q[heads, :64]), np.ascontiguousarray(k[heads]), np.ascontiguousarray(v[heads]),
                           1.0 / math.sqrt(D))
    assert oracle.max_abs_err(host(out)[heads, :64], ref) <= (2e-2 if N == 640 else ABS_TOL)


@pytest.mark.parametrize("batch,M,N", [(3, 256, 320), (8, 256, 640), (2, 512, 1024), (5, 768, 448), (64, 2048, 2048),
                                       (203, 1024, 448), (96, 2048, 384), (330, 256, 640), (1300, 256, 320)])
@pytest.mark.parametrize("v_col_major", [False, True])
def test_flash_attention_wave64_k32(tcu, oracle, device, batch, M, N, v_col_major):
    """The one-wavefront-per-SIMD design on the 16x16x32 matrix instruction (wave64_k32): against the oracle on whole
    heads at small sizes and on a sample of rows at the benchmark size, and against the 32x32x16 kernel everywhere (same
    arithmetic up to the order of the sums inside a matrix instruction); at 5 key blocks (the minimum), an odd number of
    blocks, with keys that force the rare re-basing path, and with one, two, three and a ragged number of items per
    workgroup (a workgroup takes its items one after the other and fetches the next one's first operands under the last
    steps of the current one: 5 ring positions x the two-stage regions that wrap around the ring)."""
    import torch

    D = 128
    print(f"attention wave64_k32 b{batch} {M}x{N} v_col_major={v_col_major}", flush=True)
    q = oracle.fill_normal(batch * M * D, 91).reshape(batch, M, D).astype(np.float32)
    k = oracle.fill_normal(batch * N * D, 92).reshape(batch, N, D).astype(np.float32)
    v = oracle.fill_normal(batch * N * D, 93).reshape(batch, N, D)
    if N == 640:
        qdir = q / np.linalg.norm(q, axis=-1, keepdims=True)
        for pos, gain in ((0, 30.0), (200, 60.0), (225, 120.0), (300, 200.0), (639, 400.0)):
            k[:, pos] = qdir[:, pos % M] * gain
    q, k = q.astype(np.float16), k.astype(np.float16)
    dq, dk, dv = dev(q, device), dev(k, device), dev(v, device)
    ref_kernel = tcu.flash_attention(dq, dk, dv, algo="wave64")
    out = torch.full_like(ref_kernel, float("nan"))
    if v_col_major:
        # V as the reference op takes it: the array V^T [D, N] per batch item
        dvt = dv.transpose(1, 2).contiguous()
        tcu.flash_attention_fwd(dq.view(-1), dk.view(-1), dvt.view(-1), out.view(-1), M, N, D, D, scale=1.0 / math.sqrt(D),
                                batch=batch, algo="wave64_k32")
    else:
        tcu.flash_attention(dq, dk, dv, out=out, algo="wave64_k32")
    torch.cuda.synchronize()
    tol = 2e-2 if N == 640 else ABS_TOL
    assert torch.isfinite(out).all()
    assert (out.float() - ref_kernel.float()).abs().max().item() <= tol
    heads = [0, batch - 1]
    rows = M if batch * M * N <= (1 << 21) else 64
    ref = oracle.attention(np.ascontiguousarray(q[heads, :rows]), np.ascontiguousarray(k[heads]), np.ascontiguousarray(v[heads]),
                           1.0 / math.sqrt(D))
    assert oracle.max_abs_err(host(out)[heads, :rows], ref) <= tol
    ref_tail = oracle.attention(np.ascontiguousarray(q[heads, M - 64:]), np.ascontiguousarray(k[heads]),
                                np.ascontiguousarray(v[heads]), 1.0 / math.sqrt(D))
    assert oracle.max_abs_err(host(out)[heads, M - 64:], ref_tail) <= tol


@pytest.mark.parametrize("batch,M,N", [(3, 256, 320), (8, 256, 640), (5, 768, 448), (64, 2048, 2048), (203, 1024, 448),
                                       (330, 256, 640), (1300, 256, 320)])
def test_flash_attention_wave64_k32_head_size_64(tcu, oracle, device, batch, M, N):
    """Head size 64 on the 16x16x32 one-wavefront-per-SIMD kernel (a step of 4 groups instead of 8: every matrix
    instruction carries an exponential): against the oracle and against the 8-wavefront kernel, at the minimum of 5 key
    blocks, an odd number of blocks, keys that force the rare re-basing path, and one to six items per workgroup.
    The keys that force re-basing give logits up to 400; the kernels multiply Q by scale * log2(e) and round it to f16
    once, which moves such a logit by up to ~400 * 2^-11 / sqrt(D) * a few: 0.026 on the output at D = 64 for these
    inputs (0.015 at D = 128), computed on the host from that rounding alone. Hence 3e-2 there."""
    import torch

    D = 64
    print(f"attention wave64_k32 d64 b{batch} {M}x{N}", flush=True)
    q = oracle.fill_normal(batch * M * D, 94).reshape(batch, M, D).astype(np.float32)
    k = oracle.fill_normal(batch * N * D, 95).reshape(batch, N, D).astype(np.float32)
    v = oracle.fill_normal(batch * N * D, 96).reshape(batch, N, D)
    if N == 640:
        qdir = q / np.linalg.norm(q, axis=-1, keepdims=True)
        for pos, gain in ((0, 30.0), (200, 60.0), (225, 120.0), (300, 200.0), (639, 400.0)):
            k[:, pos] = qdir[:, pos % M] * gain
    q, k = q.astype(np.float16), k.astype(np.float16)
    dq, dk, dv = dev(q, device), dev(k, device), dev(v, device)
    ref_kernel = tcu.flash_attention(dq, dk, dv, algo="mfma32_fused")
    out = torch.full_like(ref_kernel, float("nan"))
    tcu.flash_attention(dq, dk, dv, out=out, algo="wave64_k32")
    torch.cuda.synchronize()
    tol = 3e-2 if N == 640 else ABS_TOL
    assert torch.isfinite(out).all()
    assert (out.float() - ref_kernel.float()).abs().max().item() <= tol
    heads = [0, batch - 1]
    rows = M if batch * M * N <= (1 << 21) else 64
    ref = oracle.attention(np.ascontiguousarray(q[heads, :rows]), np.ascontiguousarray(k[heads]), np.ascontiguousarray(v[heads]),
                           1.0 / math.sqrt(D))
    assert oracle.max_abs_err(host(out)[heads, :rows], ref) <= tol
    ref_tail = oracle.attention(np.ascontiguousarray(q[heads, M - 64:]), np.ascontiguousarray(k[heads]),
                                np.ascontiguousarray(v[heads]), 1.0 / math.sqrt(D))
    assert oracle.max_abs_err(host(out)[heads, M - 64:], ref_tail) <= tol
    if N >= 1024 and batch * (M // 256) >= 256:
        # long sequences with a block of 256 queries per CU: what AUTO runs
        auto = tcu.flash_attention(dq, dk, dv)
        assert torch.equal(auto, out)


@pytest.mark.parametrize("batch,M,N,D", [(2, 64, 320, 128), (1, 192, 384, 128), (3, 320, 640, 128), (2, 448, 704, 128),
                                         (130, 576, 1024, 128), (3, 320, 448, 64), (2, 192, 320, 64)])
@pytest.mark.parametrize("v_col_major", [False, True])
def test_flash_attention_wave64_k32_partial_workgroups(tcu, oracle, device, batch, M, N, D, v_col_major):
    """Query counts that are multiples of 64 but not of 256 on the 16x16x32 kernel: the wavefronts of a head's last block
    whose queries lie beyond M take part in the loads and barriers, read the block's first rows in place of their own
    and write nothing (the output is followed by a guard region that must stay untouched) - also as the second and
    third item of a workgroup, whose Q is fetched under the steps of the item before (130 x 3 blocks on 256 CUs)."""
    import torch

    if v_col_major and D != 128:
        pytest.skip("a column-major V is instantiated for head size 128")
    print(f"attention wave64_k32 partial b{batch} {M}x{N}x{D} v_col_major={v_col_major}", flush=True)
    q = oracle.fill_normal(batch * M * D, 97).reshape(batch, M, D)
    k = oracle.fill_normal(batch * N * D, 98).reshape(batch, N, D)
    v = oracle.fill_normal(batch * N * D, 99).reshape(batch, N, D)
    dq, dk, dv = dev(q, device), dev(k, device), dev(v, device)
    buf = torch.full((batch * M * D + 256 * D,), 7.0, dtype=torch.float16, device=device)
    out = buf[:batch * M * D].view(batch, M, D)
    if v_col_major:
        dvt = dv.transpose(1, 2).contiguous()
        tcu.flash_attention_fwd(dq.view(-1), dk.view(-1), dvt.view(-1), out.view(-1), M, N, D, D, scale=1.0 / math.sqrt(D),
                                batch=batch, algo="wave64_k32")
    else:
        tcu.flash_attention(dq, dk, dv, out=out, algo="wave64_k32")
    torch.cuda.synchronize()
    assert bool((buf[batch * M * D:] == 7.0).all())
    heads = list(range(batch)) if batch <= 3 else [0, 57, batch - 1]
    ref = oracle.attention(np.ascontiguousarray(q[heads]), np.ascontiguousarray(k[heads]), np.ascontiguousarray(v[heads]),
                           1.0 / math.sqrt(D))
    assert oracle.max_abs_err(host(out)[heads], ref) <= ABS_TOL
    if batch > 3:  # every head, against the 8-wavefront kernel
        other = tcu.flash_attention(dq, dk, dv, algo="mfma32_fused")
        assert (out.float() - other.float()).abs().max().item() <= ABS_TOL


@pytest.mark.parametrize("algo", ["wave64", "tile_wave64", "wave64_k32"])
def test_flash_attention_wave64_with_cold_caches(tcu, oracle, device, algo):
    """The one-wavefront-per-SIMD kernels request their first operand fragments of key block 1 only behind the barrier
    that says every wavefront's quarter of the block has landed. (They once did so before it: right whenever the block
    came from the L2 in time, wrong rows in a few heads when it did not.) Every launch here starts with the caches
    evicted and is compared with the 8-wavefront kernel, which shares none of that code."""
    import torch

    B, S, D = 64, 2048, 128
    print(f"attention {algo} with cold caches", flush=True)
    g = torch.Generator(device="cpu").manual_seed(7)
    q, k, v = (torch.randn(B, S, D, generator=g).half().to(device) for _ in range(3))
    ref = tcu.flash_attention(q, k, v, algo="mfma32")
    evict = torch.zeros(256 << 20, device=device)  # 1 GiB: larger than every cache level
    for _ in range(12):
        evict.add_(1.0)
        out = torch.full_like(ref, float("nan"))
        tcu.flash_attention(q, k, v, out=out, algo=algo)
        torch.cuda.synchronize()
        assert torch.isfinite(out).all()
        assert (out.float() - ref.float()).abs().max().item() <= 1e-3


def test_flash_attention_properties(tcu, oracle, device):
    """Size-independent properties: constant V, zero scale, joint permutation of keys/values."""
    import torch

    B, S, D = 2, 256, 128
    q = dev(oracle.fill_normal(B * S * D, 31).reshape(B, S, D), device)
    k = dev(oracle.fill_normal(B * S * D, 32).reshape(B, S, D), device)
    v = dev(oracle.fill_normal(B * S * D, 33).reshape(B, S, D), device)
    vconst = v[:, :1, :].expand(B, S, D).contiguous()
    O = tcu.flash_attention(q, k, vconst)
    assert torch.allclose(O.float(), vconst.float(), atol=2e-3)
    O0 = tcu.flash_attention(q, k, v, scale=0.0)
    assert torch.allclose(O0.float(), v.float().mean(1, keepdim=True).expand(B, S, D), atol=2e-3)
    perm = torch.randperm(S, device=device, generator=torch.Generator(device=device).manual_seed(1))
    O1 = tcu.flash_attention(q, k, v)
    O2 = tcu.flash_attention(q, k[:, perm].contiguous(), v[:, perm].contiguous())
    assert torch.allclose(O1.float(), O2.float(), atol=4e-3)
    # the two tuned kernels compute the same thing
    O3 = tcu.flash_attention(q, k, v, algo="mfma32")
    assert torch.allclose(O1.float(), O3.float(), atol=2e-3)


def test_flash_attention_config4(tcu, oracle, device):
    """C4: [4, 16, 2048, 128], N(0, 1), scale 1/sqrt(128). Oracle on sampled (batch, head, row
    window) slices plus the constant-V property on the full shape."""
    import torch

    print("attention C4", flush=True)
    B, H, S, D = 4, 16, 2048, 128
    n = B * H * S * D
    q = oracle.fill_normal(n, 1238).reshape(B * H, S, D)
    k = oracle.fill_normal(n, 2238).reshape(B * H, S, D)
    v = oracle.fill_normal(n, 3238).reshape(B * H, S, D)
    dq, dk, dv = (dev(t.reshape(B, H, S, D), device) for t in (q, k, v))
    scale = 1.0 / math.sqrt(D)
    samples = [(0, (0, 128)), (17, (960, 1088)), (63, (1920, 2048))]
    refs = [oracle.attention(q[head], k[head], v[head], scale, rows=rows) for head, rows in samples]
    for algo in ("auto", "wave64", "mfma32_fused"):  # auto is wave64 at this shape
        O = tcu.flash_attention(dq, dk, dv, algo=algo)
        torch.cuda.synchronize()
        assert tuple(O.shape) == (B, H, S, D)
        Oh = host(O).reshape(B * H, S, D)
        assert np.isfinite(Oh).all()
        for (head, rows), ref in zip(samples, refs):
            assert oracle.max_abs_err(Oh[head, rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= ABS_TOL, algo
    vconst = dv[:, :, :1, :].expand(B, H, S, D).contiguous()
    Oc = tcu.flash_attention(dq, dk, vconst)
    assert torch.allclose(Oc.float(), vconst.float(), atol=2e-3)


def test_unsupported_shape_raises_runtime_error(tcu, device):
    """The reference op throws std::runtime_error("Unsupported shape") -> Python RuntimeError."""
    import torch

    q = torch.zeros(64 * 128, dtype=torch.float16, device=device)
    kk = torch.zeros(100 * 128, dtype=torch.float16, device=device)
    o = torch.zeros(64 * 128, dtype=torch.float16, device=device)
    with pytest.raises(RuntimeError):
        tcu.flash_attention_fwd(q, kk, kk, o, 64, 100, 128, 128)  # the key count must be a multiple of 64
    with pytest.raises(RuntimeError):
        tcu.gemm(torch.zeros(100, 64, dtype=torch.float16, device=device),
                 torch.zeros(64, 64, dtype=torch.float16, device=device))


# ------------------------------------------------------------------------------ LSTM
@pytest.mark.parametrize("algo", ["tile_library", "streaming"])
@pytest.mark.parametrize("T,B,I,H,with_state", [(1, 64, 128, 128, False), (4, 64, 128, 128, True),
                                                (3, 128, 64, 128, True), (2, 256, 128, 128, True),
                                                (3, 64, 256, 128, True)])
def test_lstm_small(tcu, oracle, device, T, B, I, H, with_state, algo):
    import torch

    if (algo, I) in (("streaming", 64), ("tile_library", 256)):
        pytest.skip("this (I, H) is instantiated for the other kernel only")
    print(f"lstm {algo} T{T} B{B} I{I} H{H} state={with_state}", flush=True)
    x = oracle.fill_normal(T * B * I, 41, 0, 0.5).reshape(T, B, I)
    W = oracle.fill_normal(4 * H * (I + H), 42, 0, 0.1).reshape(4 * H, I + H)
    b = oracle.fill_normal(4 * H, 43, 0, 0.1)
    h0 = oracle.fill_normal(B * H, 44, 0, 0.5).reshape(B, H) if with_state else None
    c0 = oracle.fill_normal(B * H, 45, 0, 0.5).reshape(B, H).astype(np.float32) if with_state else None
    h_all, c_T = tcu.lstm(dev(x, device), dev(W, device), dev(b, device),
                          dev(h0, device) if with_state else None, dev(c0, device) if with_state else None, algo=algo)
    torch.cuda.synchronize()
    h_ref, c_ref = oracle.lstm(x, W, b, h0, c0)
    assert oracle.max_abs_err(host(h_all), h_ref) <= ABS_TOL
    assert oracle.max_abs_err(host(c_T), c_ref) <= ABS_TOL


@pytest.mark.parametrize("T,B,I,H", [(4, 64, 128, 128), (2, 128, 256, 128), (8, 64, 128, 128), (4, 64, 512, 512),
                                     (2, 128, 384, 256), (4, 64, 128, 640), (4, 64, 768, 128)])
@pytest.mark.parametrize("with_state", [False, True])
def test_lstm_hoisted_input_projection(tcu, oracle, device, T, B, I, H, with_state):
    """tcu_lstm_f16_ws: the input half of the gates from one GEMM over all steps, then steps over h only; against the
    oracle, against the per-step streaming kernel, with a caller-owned workspace larger than needed, and twice in a row
    on the same workspace. Both kernels take any I and H in multiples of 128 (sizes as kernel arguments)."""
    import torch

    print(f"lstm hoisted T{T} B{B} I{I} H{H} state={with_state}", flush=True)
    x = oracle.fill_normal(T * B * I, 51, 0, 0.5).reshape(T, B, I)
    W = oracle.fill_normal(4 * H * (I + H), 52, 0, 0.1).reshape(4 * H, I + H)
    b = oracle.fill_normal(4 * H, 53, 0, 0.1)
    h0 = oracle.fill_normal(B * H, 54, 0, 0.5).reshape(B, H) if with_state else None
    c0 = oracle.fill_normal(B * H, 55, 0, 0.5).reshape(B, H).astype(np.float32) if with_state else None
    args = (dev(x, device), dev(W, device), dev(b, device), dev(h0, device) if with_state else None,
            dev(c0, device) if with_state else None)
    need = tcu.lstm_workspace_bytes(T, B, I, H)
    assert need == T * B * 4 * H * 4
    ws = torch.full((need + 4096,), 0xFF, dtype=torch.uint8, device=device)  # NaN patterns: nothing may be read unwritten
    h_ref, c_ref = oracle.lstm(x, W, b, h0, c0)
    h_str, c_str = tcu.lstm(*args, algo="streaming")
    for rep in range(2):
        h_all, c_T = tcu.lstm(*args, algo="hoisted", workspace=ws)
        torch.cuda.synchronize()
        assert oracle.max_abs_err(host(h_all), h_ref) <= ABS_TOL
        assert oracle.max_abs_err(host(c_T), c_ref) <= ABS_TOL
        assert float((h_all.float() - h_str.float()).abs().max()) <= 2e-3
        assert float((c_T - c_str).abs().max()) <= 2e-3
    assert bool((ws[need:] == 0xFF).all())  # nothing written past the stated size


def test_lstm_hoisted_rejects_what_it_cannot_do(tcu, device):
    import torch

    assert tcu.lstm_workspace_bytes(3, 64, 128, 128) == 0  # T * B not a multiple of 256
    assert tcu.lstm_workspace_bytes(4, 64, 64, 64) == 0    # I, H not multiples of 128
    x = torch.zeros(4, 64, 128, dtype=torch.float16, device=device)
    W = torch.zeros(512, 256, dtype=torch.float16, device=device)
    b = torch.zeros(512, dtype=torch.float16, device=device)
    with pytest.raises(RuntimeError):
        tcu.lstm(x, W, b, algo="hoisted", workspace=torch.empty(1024, dtype=torch.uint8, device=device))
    with pytest.raises(RuntimeError):
        tcu.lstm(x[:3].contiguous(), W, b, algo="hoisted")


@pytest.mark.parametrize("T,B,I,H", [(3, 16, 16, 16), (2, 48, 80, 112), (4, 32, 256, 64), (2, 64, 144, 272), (1, 80, 1024, 48)])
@pytest.mark.parametrize("with_state", [False, True])
def test_lstm_any_shape_of_whole_tiles(tcu, oracle, device, T, B, I, H, with_state):
    """Every B, I, H in multiples of 16 runs (the granularity of the tile types): AUTO routes shapes no tuned kernel is
    instantiated for to the run-time-shape step kernel; k ranges that end in a half-filled 32-wide operand tile, hidden
    sizes that leave wavefronts of the last workgroup without work, batches that are not multiples of 64."""
    import torch

    print(f"lstm ragged T{T} B{B} I{I} H{H} state={with_state}", flush=True)
    x = oracle.fill_normal(T * B * I, 81, 0, 0.5).reshape(T, B, I)
    W = oracle.fill_normal(4 * H * (I + H), 82, 0, 0.1).reshape(4 * H, I + H)
    b = oracle.fill_normal(4 * H, 83, 0, 0.1)
    h0 = oracle.fill_normal(B * H, 84, 0, 0.5).reshape(B, H) if with_state else None
    c0 = oracle.fill_normal(B * H, 85, 0, 0.5).reshape(B, H).astype(np.float32) if with_state else None
    h_ref, c_ref = oracle.lstm(x, W, b, h0, c0)
    for algo in ("auto", "ragged"):
        h_all, c_T = tcu.lstm(dev(x, device), dev(W, device), dev(b, device),
                              dev(h0, device) if with_state else None, dev(c0, device) if with_state else None, algo=algo)
        torch.cuda.synchronize()
        assert oracle.max_abs_err(host(h_all), h_ref) <= ABS_TOL
        assert oracle.max_abs_err(host(c_T), c_ref) <= ABS_TOL


def test_lstm_ragged_matches_streaming_kernel(tcu, device):
    """Where both exist, the run-time-shape kernel and the streaming kernel agree to the order of the f32 summation."""
    import torch

    T, B, I, H = 3, 64, 256, 128
    g = torch.Generator(device="cpu").manual_seed(9)
    x = (torch.randn(T, B, I, generator=g) * 0.5).half().to(device)
    W = (torch.randn(4 * H, I + H, generator=g) * 0.1).half().to(device)
    b = (torch.randn(4 * H, generator=g) * 0.1).half().to(device)
    h_a, c_a = tcu.lstm(x, W, b, algo="streaming")
    h_b, c_b = tcu.lstm(x, W, b, algo="ragged")
    assert float((h_a.float() - h_b.float()).abs().max()) <= 2e-3
    assert float((c_a - c_b).abs().max()) <= 2e-3


def test_lstm_zero_weights_closed_form(tcu, device):
    """W = 0: c_t = sigmoid(b_f) c_{t-1} + sigmoid(b_i) tanh(b_g), h_t = sigmoid(b_o) tanh(c_t)."""
    import torch

    T, B, I, H = 5, 64, 128, 128
    x = torch.randn(T, B, I, device=device, generator=torch.Generator(device=device).manual_seed(3)).half()
    W = torch.zeros(4 * H, I + H, dtype=torch.float16, device=device)
    b = (torch.arange(4 * H, device=device).float() / (4 * H) - 0.5).half()
    h_all, c_T = tcu.lstm(x, W, b)
    bi, bf, bg, bo = (b.double()[j * H:(j + 1) * H] for j in range(4))
    c = torch.zeros(H, dtype=torch.float64, device=device)
    for t in range(T):
        c = torch.sigmoid(bf) * c + torch.sigmoid(bi) * torch.tanh(bg)
        h = torch.sigmoid(bo) * torch.tanh(c)
        assert torch.allclose(h_all[t].double(), h.expand(B, H), atol=2e-3)
    assert torch.allclose(c_T.double(), c.expand(B, H), atol=1e-5)


def test_lstm_config5(tcu, oracle, device):
    """C5: batch 256, input 1024, hidden 1024, 16 steps; x, W ~ N(0, 0.05), bias ~ N(0, 0.05), h0=c0=0.
    Oracle on 8 sampled batch rows (rows are independent)."""
    import torch

    print("lstm C5", flush=True)
    T, B, I, H = 16, 256, 1024, 1024
    x = oracle.fill_normal(T * B * I, 1239, 0, 0.05).reshape(T, B, I)
    W = oracle.fill_normal(4 * H * (I + H), 2239, 0, 0.05).reshape(4 * H, I + H)
    b = oracle.fill_normal(4 * H, 3239, 0, 0.05)
    dx, dW, db = dev(x, device), dev(W, device), dev(b, device)
    refs = {rows: oracle.lstm(x, W, b, rows=rows) for rows in [(0, 4), (252, 256)]}
    for algo in ("auto", "hoisted", "persistent"):
        print(f"lstm C5 {algo}", flush=True)
        h_all, c_T = tcu.lstm(dx, dW, db, algo=algo)
        torch.cuda.synchronize()
        hh, cc = host(h_all), host(c_T)
        assert np.isfinite(hh).all() and np.isfinite(cc).all()
        for rows, (h_ref, c_ref) in refs.items():
            assert oracle.max_abs_err(hh[:, rows[0]:rows[1]], h_ref[:, rows[0]:rows[1]]) <= ABS_TOL, algo
            assert oracle.max_abs_err(cc[rows[0]:rows[1]], c_ref[rows[0]:rows[1]]) <= ABS_TOL, algo


@pytest.mark.parametrize("T,B,I,H", [(4, 64, 64, 1024), (8, 32, 192, 1024), (2, 128, 1024, 1024), (1, 256, 64, 1024),
                                     (8, 32, 64, 256), (4, 256, 256, 256), (8, 64, 128, 512), (2, 128, 512, 512),
                                     (8, 96, 64, 768), (16, 256, 768, 768)])
@pytest.mark.parametrize("with_state", [False, True])
def test_lstm_persistent_single_launch(tcu, oracle, device, T, B, I, H, with_state):
    """tcu_lstm_f16_persistent (H = 256, 512, 768, 1024: 8, 16, 24, 32 workgroups per XCD): the time loop in one
    weight-stationary launch, h exchanged inside each XCD. One to eight XCDs in use, one to sixteen steps, with and
    without an initial state; against the oracle and against the hoisted per-step path (same projection GEMM, other
    summation order); twice on one workspace, whose bytes past the stated size stay untouched."""
    import torch

    print(f"lstm persistent T{T} B{B} I{I} H{H} state={with_state}", flush=True)
    x = oracle.fill_normal(T * B * I, 61, 0, 0.5).reshape(T, B, I)
    W = oracle.fill_normal(4 * H * (I + H), 62, 0, 0.03).reshape(4 * H, I + H)
    b = oracle.fill_normal(4 * H, 63, 0, 0.1)
    h0 = oracle.fill_normal(B * H, 64, 0, 0.5).reshape(B, H) if with_state else None
    c0 = oracle.fill_normal(B * H, 65, 0, 0.5).reshape(B, H).astype(np.float32) if with_state else None
    args = (dev(x, device), dev(W, device), dev(b, device), dev(h0, device) if with_state else None,
            dev(c0, device) if with_state else None)
    need = tcu.lstm_persistent_workspace_bytes(T, B, I, H)
    assert need == 4096 + T * B * 4 * H * 2  # the pre-activations of all steps in f16
    ws = torch.full((need + 4096,), 0xFF, dtype=torch.uint8, device=device)
    refs = {rows: oracle.lstm(x, W, b, h0, c0, rows=rows) for rows in [(0, 3), (B - 3, B)]}  # first and last XCD in use
    for rep in range(2):
        h_all, c_T = tcu.lstm(*args, algo="persistent", workspace=ws)
        torch.cuda.synchronize()
        for (r0, r1), (h_ref, c_ref) in refs.items():
            assert oracle.max_abs_err(host(h_all)[:, r0:r1], h_ref[:, r0:r1]) <= ABS_TOL
            assert oracle.max_abs_err(host(c_T)[r0:r1], c_ref[r0:r1]) <= ABS_TOL
    assert bool((ws[need:] == 0xFF).all())
    if tcu.lstm_workspace_bytes(T, B, I, H):
        h_hst, c_hst = tcu.lstm(*args, algo="hoisted")
        assert float((h_all.float() - h_hst.float()).abs().max()) <= 2e-3
        assert float((c_T - c_hst).abs().max()) <= 2e-3


def test_lstm_persistent_bounded_wait(tcu, device, monkeypatch):
    """A workgroup whose peers never all arrive gives up after the time limit, raises the error word and exits; so does
    everyone waiting for it: the launch ends normally and the host is told. Forced from the host: the kernel is told to
    wait for 33 arrivals per XCD where 32 workgroups exist. The next, ordinary call on the same workspace works."""
    import torch

    T, B, I, H = 4, 64, 64, 1024
    g = torch.Generator(device="cpu").manual_seed(5)
    x = (torch.randn(T, B, I, generator=g) * 0.5).half().to(device)
    W = (torch.randn(4 * H, I + H, generator=g) * 0.03).half().to(device)
    b = (torch.randn(4 * H, generator=g) * 0.1).half().to(device)
    ws = torch.empty(tcu.lstm_persistent_workspace_bytes(T, B, I, H), dtype=torch.uint8, device=device)
    good = tcu.lstm(x, W, b, algo="persistent", workspace=ws)
    monkeypatch.setenv("TCU_LSTM_PERSISTENT_PEERS", "33")
    monkeypatch.setenv("TCU_LSTM_PERSISTENT_SPIN_US", "2000")
    print("lstm persistent: forced time-out", flush=True)
    with pytest.raises(RuntimeError, match="waited"):
        tcu.lstm(x, W, b, algo="persistent", workspace=ws)
    monkeypatch.delenv("TCU_LSTM_PERSISTENT_PEERS")
    monkeypatch.delenv("TCU_LSTM_PERSISTENT_SPIN_US")
    again = tcu.lstm(x, W, b, algo="persistent", workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(good[0], again[0]) and torch.equal(good[1], again[1])


def test_lstm_persistent_workspace_at_allocator_granularity(tcu, device):
    """torch's caching allocator hands out blocks in multiples of 512 bytes: a workspace that starts at an odd multiple
    of 512 is a valid argument (the step counters need 128-byte alignment only) and gives the same result."""
    import torch

    T, B, I, H = 4, 64, 64, 1024
    g = torch.Generator(device="cpu").manual_seed(7)
    x = (torch.randn(T, B, I, generator=g) * 0.5).half().to(device)
    W = (torch.randn(4 * H, I + H, generator=g) * 0.03).half().to(device)
    b = (torch.randn(4 * H, generator=g) * 0.1).half().to(device)
    need = tcu.lstm_persistent_workspace_bytes(T, B, I, H)
    buf = torch.empty(need + 2048, dtype=torch.uint8, device=device)
    base = (-buf.data_ptr()) % 1024  # offset of the first 1 KiB boundary inside buf
    print("lstm persistent: workspace at 1 KiB + 512", flush=True)
    aligned = tcu.lstm(x, W, b, algo="persistent", workspace=buf[base:base + need])
    odd = buf[base + 512:base + 512 + need]
    assert odd.data_ptr() % 1024 == 512
    shifted = tcu.lstm(x, W, b, algo="persistent", workspace=odd)
    torch.cuda.synchronize()
    assert torch.equal(aligned[0], shifted[0]) and torch.equal(aligned[1], shifted[1])
    with pytest.raises(RuntimeError, match="aligned"):
        tcu.lstm(x, W, b, algo="persistent", workspace=buf[base + 64:base + 64 + need])


def test_lstm_persistent_rejects_what_it_cannot_do(tcu, device):
    import torch

    assert tcu.lstm_persistent_workspace_bytes(4, 64, 64, 128) == 0    # H not in {256, 512, 768, 1024}
    assert tcu.lstm_persistent_workspace_bytes(4, 64, 64, 2048) == 0
    assert tcu.lstm_persistent_workspace_bytes(4, 48, 64, 1024) == 0   # B not a multiple of 32
    assert tcu.lstm_persistent_workspace_bytes(1, 512, 64, 1024) == 0  # more rows than 8 XCDs x 32
    assert tcu.lstm_persistent_workspace_bytes(3, 64, 64, 1024) == 0   # T * B not a multiple of 256
    x = torch.zeros(4, 64, 64, dtype=torch.float16, device=device)
    W = torch.zeros(4096, 64 + 1024, dtype=torch.float16, device=device)
    b = torch.zeros(4096, dtype=torch.float16, device=device)
    with pytest.raises(RuntimeError):
        tcu.lstm(x, W, b, algo="persistent", workspace=torch.empty(8192, dtype=torch.uint8, device=device))
    with pytest.raises(RuntimeError):
        tcu.lstm(x[:3].contiguous(), W, b, algo="persistent")


def test_smoke_entry(device):
    import __graft_entry__ as g

    g.smoke()
