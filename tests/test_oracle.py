"""Pins the CPU oracle (oracle/oracle.c) before anything is compared against it.

Each oracle function is checked against something that shares no code with it: numpy
float64 arithmetic, closed forms, brute force on tiny inputs, invariants, torch.nn.LSTM,
and the committed golden fixtures (tests/golden/golden_small.npz, written by
tests/golden/make_golden.py). The checks are chosen so that a dropped term, a wrong index
or a transposed operand fails at least one of them.
"""
import os

import numpy as np
import pytest

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "golden_small.npz"))


# ----------------------------------------------------------------------- fp16 conversion
def test_h2f_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    h = bits.view(np.float16)
    got = oracle.h2f(h)
    want = h.astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_f2h_matches_numpy_rounding(oracle):
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10,
        rng.standard_normal(100000).astype(np.float32) * 1e-5,  # subnormal range
        rng.standard_normal(50000).astype(np.float32) * 1e5,    # overflow to inf
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 5.96e-8, 2.98e-8, 2.9802322e-8, 1e-10], np.float32),
    ])
    # exact ties: halfway between two adjacent halves
    h = rng.integers(0, 0x7BFF, 20000).astype(np.uint16).view(np.float16).astype(np.float32)
    h_next = (rng.integers(0, 0x7BFF, 1).astype(np.uint16)).view(np.float16).astype(np.float32)
    ties = (h + np.nextafter(h.astype(np.float16), np.float16(np.inf)).astype(np.float32)) / 2
    x = np.concatenate([x, ties, h_next])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    got = oracle.f2h(x)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


# ----------------------------------------------------------------------- generators
def test_uniform_generator_matches_numpy_restatement(oracle):
    n, seed = 4096, 1234
    got = oracle.fill_uniform(n, seed, -1.0, 1.0)
    z = oracle.splitmix64_at(seed, np.arange(n))
    u = (z >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 16777216.0)
    want = (np.float32(-1.0) + np.float32(2.0) * u).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    assert got.min() >= -1 and got.max() <= 1
    assert abs(float(got.astype(np.float64).mean())) < 0.05
    # distinct seeds give distinct streams, same seed repeats
    assert not np.array_equal(got, oracle.fill_uniform(n, seed + 1))
    assert np.array_equal(got, oracle.fill_uniform(n, seed))


def test_normal_generator_moments_and_restatement(oracle):
    n, seed = 1 << 18, 99
    got = oracle.fill_normal(n, seed, 0.0, 1.0).astype(np.float64)
    assert abs(got.mean()) < 0.01 and abs(got.std() - 1.0) < 0.01
    assert abs(np.mean(got ** 3)) < 0.03 and abs(np.mean(got ** 4) - 3.0) < 0.06
    i = np.arange(4096)
    u1 = ((oracle.splitmix64_at(seed, 2 * i) >> np.uint64(11)).astype(np.float64) + 1.0) / 9007199254740992.0
    u2 = (oracle.splitmix64_at(seed, 2 * i + 1) >> np.uint64(11)).astype(np.float64) / 9007199254740992.0
    want = (np.sqrt(-2.0 * np.log(u1)) * np.cos(2 * np.pi * u2)).astype(np.float32)
    # libm and numpy may differ in the last ulp of log/cos: allow one fp16 ulp on a handful
    diff = np.abs(got[:4096] - want.astype(np.float16).astype(np.float64))
    assert np.count_nonzero(diff) <= 4 and diff.max() <= 2e-3
    scaled = oracle.fill_normal(4096, seed, 1.0, 0.05).astype(np.float64)
    assert abs(scaled.mean() - 1.0) < 0.01 and abs(scaled.std() - 0.05) < 0.005


# ----------------------------------------------------------------------- GEMM
REFERENCE_GEMM_SHAPES = [(16, 16, 16), (16, 32, 16), (96, 48, 80), (64, 128, 128), (128, 64, 256)]


@pytest.mark.parametrize("M,N,K", REFERENCE_GEMM_SHAPES)
def test_gemm_vs_float64(oracle, M, N, K):
    A = oracle.fill_uniform(M * K, 1 + M).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 2 + N).reshape(N, K)
    want = A.astype(np.float64) @ Bt.astype(np.float64).T
    for naive in (False, True):
        got = oracle.gemm(A, Bt, naive=naive)
        assert got.shape == (M, N)
        assert oracle.max_rel_err(got, want) < 2e-4  # f32 accumulation (the naive order is the worst) vs f64


def test_gemm_golden_ramps(oracle):
    for (M, N, K) in [(16, 16, 16), (96, 48, 80), (128, 64, 256)]:
        A, Bt, C = (GOLD[f"gemm_{M}x{N}x{K}_{s}"] for s in ("A", "Bt", "C"))
        assert oracle.max_rel_err(oracle.gemm(A, Bt), C) < 1e-4


def test_gemm_closed_forms(oracle):
    K, N = 32, 48
    Bt = oracle.fill_uniform(N * K, 7).reshape(N, K)
    eye = np.eye(K, dtype=np.float16)
    assert np.array_equal(oracle.gemm(eye, Bt), Bt.astype(np.float32).T)  # I · B = B
    ones = np.ones((5, K), np.float16)
    assert np.allclose(oracle.gemm(ones, np.ones((3, K), np.float16)), K)
    # one-hot probes pin the index convention: C[m, n] = A[m, k] * Bt[n, k]
    A = np.zeros((4, K), np.float16)
    A[2, 5] = 2.0
    B1 = np.zeros((6, K), np.float16)
    B1[4, 5] = 3.0
    C = oracle.gemm(A, B1)
    assert C[2, 4] == 6.0 and np.count_nonzero(C) == 1


def test_gemm_row_window(oracle):
    A = oracle.fill_uniform(64 * 32, 3).reshape(64, 32)
    Bt = oracle.fill_uniform(16 * 32, 4).reshape(16, 32)
    full = oracle.gemm(A, Bt)
    part = oracle.gemm(A, Bt, rows=(16, 40))
    assert np.array_equal(part[16:40], full[16:40]) and not part[:16].any() and not part[40:].any()


# ----------------------------------------------------------------------- back-to-back GEMM
def test_b2b_golden_and_float64(oracle):
    A, Bt, Ct, D = GOLD["b2b_A"], GOLD["b2b_Bt"], GOLD["b2b_Ct"], GOLD["b2b_D"]
    assert oracle.max_rel_err(oracle.b2b_gemm(A, Bt, Ct), D) < 1e-4


def test_b2b_closed_forms(oracle):
    M, N, K, P = 16, 32, 32, 32
    A = oracle.fill_normal(M * K, 5, 0, 0.1).reshape(M, K)
    Bt = oracle.fill_normal(N * K, 6, 0, 0.1).reshape(N, K)
    # C = I  =>  D = f16(A·B) exactly
    D = oracle.b2b_gemm(A, Bt, np.eye(N, dtype=np.float16))
    want = oracle.gemm(A, Bt).astype(np.float16).astype(np.float32)
    assert np.array_equal(D, want)
    # B = I (K == N)  =>  D = A·C
    Ct = oracle.fill_normal(P * N, 8, 0, 0.1).reshape(P, N)
    D2 = oracle.b2b_gemm(A, np.eye(K, dtype=np.float16), Ct)
    assert oracle.max_rel_err(D2, A.astype(np.float64) @ Ct.astype(np.float64).T) < 5e-5
    # batched = each item on its own
    Ab = np.stack([A, A[::-1].copy()])
    Bb = np.stack([Bt, Bt[::-1].copy()])
    Cb = np.stack([Ct, Ct[::-1].copy()])
    Db = oracle.b2b_gemm(Ab, Bb, Cb)
    assert np.array_equal(Db[1], oracle.b2b_gemm(Ab[1], Bb[1], Cb[1]))


# ----------------------------------------------------------------------- attention
def _softmax64(s):
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=-1, keepdims=True)


def test_attention_golden(oracle):
    Q, Kn, V, O, scale = GOLD["attn_Q"], GOLD["attn_Kn"], GOLD["attn_V"], GOLD["attn_O"], float(GOLD["attn_scale"])
    assert oracle.max_abs_err(oracle.attention(Q, Kn, V, scale), O) < 2e-6
    # column-major V (stored [P, N]) is the same function
    assert np.array_equal(oracle.attention(Q, Kn, np.ascontiguousarray(V.T), scale, v_col_major=True),
                          oracle.attention(Q, Kn, V, scale))


def test_attention_special_cases(oracle):
    M, N, K, P = 8, 32, 16, 12
    Q = oracle.fill_normal(M * K, 1).reshape(M, K)
    Kn = oracle.fill_normal(N * K, 2).reshape(N, K)
    V = oracle.fill_normal(N * P, 3).reshape(N, P)
    # V constant along N  =>  O = that constant row
    Vc = np.tile(V[:1], (N, 1))
    assert np.allclose(oracle.attention(Q, Kn, Vc, 0.3), np.tile(V[:1].astype(np.float32), (M, 1)), atol=1e-6)
    # N = 1  =>  O = V
    assert np.allclose(oracle.attention(Q, Kn[:1], V[:1], 0.3), np.tile(V[:1].astype(np.float32), (M, 1)), atol=1e-7)
    # scale = 0  =>  uniform weights: O = mean(V)
    assert np.allclose(oracle.attention(Q, Kn, V, 0.0), np.tile(V.astype(np.float64).mean(0), (M, 1)), atol=1e-6)
    # permuting keys and values together changes nothing
    perm = np.random.default_rng(1).permutation(N)
    assert np.allclose(oracle.attention(Q, Kn[perm].copy(), V[perm].copy(), 0.3), oracle.attention(Q, Kn, V, 0.3),
                       atol=1e-6)
    # float64 restatement
    want = _softmax64(0.3 * (Q.astype(np.float64) @ Kn.astype(np.float64).T)) @ V.astype(np.float64)
    assert oracle.max_abs_err(oracle.attention(Q, Kn, V, 0.3), want) < 2e-6
    # batch items are independent
    Qb = np.stack([Q, Q[::-1].copy()])
    Kb = np.stack([Kn, Kn[::-1].copy()])
    Vb = np.stack([V, V[::-1].copy()])
    assert np.array_equal(oracle.attention(Qb, Kb, Vb, 0.3)[1], oracle.attention(Qb[1], Kb[1], Vb[1], 0.3))


@pytest.mark.parametrize("n", [64, 128, 256])
def test_blockwise_recurrence_equals_softmax(oracle, n):
    """The reference's blocked recurrence (running max from 0, renormalise every block) is the
    same function as the plain softmax; shapes of its Python test (m=64, k=p=128), smaller k."""
    rng = np.random.default_rng(1234)
    M, K, P = 64, 32, 128
    Q = rng.standard_normal((M, K)).astype(np.float16)
    Kmat = (rng.standard_normal((K, n)) * 0.5).astype(np.float16)
    V = rng.standard_normal((n, P)).astype(np.float16)
    plain = oracle.attention(Q, np.ascontiguousarray(Kmat.T), V, 1.0)
    for tn in (n, n // 2, 16):
        blocked = oracle.attention_blocked_f32(Q.astype(np.float32), Kmat.astype(np.float32), V.astype(np.float32), tn)
        assert oracle.max_abs_err(blocked, plain) < 5e-5


# ----------------------------------------------------------------------- LSTM
def _sig(x):
    return 1.0 / (1.0 + np.exp(-x))


def test_lstm_golden_torch(oracle):
    x, W, b, h0, c0 = (GOLD[f"lstm_{s}"] for s in ("x", "W", "b", "h0", "c0"))
    h_all, c_T = oracle.lstm(x, W, b, h0, c0)
    # the fixture never rounds h to f16 between steps; the oracle does (the device keeps h in f16)
    assert oracle.max_abs_err(h_all, GOLD["lstm_h_all"]) < 2e-3
    assert oracle.max_abs_err(c_T, GOLD["lstm_cT"]) < 2e-3
    # step 0 consumes the exact f16 h0, so it must agree to f32 accuracy
    assert oracle.max_abs_err(h_all[0], GOLD["lstm_h_all"][0]) < 2e-6


def test_lstm_single_step_closed_form(oracle):
    B, I, H = 5, 16, 8
    x = oracle.fill_normal(B * I, 1, 0, 0.5).reshape(1, B, I)
    W = oracle.fill_normal(4 * H * (I + H), 2, 0, 0.2).reshape(4 * H, I + H)
    b = oracle.fill_normal(4 * H, 3, 0, 0.2)
    gates = x[0].astype(np.float64) @ W[:, :I].astype(np.float64).T + b.astype(np.float64)  # h0 = 0
    i, f, g, o = (gates[:, j * H:(j + 1) * H] for j in range(4))
    c = _sig(i) * np.tanh(g)  # c0 = 0
    h = _sig(o) * np.tanh(c)
    h_all, c_T = oracle.lstm(x, W, b)
    assert oracle.max_abs_err(c_T, c) < 2e-6 and oracle.max_abs_err(h_all[0], h) < 2e-6
    # gate order matters: swapping the f and g rows of W must change the answer
    W2 = W.copy()
    W2[H:2 * H], W2[2 * H:3 * H] = W[2 * H:3 * H], W[H:2 * H]
    assert oracle.max_abs_err(oracle.lstm(x, W2, b)[1], c) > 1e-3


def test_lstm_zero_weights_recurrence(oracle):
    T, B, I, H = 6, 2, 4, 4
    x = oracle.fill_normal(T * B * I, 9).reshape(T, B, I)
    W = np.zeros((4 * H, I + H), np.float16)
    b = oracle.fill_normal(4 * H, 4, 0, 0.5)
    bi, bf, bg, bo = (b.astype(np.float64)[j * H:(j + 1) * H] for j in range(4))
    c = np.zeros(H)
    hs = []
    for _ in range(T):
        c = _sig(bf) * c + _sig(bi) * np.tanh(bg)
        hs.append(_sig(bo) * np.tanh(c))
    h_all, c_T = oracle.lstm(x, W, b)
    assert oracle.max_abs_err(c_T, np.tile(c, (B, 1))) < 2e-6
    assert oracle.max_abs_err(h_all[:, 0], np.array(hs)) < 2e-6


def test_lstm_batch_window(oracle):
    T, B, I, H = 3, 6, 8, 8
    x = oracle.fill_normal(T * B * I, 9).reshape(T, B, I)
    W = oracle.fill_normal(4 * H * (I + H), 2, 0, 0.2).reshape(4 * H, I + H)
    b = oracle.fill_normal(4 * H, 3, 0, 0.2)
    full_h, full_c = oracle.lstm(x, W, b)
    part_h, part_c = oracle.lstm(x, W, b, rows=(2, 4))
    assert np.array_equal(part_h[:, 2:4], full_h[:, 2:4]) and np.array_equal(part_c[2:4], full_c[2:4])


# ----------------------------------------------------------------------- index semantics
def test_layout_and_iterator_index_helpers(oracle):
    # reference tests/cpp/cell/test_layout.cu:105-131: RowMajor<4,7> strides (7,1), ColMajor<4,7> (1,4)
    assert oracle.matrix_layout_offset(2, 3, 7, 1) == 17
    assert oracle.matrix_layout_offset(2, 3, 1, 4) == 14
    # reference tests/cpp/cell/test_global_tile_iterator.cu:35-74: 4x9 tile, 2x3 chunks
    for i in range(2):
        for j in range(3):
            assert oracle.gtile_iterator_offset(i, j, 4, 9, 2, 3, True) == i * 2 * 9 + j * 3
            assert oracle.gtile_iterator_offset(i, j, 4, 9, 2, 3, False) == i * 2 + j * 3 * 4
    assert oracle.warp_tile_origin(1, 1, 64, 32, 2, 2, "cont") == (32, 16, 32, 16)
    assert oracle.warp_tile_origin(1, 1, 64, 32, 2, 2, "row_reuse_cont") == (32, 0, 32, 32)
    assert oracle.warp_tile_origin(1, 1, 64, 32, 2, 2, "col_reuse_cont") == (0, 16, 64, 16)


def test_error_metric_floor(oracle):
    ref = np.array([100.0, -50.0, 1e-6])
    x = ref + np.array([0.01, 0.01, 0.01])
    # the tiny reference value is floored at eps * rms, so the ratio stays bounded
    assert oracle.max_rel_err(x, ref) < 0.02
    assert oracle.max_rel_err(ref, ref) == 0.0


# ---------------------------------------------------------------- scatter_nd
def test_scatter_nd_oracle_matches_numpy_indexing(oracle):
    """Pins the offset arithmetic: with distinct rows, "assign" equals numpy's advanced-index assignment (the
    statement of the reference's own test, tests/python/test_scatter_nd.py:47: data[idx[:,0], idx[:,1]] = updates);
    "add" equals numpy.add.at, duplicates included; later rows win in "assign"; k == rank scatters scalars."""
    rng = np.random.default_rng(3)
    data = rng.standard_normal((7, 8, 9, 10)).astype(np.float32)
    rows = rng.permutation(56)[:20]
    idx = np.stack(np.unravel_index(rows, (7, 8)), axis=1)
    upd = rng.standard_normal((20, 9, 10)).astype(np.float32)
    expect = data.copy()
    expect[idx[:, 0], idx[:, 1]] = upd
    assert np.array_equal(oracle.scatter_nd(data, idx, upd), expect)
    # a wrong stride or a transposed index would move a slice: every other element must be untouched
    untouched = np.ones((7, 8), bool)
    untouched[idx[:, 0], idx[:, 1]] = False
    assert np.array_equal(oracle.scatter_nd(data, idx, upd)[untouched], data[untouched])

    idx_dup = rng.integers(0, 7, size=(50, 1))
    upd_dup = rng.integers(-3, 4, size=(50, 8, 9, 10)).astype(np.float32)
    expect = data.copy()
    np.add.at(expect, (idx_dup[:, 0],), upd_dup)
    np.testing.assert_allclose(oracle.scatter_nd(data, idx_dup, upd_dup, mode="add"), expect, rtol=0, atol=1e-4)

    two = np.array([[2], [2]])
    out = oracle.scatter_nd(np.zeros((4, 3), np.float32), two, np.array([[1, 1, 1], [2, 2, 2]], np.float32))
    assert np.array_equal(out[2], [2, 2, 2])

    full = np.array([[1, 2, 3], [0, 0, 0]])
    out = oracle.scatter_nd(np.zeros((2, 3, 4), np.float32), full, np.array([5, 6], np.float32))
    assert out[1, 2, 3] == 5 and out[0, 0, 0] == 6 and out.sum() == 11
    # out-of-range rows are skipped
    out = oracle.scatter_nd(np.zeros((2, 2), np.float32), np.array([[2], [-1], [1]]), np.ones((3, 2), np.float32))
    assert np.array_equal(out, [[0, 0], [1, 1]])
