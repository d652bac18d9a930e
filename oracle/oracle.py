"""numpy/ctypes face of the CPU oracle (``oracle/oracle.c``).

TEST INFRASTRUCTURE ONLY.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this module; the shipped package
(``tiledcuda_amd``) never does.

Arrays of fp16 values travel as ``numpy.float16`` (viewed as ``uint16`` at the C
boundary).  Layout conventions are the reference's: A/Q/D row-major, B/K
column-major (stored transposed), see ``oracle.c`` for the file:line each function
follows.

The index helpers at the bottom restate the reference's layout and iterator
arithmetic in plain Python:
  * ``matrix_layout_offset``  include/types/layout.hpp:26-43
  * ``gtile_iterator_offset`` include/types/global_tile_iterator.hpp:59-106
  * ``warp_tile_origin``      include/cell/copy/warp.hpp:16-136 (which sub-block of a
                              tile a warp owns under each WarpReuse mode)
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle.c with gcc (idempotent)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "_build/liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _p(a: np.ndarray | None):
    if a is None:
        return ctypes.c_void_p(0)
    assert a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


def _i64(v):
    return ctypes.c_int64(int(v))


def num_threads() -> int:
    return int(lib().oracle_num_threads())


# ---------------------------------------------------------------- generators
def fill_uniform(n: int, seed: int, lo: float = -1.0, hi: float = 1.0) -> np.ndarray:
    out = np.empty(n, dtype=np.float16)
    lib().oracle_fill_uniform(_p(out), _i64(n), ctypes.c_uint64(seed), ctypes.c_float(lo), ctypes.c_float(hi))
    return out


def fill_normal(n: int, seed: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    out = np.empty(n, dtype=np.float16)
    lib().oracle_fill_normal(_p(out), _i64(n), ctypes.c_uint64(seed), ctypes.c_float(mean), ctypes.c_float(std))
    return out


def splitmix64_at(seed: int, i: np.ndarray) -> np.ndarray:
    """numpy restatement of the generator's counter hash (for pinning the C code)."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (i.astype(np.uint64) + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


# ---------------------------------------------------------------- kernels' math
def h2f(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float16)
    out = np.empty(a.shape, dtype=np.float32)
    lib().oracle_h2f(_p(a), _p(out), _i64(a.size))
    return out


def f2h(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.float16)
    lib().oracle_f2h(_p(a), _p(out), _i64(a.size))
    return out


def gemm(A: np.ndarray, Bt: np.ndarray, rows: tuple[int, int] | None = None, naive: bool = False) -> np.ndarray:
    """C[M,N] f32 = A[M,K] · Btᵀ, Bt = [N,K] (B column-major).  ``rows`` bounds the work."""
    M, K = A.shape
    N, K2 = Bt.shape
    assert K == K2 and A.dtype == np.float16 and Bt.dtype == np.float16
    C = np.zeros((M, N), dtype=np.float32)
    if naive:
        lib().oracle_gemm_f16_naive(_p(A), _p(Bt), _p(C), _i64(M), _i64(N), _i64(K))
    else:
        m0, m1 = rows if rows is not None else (0, M)
        lib().oracle_gemm_f16_rows(_p(A), _p(Bt), _p(C), _i64(M), _i64(N), _i64(K), _i64(m0), _i64(m1))
    return C


def b2b_gemm(A: np.ndarray, Bt: np.ndarray, Ct: np.ndarray) -> np.ndarray:
    """D[b,M,P] f32 = f16(A[b,M,K]·B)·C; Bt = [b,N,K], Ct = [b,P,N] (both column-major operands)."""
    if A.ndim == 2:
        return b2b_gemm(A[None], Bt[None], Ct[None])[0]
    b, M, K = A.shape
    _, N, _ = Bt.shape
    _, P, _ = Ct.shape
    assert Bt.shape == (b, N, K) and Ct.shape == (b, P, N)
    D = np.zeros((b, M, P), dtype=np.float32)
    lib().oracle_b2b_gemm_f16(_p(A), _p(Bt), _p(Ct), _p(D), _i64(M), _i64(N), _i64(K), _i64(P), _i64(b))
    return D


def attention(Q: np.ndarray, Kn: np.ndarray, V: np.ndarray, scale: float, v_col_major: bool = False,
              rows: tuple[int, int] | None = None) -> np.ndarray:
    """O[b,M,P] f32.  Q [b,M,K]; Kn [b,N,K]; V [b,N,P] (or [b,P,N] when ``v_col_major``)."""
    if Q.ndim == 2:
        return attention(Q[None], Kn[None], V[None], scale, v_col_major, rows)[0]
    b, M, K = Q.shape
    _, N, _ = Kn.shape
    P = V.shape[1] if v_col_major else V.shape[2]
    O = np.zeros((b, M, P), dtype=np.float32)
    m0, m1 = rows if rows is not None else (0, M)
    lib().oracle_attention_f16_rows(_p(Q), _p(Kn), _p(V), _p(O), _i64(b), _i64(M), _i64(N), _i64(K), _i64(P),
                                    ctypes.c_float(scale), ctypes.c_int(1 if v_col_major else 0), _i64(m0), _i64(m1))
    return O


def attention_blocked_f32(Q: np.ndarray, Kmat: np.ndarray, V: np.ndarray, tn: int, scale: float = 1.0) -> np.ndarray:
    """Blockwise recurrence of the reference's Python test (Q [M,K], Kmat [K,N], V [N,P], all f32)."""
    M, K = Q.shape
    _, N = Kmat.shape
    P = V.shape[1]
    assert N % tn == 0
    O = np.zeros((M, P), dtype=np.float32)
    lib().oracle_attention_blocked_f32(_p(np.ascontiguousarray(Q, np.float32)), _p(np.ascontiguousarray(Kmat, np.float32)),
                                       _p(np.ascontiguousarray(V, np.float32)), _p(O), _i64(M), _i64(N), _i64(K),
                                       _i64(P), _i64(tn), ctypes.c_float(scale))
    return O


def lstm(x: np.ndarray, W: np.ndarray, bias: np.ndarray, h0: np.ndarray | None = None,
         c0: np.ndarray | None = None, rows: tuple[int, int] | None = None):
    """x [T,B,I] f16, W [4H,I+H] f16, bias [4H] f16 → (h_all [T,B,H] f32, c_T [B,H] f32)."""
    T, B, I = x.shape
    H = W.shape[0] // 4
    assert W.shape == (4 * H, I + H) and bias.shape == (4 * H,)
    h_all = np.zeros((T, B, H), dtype=np.float32)
    c_out = np.zeros((B, H), dtype=np.float32)
    b0, b1 = rows if rows is not None else (0, B)
    lib().oracle_lstm_f16_rows(_p(x), _p(W), _p(bias), _p(h0), _p(c0), _p(h_all), _p(c_out), _i64(T), _i64(B),
                               _i64(I), _i64(H), _i64(b0), _i64(b1))
    return h_all, c_out


def scatter_nd(data: np.ndarray, indices: np.ndarray, updates: np.ndarray, mode: str = "assign") -> np.ndarray:
    """data[indices[i, 0], ..., indices[i, k-1], ...] (= | +=) updates[i] over the index rows in order; returns a copy.
    Offset arithmetic as the reference computes it (src/kernels/scatter_nd.cu:37-46: out_index = sum_c idx[c] *
    strides[c], slice of prod(data.shape[k:]) elements, strides from :66-70); "assign" is the semantics its test
    checks (tests/python/test_scatter_nd.py:47-56), "add" the accumulation its kernel body performs (:48-51).
    A plain loop over rows on the flattened array: later rows win in "assign" mode. Rows with an index outside the
    data are skipped."""
    out = np.array(data, copy=True)
    flat = out.reshape(-1)
    k = indices.shape[-1]
    rank = data.ndim
    strides = [1] * rank
    for d in range(rank - 2, -1, -1):
        strides[d] = strides[d + 1] * data.shape[d + 1]
    slice_size = int(np.prod(data.shape[k:], dtype=np.int64)) if k < rank else 1
    idx = np.asarray(indices, dtype=np.int64).reshape(-1, k)
    upd = np.asarray(updates).reshape(idx.shape[0], slice_size)
    for i in range(idx.shape[0]):
        if any(idx[i, c] < 0 or idx[i, c] >= data.shape[c] for c in range(k)):
            continue
        base = sum(int(idx[i, c]) * strides[c] for c in range(k))
        if mode == "assign":
            flat[base:base + slice_size] = upd[i]
        elif mode == "add":
            flat[base:base + slice_size] = (flat[base:base + slice_size].astype(np.float32) +
                                            upd[i].astype(np.float32)).astype(flat.dtype)
        else:
            raise ValueError(mode)
    return out


# ---------------------------------------------------------------- error metrics
def max_rel_err(x: np.ndarray, ref: np.ndarray, eps: float = 1e-2) -> float:
    """max |x-ref| / max(|ref|, eps·rms(ref)): relative error with a floor, so outputs that
    happen to land next to zero (cancellation in a K-long dot product) do not blow the ratio up."""
    x = np.asarray(x, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    floor = max(eps * rms, 1e-30)
    return float(np.max(np.abs(x - ref) / np.maximum(np.abs(ref), floor))) if ref.size else 0.0


def max_abs_err(x: np.ndarray, ref: np.ndarray) -> float:
    return float(np.max(np.abs(np.asarray(x, np.float64) - np.asarray(ref, np.float64)))) if ref.size else 0.0


# ---------------------------------------------------------------- index semantics
def matrix_layout_offset(i: int, j: int, row_stride: int, col_stride: int) -> int:
    return i * row_stride + j * col_stride


def gtile_iterator_offset(x: int, y: int, rows: int, cols: int, chunk_rows: int, chunk_cols: int,
                          row_major: bool, stride: int | None = None) -> int:
    """Element offset of sub-tile (x, y) of a [rows, cols] tile chunked by [chunk_rows, chunk_cols].
    Taken from logical coordinates (first element of the chunk)."""
    if row_major:
        rs = stride if stride is not None else cols
        return x * chunk_rows * rs + y * chunk_cols
    cs = stride if stride is not None else rows
    return x * chunk_rows + y * chunk_cols * cs


def warp_tile_origin(warp_row: int, warp_col: int, tile_rows: int, tile_cols: int, warps_r: int,
                     warps_c: int, mode: str) -> tuple[int, int, int, int]:
    """(row0, col0, nrows, ncols) of the sub-block of a tile owned by warp (warp_row, warp_col).
    mode ∈ {"cont", "row_reuse_cont", "col_reuse_cont"}."""
    if mode == "cont":
        nr, nc = tile_rows // warps_r, tile_cols // warps_c
        return warp_row * nr, warp_col * nc, nr, nc
    if mode == "row_reuse_cont":  # warps of one warp-row all load that row-block, full width
        nr = tile_rows // warps_r
        return warp_row * nr, 0, nr, tile_cols
    if mode == "col_reuse_cont":
        nc = tile_cols // warps_c
        return 0, warp_col * nc, tile_rows, nc
    raise NotImplementedError(mode)
