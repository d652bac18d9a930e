"""Device unit tests of the tile primitives (tests/device/tile_tests.hip): every case of the
registry is run on the GPU and checked on the host against the identity or the CPU oracle.
Shapes and warp layouts are those of the reference's tests/cpp/cell/*.cu."""
import ctypes
import os

import numpy as np
import pytest
import torch  # before any HIP library is loaded: the process must share torch's HIP runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "tests", "device", "_build", "libtcu_tile_tests.so")

pytestmark = pytest.mark.gpu


def _load():
    handle = ctypes.CDLL(LIB)
    handle.tt_num_cases.restype = ctypes.c_int
    handle.tt_case_info.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(ctypes.c_char_p),
                                    ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                    ctypes.POINTER(ctypes.c_int)]
    handle.tt_run_case.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 5
    handle.tt_last_error.restype = ctypes.c_char_p
    return handle


def _cases():
    if not os.path.exists(LIB):
        return []
    handle = _load()
    out = []
    for i in range(handle.tt_num_cases()):
        kind, name = ctypes.c_char_p(), ctypes.c_char_p()
        dims = (ctypes.c_int * 8)()
        threads, lds = ctypes.c_int(), ctypes.c_int()
        assert handle.tt_case_info(i, ctypes.byref(kind), ctypes.byref(name), dims, ctypes.byref(threads),
                                   ctypes.byref(lds)) == 0
        out.append((i, kind.value.decode(), name.value.decode(), list(dims)))
    return out


CASES = _cases()


def test_registry_is_populated():
    assert os.path.exists(LIB), "device test library missing: run __graft_entry__.build()"
    kinds = {c[1] for c in CASES}
    assert kinds == {"g2s_roundtrip", "s2r_identity", "store_roundtrip", "g2r_roundtrip", "tile_gemm", "tile_b2b",
                     "row_ops", "col_ops", "elementwise"}


def _np_dtype(nbytes):
    return np.float16 if nbytes == 2 else np.float32


@pytest.mark.parametrize("case", CASES, ids=[f"{c[1]}-{c[2]}" for c in CASES])
def test_tile_case(case, device, oracle):
    import torch

    idx, kind, name, dims = case
    print(f"tile case {idx} {kind} {name}", flush=True)
    handle = _load()
    stream = torch.cuda.current_stream().cuda_stream

    def run(a, b, c, d):
        rc = handle.tt_run_case(idx, a.data_ptr() if a is not None else 0, b.data_ptr() if b is not None else 0,
                                c.data_ptr() if c is not None else 0, d.data_ptr() if d is not None else 0, stream)
        assert rc == 0, handle.tt_last_error()
        torch.cuda.synchronize()

    if kind in ("g2s_roundtrip", "s2r_identity", "store_roundtrip", "g2r_roundtrip"):
        rows, cols, _, nbytes = dims[:4]
        dt = _np_dtype(nbytes)
        # the reference's ramp (i % 2048), distinct per element for these sizes, exact in f16 up to 2048
        src = (np.arange(rows * cols) % 2048).astype(dt)
        a = torch.from_numpy(src).to(device)
        c = torch.full((rows * cols,), -1.0, dtype=a.dtype, device=device)
        run(a, None, c, None)
        assert np.array_equal(c.cpu().numpy(), src)
    elif kind == "tile_gemm":
        M, N, K = dims[:3]
        A = oracle.fill_uniform(M * K, 100 + idx).reshape(M, K)
        Bt = oracle.fill_uniform(N * K, 200 + idx).reshape(N, K)
        # dims[4] = 1: the kernel takes B stored row-major [K, N] (and transposes it on the way to registers)
        b_mem = np.ascontiguousarray(Bt.T) if dims[4] else Bt
        a, b = torch.from_numpy(A).to(device), torch.from_numpy(b_mem).to(device)
        c = torch.full((M, N), float("nan"), dtype=torch.float32, device=device)
        run(a, b, c, None)
        err = oracle.max_rel_err(c.cpu().numpy(), oracle.gemm(A, Bt))
        assert err <= 1e-3, f"max rel err {err}"
    elif kind == "tile_b2b":
        # D = f16(A B) V: B column-major (stored [N, K]) followed by V row-major [N, P] in one buffer
        M, N, K, P = dims[:4]
        A = oracle.fill_normal(M * K, 300 + idx, 0, 0.5).reshape(M, K)
        Bt = oracle.fill_normal(N * K, 400 + idx, 0, 0.5).reshape(N, K)
        V = oracle.fill_normal(N * P, 500 + idx, 0, 0.5).reshape(N, P)
        a = torch.from_numpy(A).to(device)
        b = torch.from_numpy(np.concatenate([Bt.reshape(-1), V.reshape(-1)])).to(device)
        c = torch.full((M, P), float("nan"), dtype=torch.float32, device=device)
        run(a, b, c, None)
        ref = oracle.b2b_gemm(A[None], Bt[None], np.ascontiguousarray(V.T)[None])[0]
        err = oracle.max_rel_err(c.cpu().numpy(), ref, eps=1.0)
        assert err <= 1e-3, f"max err relative to rms {err}"
    elif kind in ("row_ops", "col_ops"):
        rows, cols, op, nbytes = dims[:4]
        dt = _np_dtype(nbytes)
        rng = np.random.default_rng(42 + idx)  # the reference's softmax test seeds with 42, U[-5, 5]
        x = rng.uniform(-5, 5, (rows, cols)).astype(dt)
        row_major = kind == "row_ops"
        mem = x if row_major else np.ascontiguousarray(x.T)  # column-major storage
        a = torch.from_numpy(mem.copy()).to(device)
        nvec = rows if row_major else cols
        vec = torch.full((nvec,), float("nan"), dtype=a.dtype, device=device)
        tile = torch.full(mem.shape, float("nan"), dtype=a.dtype, device=device)
        run(a, None, vec, tile)
        v = vec.cpu().numpy().astype(np.float64)
        t = tile.cpu().numpy().astype(np.float64)
        if not row_major:
            t = t.T
        x64 = x.astype(np.float64)
        axis = 1 if row_major else 0
        tol = 1e-3 if dt == np.float32 else 0.15  # f16 sums of up to 64 values of magnitude 5
        names = (["sum", "max", "bcast_sum", "sub_max", "softmax", "add_sum", "mul_max", "div_sum"] if row_major
                 else ["sum", "max", "sub_max", "bcast_sum", "softmax", "mul_max"])
        opname = names[op]
        keep = dict(axis=axis, keepdims=True)
        if opname == "sum":
            assert np.allclose(v, x64.sum(axis), atol=tol)
            assert np.array_equal(t, x64)
        elif opname == "max":
            assert np.array_equal(v, x64.max(axis))
        elif opname == "bcast_sum":
            assert np.allclose(v, x64.sum(axis), atol=tol)
            assert np.allclose(t, np.broadcast_to(x64.sum(**keep), x64.shape), atol=tol)
        elif opname == "sub_max":
            assert np.allclose(t, x64 - x64.max(axis, keepdims=True), atol=1e-6 if dt == np.float32 else 1e-2)
        elif opname == "softmax":
            e = np.exp(x64 - x64.max(**keep))
            assert np.allclose(t, e / e.sum(**keep), atol=1e-3)  # the reference's tolerance
        elif opname == "add_sum":
            assert np.allclose(t, x64 + x64.sum(**keep), atol=tol)
        elif opname == "mul_max":
            assert np.allclose(t, x64 * x64.max(**keep), atol=1e-5 if dt == np.float32 else 0.05)
        elif opname == "div_sum":
            # sums of U[-5, 5] values can come close to 0: compare x = t * sum instead of dividing
            assert np.allclose(t * x64.sum(**keep), x64, atol=1e-3 if dt == np.float32 else 0.5)
    elif kind == "elementwise":
        rows, cols, op, nbytes, row_major = dims[:5]
        dt = _np_dtype(nbytes)
        rng = np.random.default_rng(77 + idx)
        opname = ["exp", "log", "relu", "add", "sub", "mul", "div", "max", "min", "convert_f16"][op]
        xa = rng.uniform(-4, 4, (rows, cols)).astype(dt)
        xb = rng.uniform(-4, 4, (rows, cols)).astype(dt)
        if opname == "log":
            xa = np.abs(xa) + dt(0.05)
        if opname == "div":
            xb = (np.sign(xb) * (np.abs(xb) + dt(0.25))).astype(dt)
        store = (lambda m: m) if row_major else (lambda m: np.ascontiguousarray(m.T))
        a, b = (torch.from_numpy(store(m).copy()).to(device) for m in (xa, xb))
        out_dt = torch.float16 if opname == "convert_f16" else a.dtype
        c = torch.full(store(xa).shape, float("nan"), dtype=out_dt, device=device)
        run(a, b, c, None)
        got = c.cpu().numpy()
        got = (got if row_major else got.T).astype(np.float64)
        a64, b64 = xa.astype(np.float64), xb.astype(np.float64)
        exact = {"relu": np.maximum(a64, 0), "max": np.maximum(a64, b64), "min": np.minimum(a64, b64)}
        if opname in exact:
            assert np.array_equal(got, exact[opname])
        elif opname == "convert_f16":
            assert np.array_equal(got, xa.astype(np.float16).astype(np.float64))  # round-to-nearest-even
        else:
            want = {"exp": lambda: np.exp(a64), "log": lambda: np.log(a64), "add": lambda: a64 + b64,
                    "sub": lambda: a64 - b64, "mul": lambda: a64 * b64, "div": lambda: a64 / b64}[opname]()
            # f32: the fast-math exp/log/div of the reference's functors (__expf, __logf) are good to ~1e-6 relative;
            # f16: one rounding of the result (2^-11) plus the rounding inside hexp/hlog
            rtol = 2e-6 if dt == np.float32 else 2e-3
            assert np.allclose(got, want, rtol=rtol, atol=rtol)
    else:
        raise AssertionError(kind)


def test_tile_printers_show_matrix_order(device, capfd):
    """RegTilePrinter / RegVecPrinter (the reference's include/util/print.hpp:67-175): a register tile spread over the
    64 lanes prints as the matrix it stands for - a 32 x 48 f16 tile of 2 x 3 BaseTiles, its row maxima, and a
    32 x 32 MFMA accumulator tile whose element (r, c) was set to r + c / 100 in its lane-local layout."""
    handle = _load()
    handle.tt_print_tiles.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    src = (np.arange(32 * 48) % 2048).astype(np.float16).reshape(32, 48)
    a = torch.from_numpy(src).to(device)
    capfd.readouterr()
    assert handle.tt_print_tiles(a.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0, handle.tt_last_error()
    torch.cuda.synchronize()
    out = capfd.readouterr().out
    blocks = [b for b in out.strip().split("\n\n") if b.strip()]
    assert len(blocks) == 3, out
    rows = [[float(x) for x in line.rstrip(", ").split(", ")] for line in blocks[0].strip().split("\n")]
    assert np.array_equal(np.array(rows), src.astype(np.float64))
    vec = [float(x) for x in blocks[1].strip().rstrip(",").split(", ")]
    assert np.array_equal(np.array(vec), src.max(axis=1).astype(np.float64))
    acc = np.array([[float(x) for x in line.rstrip(", ").split(", ")] for line in blocks[2].strip().split("\n")])
    want = np.arange(32)[:, None] + np.arange(32)[None, :] * 0.01
    assert acc.shape == (32, 32) and np.allclose(acc, want, atol=6e-4)  # printed with three decimals
