"""MI355X-native tile kernels behind the reference's Python surface.

Mirrors ``pytiledcuda/__init__.py`` of the reference (``flash_attention_fwd``,
``TiledFlashAttention``) and adds the other kernel entries (``gemm``, ``b2b_gemm``,
``lstm``, ``flash_attention``).  Everything runs through the C-ABI shared library
``lib/libtiledcuda_amd.so`` (declared in ``include/tcu_c_api.h``); there is no CPU or
PyTorch fallback: if the library is missing, importing any op raises.

PyTorch is used only for device memory and the current HIP stream.
"""
from __future__ import annotations

import ctypes
import math
import os

import torch

__all__ = [
    "TcuError", "library_path", "lib", "last_error", "gemm", "gemm_workspace_bytes", "b2b_gemm", "flash_attention_fwd",
    "flash_attention", "TiledFlashAttention", "lstm", "lstm_workspace_bytes", "lstm_persistent_workspace_bytes", "lstm_persistent_status", "scatter_nd", "GEMM_ALGOS", "ATTN_ALGOS", "LSTM_ALGOS", "B2B_ALGOS",
    "SCATTER_MODES",
]

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "lib", "libtiledcuda_amd.so")
_lib = None

TCU_OK = 0
TCU_ERR_INVALID_ARGUMENT = -1
TCU_ERR_UNSUPPORTED_SHAPE = -2
TCU_ERR_HIP = -3
TCU_ERR_NO_DEVICE = -4

TCU_DTYPE_F32 = 0
TCU_DTYPE_F16 = 1

GEMM_ALGOS = {"auto": 0, "global_reg": 1, "all_mem": 2, "pipelined": 3, "wave128": 4, "tile_pipelined": 5, "ragged": 6, "tile_wave128": 7, "wave128_ksplit": 8, "wave128_narrow": 9}

TCU_V_COL_MAJOR = 0
TCU_V_ROW_MAJOR = 1

ATTN_ALGOS = {"auto": 0, "tile_library": 1, "mfma32": 2, "mfma32_fused": 3, "wave64": 4, "tile_wave64": 5, "wave64_k32": 6}
LSTM_ALGOS = {"auto": 0, "tile_library": 1, "streaming": 2, "ragged": 3}
B2B_ALGOS = {"auto": 0, "tile_library": 1, "resident": 2, "rows": 3, "tile_resident": 4}
SCATTER_MODES = {"assign": 0, "add": 1}

# every exported symbol with its ctypes signature (also what the symbol test checks)
_SIGNATURES = {
    "tcu_version": (ctypes.c_int, []),
    "tcu_last_error": (ctypes.c_char_p, []),
    "tcu_device_count": (ctypes.c_int, []),
    "tcu_gemm_f16": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_int] * 5 + [ctypes.c_void_p]),
    "tcu_gemm_workspace_bytes": (ctypes.c_ulonglong, [ctypes.c_int] * 3),
    "tcu_gemm_f16_ws": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.c_ulonglong,
                                                                                  ctypes.c_void_p]),
    "tcu_b2b_gemm_f16": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_int] * 6 + [ctypes.c_void_p]),
    "tcu_b2b_gemm_f16_algo": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_int] * 7 + [ctypes.c_void_p]),
    "tcu_flash_attn_fwd_f16": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_int] * 5 + [ctypes.c_float, ctypes.c_int,
                                                                                           ctypes.c_void_p]),
    "tcu_flash_attn_fwd_f16_algo": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_int] * 5 + [ctypes.c_float, ctypes.c_int,
                                                                                                ctypes.c_int, ctypes.c_void_p]),
    "tcu_lstm_f16": (ctypes.c_int, [ctypes.c_void_p] * 7 + [ctypes.c_int] * 4 + [ctypes.c_void_p]),
    "tcu_lstm_f16_algo": (ctypes.c_int, [ctypes.c_void_p] * 7 + [ctypes.c_int] * 5 + [ctypes.c_void_p]),
    "tcu_lstm_workspace_bytes": (ctypes.c_ulonglong, [ctypes.c_int] * 4),
    "tcu_lstm_f16_ws": (ctypes.c_int, [ctypes.c_void_p] * 7 + [ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.c_ulonglong,
                                                                                     ctypes.c_void_p]),
    "tcu_lstm_persistent_workspace_bytes": (ctypes.c_ulonglong, [ctypes.c_int] * 4),
    "tcu_lstm_f16_persistent": (ctypes.c_int, [ctypes.c_void_p] * 7 + [ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.c_ulonglong,
                                                                                          ctypes.c_void_p]),
    "tcu_lstm_persistent_status": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p]),
    "tcu_lstm_noalloc_max_bytes": (ctypes.c_ulonglong, []),
    "tcu_lstm_f16_noalloc": (ctypes.c_int, [ctypes.c_void_p] * 7 + [ctypes.c_int] * 4 + [ctypes.c_void_p]),
    "tcu_scatter_nd": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.POINTER(ctypes.c_longlong), ctypes.c_int,
                                                             ctypes.c_longlong, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                             ctypes.c_void_p, ctypes.c_void_p]),
}


class TcuError(RuntimeError):
    """A C-ABI call returned a negative status (the reference op raises RuntimeError too)."""

    def __init__(self, status: int, message: str):
        super().__init__(f"tiledcuda_amd status {status}: {message}")
        self.status = status


def library_path() -> str:
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    """Load the HIP extension (once). Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                f"{_LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc --offload-arch=gfx950). There is no fallback path.")
        handle = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def last_error() -> str:
    return lib().tcu_last_error().decode()


def _check(status: int) -> None:
    if status != TCU_OK:
        raise TcuError(status, last_error())


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev_ptr(t: torch.Tensor | None, dtype: torch.dtype, name: str) -> int:
    if t is None:
        return 0
    if not t.is_cuda:
        raise ValueError(f"{name} must live in device memory")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t.data_ptr()


def _out_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return TCU_DTYPE_F32
    if dtype == torch.float16:
        return TCU_DTYPE_F16
    raise ValueError("out dtype must be torch.float32 or torch.float16")


# ------------------------------------------------------------------------------ GEMM
def gemm(a: torch.Tensor, b_t: torch.Tensor, out: torch.Tensor | None = None,
         out_dtype: torch.dtype = torch.float16, algo: str = "auto",
         workspace: torch.Tensor | None | bool = None) -> torch.Tensor:
    """C[M, N] = A[M, K] · B with B column-major, i.e. ``b_t`` is the [N, K] array (``a @ b_t.T``).

    Mirrors the reference's GEMM examples (A row-major, B column-major, f32 accumulate). With ``algo="auto"`` a
    product with few output tiles and a long K is split over K (``tcu_gemm_f16_ws``) through ``workspace`` (a contiguous
    device tensor of at least ``gemm_workspace_bytes(M, N, K)`` bytes), or, when none is given, through one taken from
    torch's caching allocator for the call; ``workspace=False`` never splits (use it, or a workspace of your own, when
    the call is being captured into a HIP graph: an allocation has no place in a captured stream).
    """
    M, K = a.shape
    N, K2 = b_t.shape
    if K != K2:
        raise ValueError("mismatched K dimension")
    if out is None:
        out = torch.empty(M, N, dtype=out_dtype, device=a.device)
    elif tuple(out.shape) != (M, N):
        raise ValueError("out has the wrong shape")
    if workspace is None and algo == "auto" and a.is_cuda:
        need = gemm_workspace_bytes(M, N, K)
        if need > 0:
            workspace = torch.empty(need, dtype=torch.uint8, device=a.device)
    if workspace is False:
        workspace = None
    if workspace is not None:
        if algo != "auto":
            raise ValueError("a workspace goes with algo='auto'")
        if not workspace.is_cuda or not workspace.is_contiguous():
            raise ValueError("workspace must be a contiguous device tensor")
        _check(lib().tcu_gemm_f16_ws(_dev_ptr(a, torch.float16, "a"), _dev_ptr(b_t, torch.float16, "b_t"),
                                     _dev_ptr(out, out.dtype, "out"), M, N, K, _out_code(out.dtype), workspace.data_ptr(),
                                     workspace.numel() * workspace.element_size(), _stream()))
        return out
    _check(lib().tcu_gemm_f16(_dev_ptr(a, torch.float16, "a"), _dev_ptr(b_t, torch.float16, "b_t"),
                              _dev_ptr(out, out.dtype, "out"), M, N, K, _out_code(out.dtype), GEMM_ALGOS[algo],
                              _stream()))
    return out


def gemm_workspace_bytes(M: int, N: int, K: int) -> int:
    """Device bytes ``gemm(..., workspace=...)`` uses for a split over K; 0 when the product is not split."""
    return int(lib().tcu_gemm_workspace_bytes(M, N, K))


# ------------------------------------------------------------------------------ b2b GEMM
def b2b_gemm(a: torch.Tensor, b_t: torch.Tensor, c_t: torch.Tensor, out: torch.Tensor | None = None,
             out_dtype: torch.dtype = torch.float16, algo: str = "auto") -> torch.Tensor:
    """D = (A · B) · C per batch item; ``b_t`` [.., N, K] and ``c_t`` [.., P, N] are the
    column-major operands of the reference's fused two-GEMM example stored as arrays."""
    batched = a.dim() == 3
    if any(t.dim() != a.dim() for t in (b_t, c_t)) or a.dim() not in (2, 3):
        raise ValueError("operands must all be 2-D or all be 3-D (batched)")
    a3, b3, c3 = (t if batched else t.unsqueeze(0) for t in (a, b_t, c_t))
    batch, M, K = a3.shape
    _, N, _ = b3.shape
    _, P, _ = c3.shape
    if tuple(b3.shape) != (batch, N, K) or tuple(c3.shape) != (batch, P, N):
        raise ValueError("operand shapes do not chain: A [b,M,K], b_t [b,N,K], c_t [b,P,N]")
    if out is None:
        out = torch.empty(batch, M, P, dtype=out_dtype, device=a.device)
    elif tuple(out.shape) != (batch, M, P) and not (not batched and tuple(out.shape) == (M, P)):
        raise ValueError(f"out must be [{batch}, {M}, {P}], got {tuple(out.shape)}")
    _check(lib().tcu_b2b_gemm_f16_algo(_dev_ptr(a3, torch.float16, "a"), _dev_ptr(b3, torch.float16, "b_t"),
                                       _dev_ptr(c3, torch.float16, "c_t"), _dev_ptr(out, out.dtype, "out"), M, N, K, P,
                                       batch, _out_code(out.dtype), B2B_ALGOS[algo], _stream()))
    return out if batched else out.view(M, P) if out.dim() == 3 else out


# ------------------------------------------------------------------------------ attention
def flash_attention_fwd(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, O: torch.Tensor, m: int, n: int, k: int,
                        p: int, scale: float = 1.0, batch: int = 1, algo: str = "auto") -> None:
    """Same call shape as the reference's ``pytiledcuda.flash_attention_fwd`` (flattened fp16
    device tensors; K as [n, k], V as [p, n]; O written in place; ``scale`` defaults to the
    reference's 1; ``algo`` picks a kernel, as in ``flash_attention``).  Unsupported shapes raise
    ``RuntimeError`` like the reference op."""
    if min(m, n, k, p, batch) <= 0:
        raise ValueError("m, n, k, p and batch must be positive")
    for name, t, want in (("Q", Q, batch * m * k), ("K", K, batch * n * k), ("V", V, batch * p * n),
                          ("O", O, batch * m * p)):
        if t.numel() != want:
            raise ValueError(f"{name} must hold batch*rows*cols = {want} elements, got {t.numel()}")
    _check(lib().tcu_flash_attn_fwd_f16_algo(_dev_ptr(Q, torch.float16, "Q"), _dev_ptr(K, torch.float16, "K"),
                                             _dev_ptr(V, torch.float16, "V"), _dev_ptr(O, torch.float16, "O"), batch, m,
                                             n, k, p, float(scale), TCU_V_COL_MAJOR, ATTN_ALGOS[algo], _stream()))


def flash_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float | None = None,
                    out: torch.Tensor | None = None, algo: str = "auto") -> torch.Tensor:
    """softmax(scale · q kᵀ) v for [..., S, D] tensors in the usual layout (V row-major [S, D]).
    ``scale`` defaults to 1/sqrt(D)."""
    if q.dim() < 2 or k.dim() < 2 or v.dim() < 2:
        raise ValueError("q, k and v must be [..., S, D]")
    *lead, M, D = q.shape
    N = k.shape[-2]
    P = v.shape[-1]
    # the kernel strides every operand by the same leading index: broadcast (MQA/GQA-style) operands would be read
    # past their end
    if tuple(k.shape) != (*lead, N, D):
        raise ValueError(f"k must be {(*lead, N, D)} (same leading dimensions and head size as q), got {tuple(k.shape)}")
    if tuple(v.shape) != (*lead, N, P):
        raise ValueError(f"v must be {(*lead, N, P)} (same leading dimensions and key count as k), got {tuple(v.shape)}")
    batch = int(math.prod(lead)) if lead else 1
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    if out is None:
        out = torch.empty(*lead, M, P, dtype=torch.float16, device=q.device)
    elif tuple(out.shape) != (*lead, M, P):
        raise ValueError(f"out must be {(*lead, M, P)}, got {tuple(out.shape)}")
    _check(lib().tcu_flash_attn_fwd_f16_algo(_dev_ptr(q, torch.float16, "q"), _dev_ptr(k, torch.float16, "k"),
                                             _dev_ptr(v, torch.float16, "v"), _dev_ptr(out, torch.float16, "out"),
                                             batch, M, N, D, P, float(scale), TCU_V_ROW_MAJOR, ATTN_ALGOS[algo],
                                             _stream()))
    return out


class TiledFlashAttention:
    """Mirror of the reference's ``pytiledcuda.TiledFlashAttention``: ``query`` [m, k],
    ``key`` [k, n], ``value`` [n, p]; ``forward()`` returns O [m, p] in fp16 (scale 1)."""

    def __init__(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, scale: float = 1.0):
        self.m, self.k = query.size(-2), query.size(-1)
        self.n, self.p = value.size(-2), value.size(-1)
        self.scale = scale

        self.query = query.half().flatten().contiguous()
        # the kernel consumes K and V column-major: store their transposes
        self.key = key.half().t().contiguous().flatten()
        self.value = value.half().t().contiguous().flatten()

        self.output = torch.empty(self.m, self.p, dtype=torch.half, device=query.device).flatten()

    def forward(self) -> torch.Tensor:
        flash_attention_fwd(self.query, self.key, self.value, self.output, self.m, self.n, self.k, self.p,
                            scale=self.scale)
        return self.output.view(self.m, self.p)


# ------------------------------------------------------------------------------ LSTM
def lstm(x: torch.Tensor, W: torch.Tensor, bias: torch.Tensor, h0: torch.Tensor | None = None,
         c0: torch.Tensor | None = None, algo: str = "auto", workspace: torch.Tensor | None | bool = None,
         out: tuple[torch.Tensor, torch.Tensor] | None = None, check: bool = True
         ) -> tuple[torch.Tensor, torch.Tensor]:
    """Fused LSTM layer. x [T, B, I] f16, W [4H, I+H] f16 (gate rows i,f,g,o), bias [4H] f16,
    h0 [B, H] f16 / c0 [B, H] f32 (None = zeros). Returns (h_all [T, B, H] f16, c_T [B, H] f32).

    ``algo="hoisted"`` computes the input half of the gates for all steps in one GEMM first (``tcu_lstm_f16_ws``); it
    needs ``lstm_workspace_bytes(T, B, I, H)`` bytes of device memory, taken from ``workspace`` (any dtype) if given,
    else allocated here. ``algo="auto"`` takes that path where it applies and pays (I >= 512, T >= 4) unless
    ``workspace=False`` (use that, or a workspace of your own, under HIP graph capture), else one fused kernel per step. ``out`` = (h_all, c_T) tensors to write into instead of allocating them.

    ``algo="persistent"`` runs the whole time loop in one weight-stationary launch after the same GEMM
    (``tcu_lstm_f16_persistent``: H in {256, 512, 768, 1024}, B <= 256 in multiples of 32; ``lstm_persistent_workspace_bytes``). Its
    workgroups wait for each other with a time limit; with ``check=True`` (the default) the stream is synchronised and
    a RuntimeError raised if a wait expired, ``check=False`` leaves that to a later ``lstm_persistent_status(workspace)``."""
    if x.dim() != 3 or W.dim() != 2:
        raise ValueError("x must be [T, B, I] and W [4H, I+H]")
    T, B, I = x.shape
    H = W.shape[0] // 4
    if tuple(W.shape) != (4 * H, I + H) or tuple(bias.shape) != (4 * H,):
        raise ValueError("W must be [4H, I+H] and bias [4H]")
    if h0 is not None and tuple(h0.shape) != (B, H):
        raise ValueError(f"h0 must be [{B}, {H}], got {tuple(h0.shape)}")
    if c0 is not None and tuple(c0.shape) != (B, H):
        raise ValueError(f"c0 must be [{B}, {H}], got {tuple(c0.shape)}")
    if out is None:
        h_all = torch.empty(T, B, H, dtype=torch.float16, device=x.device)
        c_out = torch.empty(B, H, dtype=torch.float32, device=x.device)
    else:
        h_all, c_out = out
        if tuple(h_all.shape) != (T, B, H) or tuple(c_out.shape) != (B, H):
            raise ValueError(f"out must be (h_all [{T}, {B}, {H}], c_T [{B}, {H}])")
    if algo == "persistent":
        need = lstm_persistent_workspace_bytes(T, B, I, H)
        if workspace is None:
            workspace = torch.empty(max(need, 4096), dtype=torch.uint8, device=x.device)
        if not workspace.is_cuda or not workspace.is_contiguous():
            raise ValueError("workspace must be a contiguous device tensor")
        _check(lib().tcu_lstm_f16_persistent(_dev_ptr(x, torch.float16, "x"), _dev_ptr(W, torch.float16, "W"),
                                             _dev_ptr(bias, torch.float16, "bias"), _dev_ptr(h0, torch.float16, "h0"),
                                             _dev_ptr(c0, torch.float32, "c0"), _dev_ptr(h_all, torch.float16, "h_all"),
                                             _dev_ptr(c_out, torch.float32, "c_out"), T, B, I, H, workspace.data_ptr(),
                                             workspace.numel() * workspace.element_size(), _stream()))
        if check:
            lstm_persistent_status(workspace)
        return h_all, c_out
    if algo == "auto" and workspace is not False and x.is_cuda and I >= 512 and T >= 4 and lstm_workspace_bytes(T, B, I, H) > 0:
        algo = "hoisted"  # a long input size: its half of the gates is cheaper as one GEMM over all steps
    if algo == "hoisted":
        need = lstm_workspace_bytes(T, B, I, H)
        if workspace is None or workspace is False:
            workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=x.device)
        if not workspace.is_cuda or not workspace.is_contiguous():
            raise ValueError("workspace must be a contiguous device tensor")
        _check(lib().tcu_lstm_f16_ws(_dev_ptr(x, torch.float16, "x"), _dev_ptr(W, torch.float16, "W"),
                                     _dev_ptr(bias, torch.float16, "bias"), _dev_ptr(h0, torch.float16, "h0"),
                                     _dev_ptr(c0, torch.float32, "c0"), _dev_ptr(h_all, torch.float16, "h_all"),
                                     _dev_ptr(c_out, torch.float32, "c_out"), T, B, I, H, workspace.data_ptr(),
                                     workspace.numel() * workspace.element_size(), _stream()))
        return h_all, c_out
    _check(lib().tcu_lstm_f16_algo(_dev_ptr(x, torch.float16, "x"), _dev_ptr(W, torch.float16, "W"),
                                   _dev_ptr(bias, torch.float16, "bias"), _dev_ptr(h0, torch.float16, "h0"),
                                   _dev_ptr(c0, torch.float32, "c0"), _dev_ptr(h_all, torch.float16, "h_all"),
                                   _dev_ptr(c_out, torch.float32, "c_out"), T, B, I, H, LSTM_ALGOS[algo], _stream()))
    return h_all, c_out


def lstm_workspace_bytes(T: int, B: int, I: int, H: int) -> int:
    """Device bytes ``lstm(..., algo="hoisted")`` needs; 0 if that path is not instantiated for the shape."""
    return int(lib().tcu_lstm_workspace_bytes(T, B, I, H))


def lstm_persistent_workspace_bytes(T: int, B: int, I: int, H: int) -> int:
    """Device bytes ``lstm(..., algo="persistent")`` needs; 0 if that path does not take the shape."""
    return int(lib().tcu_lstm_persistent_workspace_bytes(T, B, I, H))


def lstm_persistent_status(workspace: torch.Tensor) -> None:
    """Synchronise the current stream and raise RuntimeError if the last ``lstm(..., algo="persistent")`` call that used
    ``workspace`` gave up a wait (its outputs are then invalid)."""
    _check(lib().tcu_lstm_persistent_status(workspace.data_ptr(), _stream()))


# ------------------------------------------------------------------------------ scatter_nd
def scatter_nd(scatter_data: torch.Tensor, scatter_indices: torch.Tensor, scatter_updates: torch.Tensor,
               mode: str = "assign", skipped_rows: torch.Tensor | None = None) -> None:
    """``data[indices[i, 0], ..., indices[i, k-1]] (= | +=) updates[i]`` in place, argument order of the
    reference's ``pytiledcuda.scatter_nd(scatter_data, scatter_indices, scatter_updates)``.

    ``scatter_data`` [d0, ..., d_{r-1}] f32 or f16, ``scatter_indices`` int64 [..., k], ``scatter_updates``
    [..., d_k, ..., d_{r-1}]. (The reference wrapper is handed flattened tensors, which loses the shapes its op
    reads them from; pass the shaped tensors here.) Rows with an out-of-range index are skipped; if
    ``skipped_rows`` (uint32/int32 device tensor of one element, zeroed by the caller) is given it counts them."""
    k = scatter_indices.shape[-1]
    rank = scatter_data.dim()
    n = scatter_indices.numel() // k if k else 0
    slice_shape = tuple(scatter_data.shape[k:])
    if k > rank or rank > 8:
        raise ValueError("scatter_nd needs k <= rank(data) <= 8")
    if scatter_updates.numel() != n * int(math.prod(slice_shape)):
        raise ValueError("updates must have one slice data.shape[k:] per index row")
    if scatter_data.dtype not in (torch.float32, torch.float16) or scatter_updates.dtype != scatter_data.dtype:
        raise ValueError("data and updates must both be float32 or both float16")
    dims = (ctypes.c_longlong * rank)(*scatter_data.shape)
    skipped = 0
    if skipped_rows is not None:
        if not skipped_rows.is_cuda or skipped_rows.element_size() != 4 or skipped_rows.numel() != 1:
            raise ValueError("skipped_rows must be a one-element 32-bit device tensor")
        skipped = skipped_rows.data_ptr()
    _check(lib().tcu_scatter_nd(_dev_ptr(scatter_data, scatter_data.dtype, "data"),
                                _dev_ptr(scatter_updates, scatter_data.dtype, "updates"),
                                _dev_ptr(scatter_indices, torch.int64, "indices"), dims, rank, n, k,
                                _out_code(scatter_data.dtype), SCATTER_MODES[mode], skipped, _stream()))
