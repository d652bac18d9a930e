"""Run-time compilation of GEMM instantiations and a tile-shape sweep.

Mirrors the reference's examples/python/gemm: ``Compile`` (compile.py:22-137) writes a translation unit that
fixes the problem and tile shape as template arguments, compiles it to a shared library exporting
``extern "C" int kernel_entry(__half*, __half*, float*)`` (entry.py:56-67) and calls it through ctypes;
``gemm_func`` (gemm.py:13-42) compiles on first use and launches; ``sweep`` is the tile-shape loop of main.py:90-112
with the timings returned instead of printed. The compiler is hipcc for gfx950, the kernels are this
repository's headers (``include/kernels/gemm.hpp`` for the tile-library kernel the reference example builds and, as
``kernel="tile_wave128"``, for the one-wavefront-per-SIMD kernel composed from tile-library functors at any M, N in
multiples of 256 and K in multiples of 64; ``include/kernels/gemm_pipelined.hpp`` for the hand-indexed one). A is [M, K] row-major, B is [N, K] (column-major
operand), C is [M, N] fp32.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import tempfile

import torch

__all__ = ["Compile", "gemm_func", "sweep"]

_HERE = os.path.dirname(os.path.abspath(__file__))
INCLUDE_DIR = os.path.join(os.path.dirname(_HERE), "include")

_TILE_LIBRARY_SOURCE = """#include "kernels/gemm.hpp"
using namespace tiledcuda;
using namespace tiledcuda::kernels;

using Config = GemmTraits<__half, float, GemmShape<{M}, {N}, {K}>, {TM}, {TN}, tl::RowMajor<{wr}, {wc}>, {chunk}>;
static_assert({M} % {TM} == 0 && {N} % {TN} == 0 && {K} % {chunk} == 0, "the tile must divide the problem");

static int launch(const __half* a, const __half* b, float* c, hipStream_t stream) {{
    auto kernel = &simple_gemm<__half, float, {M}, {N}, {K}, {TM}, {TN}, Config::IteratorA, Config::RegA, Config::ALoader,
                               Config::IteratorB, Config::RegB, Config::BLoader, Config::GlobalC, Config::RegC,
                               Config::CStorer>;
    hipLaunchKernelGGL(kernel, dim3({M} / {TM}, {N} / {TN}, 1), dim3(Config::kThreads, 1, 1), 0, stream, a, b, c);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}}
"""

_PIPELINED_SOURCE = """#include "kernels/gemm_pipelined.hpp"
using namespace tiledcuda;
using namespace tiledcuda::kernels;

using Config = PipelinedGemmTraits<{TM}, {TN}, 64, {wr}, {wc}, 2>;
static_assert({M} % {TM} == 0 && {N} % {TN} == 0 && {K} % 64 == 0, "the tile must divide the problem");

static int launch(const __half* a, const __half* b, float* c, hipStream_t stream) {{
    auto kernel = &gemm_pipelined<Config, float>;
    constexpr int lds = Config::template lds_bytes<float>();
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {{
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -3;
        raised = true;
    }}
    hipLaunchKernelGGL(kernel, dim3(({M} / {TM}) * ({N} / {TN})), dim3(Config::kThreads), lds, stream, a, b, c, {M}, {N}, {K}, {N});
    return hipGetLastError() == hipSuccess ? 0 : -3;
}}
"""

_TILE_WAVE128_SOURCE = """#include "kernels/gemm.hpp"
using namespace tiledcuda;
using namespace tiledcuda::kernels;

// the one-wavefront-per-SIMD kernel composed from tile-library functors: its tile and wavefront layout are fixed
static_assert({TM} == 256 && {TN} == 256 && {chunk} == 64 && {wr} == 2 && {wc} == 2,
              "tile_wave128 is a 256 x 256 x 64 tile on 2 x 2 wavefronts");
using Config = ScheduledGemmTileTraits<__half, float, GemmShape<{M}, {N}, {K}>>;

static int launch(const __half* a, const __half* b, float* c, hipStream_t stream) {{
    auto kernel = &gemm_tile_w128<__half, float, Config>;
    static bool raised = false;
    if (!raised) {{
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, Config::kShmBytes) != hipSuccess) return -3;
        raised = true;
    }}
    hipLaunchKernelGGL(kernel, dim3(({M} / 256) * ({N} / 256)), dim3(Config::kThreads), Config::kShmBytes, stream, a, b, c);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}}
"""

_ENTRY = """
extern "C" int kernel_entry(__half* parameter1, __half* parameter2, float* parameter3) {
    return launch(parameter1, parameter2, parameter3, nullptr);
}

extern "C" int kernel_entry_stream(__half* parameter1, __half* parameter2, float* parameter3, void* stream) {
    return launch(parameter1, parameter2, parameter3, static_cast<hipStream_t>(stream));
}
"""


_SOURCES = {"tile_library": _TILE_LIBRARY_SOURCE, "pipelined": _PIPELINED_SOURCE, "tile_wave128": _TILE_WAVE128_SOURCE}


def _default_cache_dir() -> str:
    """A directory only this user can write (mode 0700): the libraries in it are loaded into the process, so a
    world-writable location would let another user of the host plant one."""
    base = os.environ.get("XDG_CACHE_HOME") or os.path.join(os.path.expanduser("~"), ".cache")
    path = os.path.join(base, "tiledcuda_amd", "jit")
    try:
        os.makedirs(path, mode=0o700, exist_ok=True)
        if os.stat(path).st_uid == os.getuid() and os.access(path, os.W_OK):
            return path
    except OSError:
        pass
    return tempfile.mkdtemp(prefix="tiledcuda_amd_jit_")  # created 0700, unique to this process


def _headers_digest() -> str:
    """Digest of the contents of every header under include/ (the generated sources include them)."""
    h = hashlib.sha256()
    for root, _dirs, files in sorted(os.walk(INCLUDE_DIR)):
        for name in sorted(files):
            if name.endswith((".hpp", ".h")):
                with open(os.path.join(root, name), "rb") as f:
                    h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def _find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"),
                 os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("Cannot find hipcc (set HIPCC or ROCM_PATH)")


class Compile:
    """Same surface as the reference's ``Compile``: ``compile(...)`` returns the path of the shared library
    (cached by file name in ``tmp_dir``), ``apply(lib_path, [A, B, C], device)`` calls its ``kernel_entry``."""

    def __init__(self, file_prefix: str = "gemm", tmp_dir: str | None = None, kernel: str = "tile_library"):
        if kernel not in _SOURCES:
            raise ValueError("kernel must be one of " + ", ".join(repr(k) for k in _SOURCES))
        self.tmp_dir = tmp_dir or _default_cache_dir()
        self.file_prefix = file_prefix
        self.kernel = kernel
        os.makedirs(self.tmp_dir, mode=0o700, exist_ok=True)
        self.hipcc_path = _find_hipcc()
        self._libs: dict[str, ctypes.CDLL] = {}

    def _create_entry_code(self, M, N, K, TM, TN, kChunkK, warp_per_row, warp_per_col) -> str:
        template = _SOURCES[self.kernel]
        return template.format(M=M, N=N, K=K, TM=TM, TN=TN, chunk=kChunkK, wr=warp_per_row, wc=warp_per_col) + _ENTRY

    def compile(self, M: int, N: int, K: int, TM: int, TN: int, kChunkK: int, warp_per_row: int, warp_per_col: int,
                timeout: float | None = None) -> str | None:
        """Returns the library path, None on a compiler timeout; raises RuntimeError (with the compiler's
        output) if the instantiation does not compile, e.g. a tile that does not divide over the wavefronts."""
        source = self._create_entry_code(M, N, K, TM, TN, kChunkK, warp_per_row, warp_per_col)
        # the name carries a digest of the generated source and of every header it can include, so that an edited
        # kernel header never resolves to a library built from the old one
        digest = hashlib.sha256((source + _headers_digest()).encode()).hexdigest()[:16]
        file_name = (f"{self.file_prefix}_{self.kernel}_{M}_{N}_{K}_{TM}_{TN}_{kChunkK}_{warp_per_row}_{warp_per_col}"
                     f"_{digest}")
        lib_path = os.path.join(self.tmp_dir, f"{file_name}.so")
        if os.path.exists(lib_path):
            return lib_path
        source_path = os.path.join(self.tmp_dir, f"{file_name}.hip")
        with open(source_path, "w") as f:
            f.write(source)
        tmp_out = lib_path + f".{os.getpid()}.tmp"
        command = [self.hipcc_path, "--offload-arch=gfx950", "-std=c++20", "-O3", "-fPIC", "-shared",
                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", f"-I{INCLUDE_DIR}",
                   source_path, "-o", tmp_out]
        try:
            ret = subprocess.run(command, timeout=timeout, capture_output=True, text=True)
        except subprocess.TimeoutExpired:
            return None
        if ret.returncode != 0:
            errors = "\n".join(line for line in ret.stderr.splitlines() if "error" in line)[:2000]
            raise RuntimeError(f"Compilation failed for {file_name}:\n{errors}")
        os.replace(tmp_out, lib_path)
        return lib_path

    def _load(self, lib_path: str) -> ctypes.CDLL:
        lib = self._libs.get(lib_path)
        if lib is None:
            lib = ctypes.CDLL(lib_path)
            lib.kernel_entry.restype = ctypes.c_int
            lib.kernel_entry.argtypes = [ctypes.c_void_p] * 3
            lib.kernel_entry_stream.restype = ctypes.c_int
            lib.kernel_entry_stream.argtypes = [ctypes.c_void_p] * 4
            self._libs[lib_path] = lib
        return lib

    def apply(self, lib_path: str, torch_array: list, device: int = 0, stream: int | None = None) -> int:
        """Launch on torch's current stream of ``device`` (the reference launches on the default stream)."""
        lib = self._load(lib_path)
        torch.cuda.set_device(device)
        if stream is None:
            stream = torch.cuda.current_stream().cuda_stream
        return lib.kernel_entry_stream(*[ctypes.c_void_p(arr.data_ptr()) for arr in torch_array], ctypes.c_void_p(stream))


_builders: dict[tuple, Compile] = {}


def gemm_func(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor, M: int, N: int, K: int, kM: int, kN: int, kChunkK: int,
              warp_per_row: int, warp_per_col: int, kernel: str = "tile_library", tmp_dir: str | None = None) -> torch.Tensor:
    """C = A @ B.T with the instantiation (kM x kN tile, kChunkK k-chunk, warp layout) compiled on first use."""
    if tuple(A.shape) != (M, K) or tuple(B.shape) != (N, K) or tuple(C.shape) != (M, N):
        raise ValueError("A must be [M, K], B [N, K], C [M, N]")
    if A.dtype != torch.float16 or B.dtype != torch.float16 or C.dtype != torch.float32:
        raise ValueError("A and B must be float16 and C float32")
    if not (A.is_cuda and B.is_cuda and C.is_cuda and A.is_contiguous() and B.is_contiguous() and C.is_contiguous()):
        raise ValueError("operands must be contiguous device tensors")
    builder = _builders.setdefault((kernel, tmp_dir), Compile(file_prefix="gemm", tmp_dir=tmp_dir, kernel=kernel))
    lib_name = builder.compile(M, N, K, kM, kN, kChunkK, warp_per_row, warp_per_col)
    if lib_name is None:
        raise RuntimeError("Failed to compile the library.")
    rc = builder.apply(lib_name, [A, B, C], device=A.device.index or 0)
    if rc != 0:
        raise RuntimeError(f"kernel_entry returned {rc}")
    return C


def sweep(M: int, N: int, K: int, candidates, kernel: str = "tile_library", iters: int = 50, warmup: int = 5,
          epsilon: float = 5e-2, tmp_dir: str | None = None):
    """Time every (TM, TN, kChunkK, (warp_per_row, warp_per_col)) of ``candidates`` on random operands, checking
    each against ``a @ b.t()`` with the reference's criterion (mean absolute difference <= epsilon,
    main.py:29-33). Returns a list of dicts sorted by time; instantiations that do not compile are reported with
    ``ms = None`` and the compiler's message."""
    device = torch.device("cuda")
    a = torch.randn(M, K, device=device, dtype=torch.float16)
    b = torch.randn(N, K, device=device, dtype=torch.float16)
    c = torch.zeros(M, N, device=device, dtype=torch.float32)
    ref = a.float() @ b.float().t()
    results = []
    for TM, TN, chunk, (wr, wc) in candidates:
        entry = {"tile": (TM, TN, chunk), "warps": (wr, wc), "threads": wr * wc * 64, "ms": None}
        try:
            gemm_func(a, b, c, M, N, K, TM, TN, chunk, wr, wc, kernel=kernel, tmp_dir=tmp_dir)
        except RuntimeError as e:
            entry["error"] = str(e).splitlines()[0]
            results.append(entry)
            continue
        entry["mean_abs_diff"] = float((ref - c).abs().mean())
        entry["ok"] = entry["mean_abs_diff"] <= epsilon
        for _ in range(warmup):
            gemm_func(a, b, c, M, N, K, TM, TN, chunk, wr, wc, kernel=kernel, tmp_dir=tmp_dir)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            gemm_func(a, b, c, M, N, K, TM, TN, chunk, wr, wc, kernel=kernel, tmp_dir=tmp_dir)
        stop.record()
        torch.cuda.synchronize()
        entry["ms"] = start.elapsed_time(stop) / iters
        entry["tflops"] = 2.0 * M * N * K / (entry["ms"] * 1e-3) / 1e12
        results.append(entry)
    return sorted(results, key=lambda r: (r["ms"] is None, r["ms"] or 0.0))
