"""``torch.ops.tiledcuda.*``: the reference's operator library on PyTorch-ROCm.

The reference registers two ops with ``TORCH_LIBRARY(tiledcuda, t)`` (src/torch_bind.cc:8-11):
``scatter_nd(Tensor(a!) data, Tensor updates, Tensor indices) -> ()`` and
``flash_attention_fwd(Tensor Q, Tensor K, Tensor V, Tensor(a!) O, int m, int n, int k, int p) -> ()``
(schemas inferred from kernels/scatter_nd.hpp:39-40 and kernels/flash_attn.hpp:35-37), and its Python package loads
that library with ``torch.ops.load_library`` (pytiledcuda/__init__.py:3). Importing this module does the same with
``lib/libtiledcuda_torch.so`` (built from ``csrc/torch_bind.cc`` against the installed torch): the same two ops, with
the same names and argument order, plus ``gemm``, ``b2b_gemm`` and ``lstm`` for the other kernel entries, registered
from C++ so that a C++ program can load the same file. Every implementation is a call into the C-ABI library on
torch's current HIP stream; nothing synchronises the device (the reference op launches on stream 0 and calls
``cudaDeviceSynchronize()``, src/kernels/flash_attn.cu:418-421) and there is no CPU implementation: calling an op
with CPU tensors raises, as an op registered for one backend does.
"""
from __future__ import annotations

import os

import torch

import tiledcuda_amd as _tcu

SCHEMAS = ("scatter_nd", "flash_attention_fwd", "gemm", "b2b_gemm", "lstm")

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libtiledcuda_torch.so")


def library_path() -> str:
    """The shared library holding the C++ registrations (what a C++ caller passes to torch's library loader)."""
    return _LIB_PATH


if not os.path.exists(_LIB_PATH):
    raise ImportError(f"{_LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`. "
                      "There is no Python fallback registration.")
_tcu.lib()  # the operator library links against the C-ABI library next to it
torch.ops.load_library(_LIB_PATH)
