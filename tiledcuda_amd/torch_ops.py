"""``torch.ops.tiledcuda.*``: the reference's operator library on PyTorch-ROCm.

The reference registers two ops with ``TORCH_LIBRARY(tiledcuda, t)`` (src/torch_bind.cc:8-11):
``scatter_nd(Tensor(a!) data, Tensor updates, Tensor indices) -> ()`` and
``flash_attention_fwd(Tensor Q, Tensor K, Tensor V, Tensor(a!) O, int m, int n, int k, int p) -> ()``
(schemas inferred from kernels/scatter_nd.hpp:39-40 and kernels/flash_attn.hpp:35-37). Importing this module
defines the same two ops, with the same names and argument order, plus ``gemm``, ``b2b_gemm`` and ``lstm``
for the other kernel entries. Every implementation is a call into the C-ABI library on torch's current HIP
stream; nothing synchronises the device (the reference op launches on stream 0 and calls
``cudaDeviceSynchronize()``, src/kernels/flash_attn.cu:418-421) and there is no CPU implementation: calling an
op with CPU tensors raises, as an op registered for one backend does.
"""
from __future__ import annotations

import torch

import tiledcuda_amd as _tcu

_lib = torch.library.Library("tiledcuda", "DEF")
_lib.define("scatter_nd(Tensor(a!) data, Tensor updates, Tensor indices) -> ()")
_lib.define("flash_attention_fwd(Tensor Q, Tensor K, Tensor V, Tensor(a!) O, int m, int n, int k, int p) -> ()")
_lib.define("gemm(Tensor A, Tensor B, Tensor(a!) C) -> ()")
_lib.define("b2b_gemm(Tensor A, Tensor B, Tensor C, Tensor(a!) D) -> ()")
_lib.define("lstm(Tensor x, Tensor W, Tensor bias, Tensor? h0, Tensor? c0) -> (Tensor, Tensor)")

SCHEMAS = ("scatter_nd", "flash_attention_fwd", "gemm", "b2b_gemm", "lstm")


def _scatter_nd(data, updates, indices):
    # the reference op's argument order: (data, updates, indices)
    _tcu.scatter_nd(data, indices, updates)


def _flash_attention_fwd(Q, K, V, O, m, n, k, p):
    _tcu.flash_attention_fwd(Q, K, V, O, m, n, k, p)


def _gemm(A, B, C):
    _tcu.gemm(A, B, out=C)


def _b2b_gemm(A, B, C, D):
    _tcu.b2b_gemm(A, B, C, out=D if D.dim() == 3 else D.unsqueeze(0))


def _lstm(x, W, bias, h0, c0):
    return _tcu.lstm(x, W, bias, h0, c0)


for _name, _fn in (("scatter_nd", _scatter_nd), ("flash_attention_fwd", _flash_attention_fwd), ("gemm", _gemm),
                   ("b2b_gemm", _b2b_gemm), ("lstm", _lstm)):
    _lib.impl(_name, _fn, "CUDA")
