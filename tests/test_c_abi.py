"""The C-ABI boundary without a GPU: the library loads, exports every symbol declared in
include/tcu_c_api.h, and rejects bad arguments with a status code and a message instead of
touching the device (the reference's launcher calls exit() on errors, cuda_utils.hpp:20-27;
its op throws on unsupported shapes, src/kernels/flash_attn.cu:453-455)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tcu_c_api.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tcu_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_entry_points():
    syms = declared_symbols()
    for name in ("tcu_gemm_f16", "tcu_b2b_gemm_f16", "tcu_flash_attn_fwd_f16", "tcu_lstm_f16", "tcu_flash_attn_fwd_f16_algo", "tcu_lstm_f16_algo", "tcu_lstm_f16_ws", "tcu_lstm_workspace_bytes", "tcu_lstm_f16_noalloc", "tcu_lstm_noalloc_max_bytes", "tcu_last_error",
                 "tcu_version", "tcu_device_count"):
        assert name in syms


def test_library_exports_every_declared_symbol(tcu):
    handle = ctypes.CDLL(tcu.library_path())
    for name in declared_symbols():
        assert hasattr(handle, name), f"{name} declared in tcu_c_api.h but not exported"
    # and the Python binding table covers the same set
    assert sorted(tcu._SIGNATURES) == declared_symbols()


def test_version_and_error_string(tcu):
    assert tcu.lib().tcu_version() >= 100
    assert isinstance(tcu.last_error(), str)


@pytest.mark.parametrize("call", [
    lambda l: l.tcu_gemm_f16(0, 0, 0, 128, 64, 256, 0, 0, 0),
    lambda l: l.tcu_b2b_gemm_f16(0, 0, 0, 0, 64, 64, 64, 64, 1, 0, 0),
    lambda l: l.tcu_flash_attn_fwd_f16(0, 0, 0, 0, 1, 64, 64, 128, 128, 1.0, 0, 0),
    lambda l: l.tcu_lstm_f16(0, 0, 0, 0, 0, 0, 0, 1, 64, 128, 128, 0),
])
def test_null_pointers_are_rejected(tcu, call):
    assert call(tcu.lib()) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert "null pointer" in tcu.last_error()


def test_misaligned_operands_are_rejected(tcu):
    """The kernels move 16 bytes per lane: an operand that does not start on a 16-byte boundary is refused before
    anything is launched."""
    l = tcu.lib()
    p, q = 0x1000, 0x1002
    assert l.tcu_gemm_f16(q, p, p, 64, 64, 64, 0, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert "16-byte aligned" in tcu.last_error()
    assert l.tcu_b2b_gemm_f16(p, p, q, p, 64, 64, 64, 64, 1, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_flash_attn_fwd_f16(p, p, p, q, 1, 64, 64, 128, 128, 1.0, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_lstm_f16(p, p, p, 0, q, p, p, 1, 64, 128, 128, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert "16-byte aligned" in tcu.last_error()


def test_lstm_workspace_entry_point_checks_its_arguments(tcu):
    """tcu_lstm_f16_ws / tcu_lstm_workspace_bytes: everything that can be refused is refused before a launch."""
    l = tcu.lib()
    p = 0x1000
    assert l.tcu_lstm_workspace_bytes(16, 256, 1024, 1024) == 16 * 256 * 4096 * 4
    assert l.tcu_lstm_workspace_bytes(4, 64, 128, 128) == 4 * 64 * 512 * 4
    assert l.tcu_lstm_workspace_bytes(3, 64, 128, 128) == 0    # T * B not a multiple of 256
    assert l.tcu_lstm_workspace_bytes(4, 32, 128, 128) == 0    # B not a multiple of 64
    assert l.tcu_lstm_workspace_bytes(4, 64, 64, 128) == 0     # (I, H) not instantiated for this path
    assert l.tcu_lstm_workspace_bytes(0, 64, 128, 128) == 0
    need = 4 * 64 * 512 * 4
    assert l.tcu_lstm_f16_ws(p, p, p, 0, 0, p, p, 4, 64, 128, 128, 0, need, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert "null pointer" in tcu.last_error()
    assert l.tcu_lstm_f16_ws(p, p, p, 0, 0, p, p, 4, 64, 128, 128, p, need - 1, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert "workspace" in tcu.last_error()
    assert l.tcu_lstm_f16_ws(p, p, p, 0, 0, p, p, 4, 64, 128, 128, p + 4, need, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_lstm_f16_ws(p, p, p, 0, 0, p, p, 3, 64, 128, 128, p, need, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_lstm_f16_ws(p, p, p, 0, 0, p, p, 4, 64, 128, -1, p, need, 0) == tcu.TCU_ERR_INVALID_ARGUMENT


def test_no_alloc_lstm_entry_point_checks_its_arguments(tcu):
    """tcu_lstm_f16_noalloc refuses, before any device call, what its fixed buffer cannot hold."""
    l = tcu.lib()
    p = 0x1000
    limit = l.tcu_lstm_noalloc_max_bytes()
    assert limit == 64 << 20 == l.tcu_lstm_workspace_bytes(16, 256, 1024, 1024)
    assert l.tcu_lstm_f16_noalloc(p, p, p, 0, 0, p, p, 32, 256, 1024, 1024, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert "static scratch buffer" in tcu.last_error() and str(limit) in tcu.last_error()
    assert l.tcu_lstm_f16_noalloc(p, p, p, 0, 0, p, p, 3, 64, 128, 128, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_lstm_f16_noalloc(p, p, 0, 0, 0, p, p, 4, 64, 128, 128, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert "null pointer" in tcu.last_error()
    assert l.tcu_lstm_f16_noalloc(p, p, p, 0, 0, p + 2, p, 4, 64, 128, 128, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_lstm_f16_noalloc(p, p, p, 0, 0, p, p, 4, 64, 128, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT


def test_bad_sizes_and_enums_are_rejected(tcu):
    l = tcu.lib()
    p = 0x1000  # never dereferenced: argument checks come first
    assert l.tcu_gemm_f16(p, p, p, 0, 64, 64, 0, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_gemm_f16(p, p, p, 64, 64, 64, 7, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert "out_dtype" in tcu.last_error()
    assert l.tcu_gemm_f16(p, p, p, 64, 64, 64, 0, 10, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_b2b_gemm_f16(p, p, p, p, 64, 64, 64, 64, -1, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_b2b_gemm_f16_algo(p, p, p, p, 64, 256, 128, 128, 1, 0, 9, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_b2b_gemm_f16_algo(p, p, p, p, 64, 64, 64, 64, 1, 0, 2, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_flash_attn_fwd_f16(p, p, p, p, 1, 64, 64, 128, 128, 1.0, 5, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    dims = (ctypes.c_longlong * 2)(4, 4)
    assert l.tcu_scatter_nd(0, p, p, dims, 2, 1, 1, 0, 0, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_scatter_nd(p, p, p, dims, 2, 1, 3, 0, 0, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT  # k > rank
    assert l.tcu_scatter_nd(p, p, p, dims, 9, 1, 1, 0, 0, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT  # rank > 8
    assert l.tcu_scatter_nd(p, p, p, dims, 2, 1, 1, 0, 7, 0, 0) == tcu.TCU_ERR_INVALID_ARGUMENT  # mode
    assert l.tcu_scatter_nd(p, p, p, dims, 2, 0, 1, 0, 0, 0, 0) == tcu.TCU_OK  # no rows: nothing to launch
    assert l.tcu_lstm_f16(p, p, p, 0, 0, p, p, 0, 64, 128, 128, 0) == tcu.TCU_ERR_INVALID_ARGUMENT


def test_unsupported_shapes_are_reported_not_launched(tcu):
    l = tcu.lib()
    p = 0x1000
    assert l.tcu_gemm_f16(p, p, p, 100, 64, 64, 0, 0, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_gemm_f16(p, p, p, 64, 64, 40, 0, 3, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_gemm_f16(p, p, p, 64, 72, 64, 0, 6, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # whole 16 x 16 tiles only
    assert l.tcu_gemm_f16(p, p, p, 64, 64, 40, 0, 0, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_gemm_f16(p, p, p, 256, 256, 256, 0, 1, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_gemm_f16(p, p, p, 128, 256, 40, 0, 4, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # one wavefront per SIMD: M, N, K % 16
    assert l.tcu_gemm_f16(p, p, p, 120, 256, 64, 0, 4, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_gemm_f16(p, p, p, 512, 512, 512, 0, 7, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # tile-API kernels: fixed shapes
    assert l.tcu_gemm_f16(p, p, p, 256, 256, 192, 0, 8, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # K-splitting kernel: K % 128
    assert l.tcu_gemm_f16(p, p, p, 200, 256, 256, 0, 8, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # ... and M, N % 16 (edge tiles)
    assert l.tcu_gemm_f16(p, p, p, 256, 256, 256, 0, 10, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_gemm_f16(p, p, p, 256, 200, 256, 1, 9, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # 256 x 128 tiles: M, N % 16 (edge tiles)
    assert l.tcu_gemm_f16(p, p, p, 256, 256, 96, 1, 9, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # ... and K % 64
    assert l.tcu_b2b_gemm_f16(p, p, p, p, 64, 96, 64, 64, 1, 0, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_flash_attn_fwd_f16(p, p, p, p, 1, 64, 64, 128, 64, 1.0, 0, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_flash_attn_fwd_f16(p, p, p, p, 1, 64, 100, 128, 128, 1.0, 1, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_flash_attn_fwd_f16(p, p, p, p, 1, 64, 192, 64, 64, 1.0, 0, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # col-major V: D 128 only
    assert l.tcu_flash_attn_fwd_f16_algo(p, p, p, p, 1, 64, 192, 128, 128, 1.0, 0, 1, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # tile library: fixed N
    assert l.tcu_flash_attn_fwd_f16_algo(p, p, p, p, 1, 256, 256, 64, 64, 1.0, 1, 4, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # wave64: D 128 only
    assert l.tcu_flash_attn_fwd_f16_algo(p, p, p, p, 1, 512, 512, 128, 128, 1.0, 1, 5, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # tile-API wave64: fixed (M, N)
    assert l.tcu_flash_attn_fwd_f16_algo(p, p, p, p, 1, 2048, 2048, 128, 128, 1.0, 0, 5, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # ... and a row-major V
    assert l.tcu_flash_attn_fwd_f16_algo(p, p, p, p, 1, 256, 256, 128, 128, 1.0, 1, 6, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # 16x16x32 wave64: N >= 320
    assert l.tcu_flash_attn_fwd_f16_algo(p, p, p, p, 1, 256, 640, 64, 64, 1.0, 0, 6, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # ... head size 64 only with a row-major V
    assert l.tcu_flash_attn_fwd_f16_algo(p, p, p, p, 1, 256, 256, 128, 128, 1.0, 1, 7, 0) == tcu.TCU_ERR_INVALID_ARGUMENT  # no such algo
    assert l.tcu_b2b_gemm_f16_algo(p, p, p, p, 64, 512, 128, 128, 1, 1, 4, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE  # tile-API resident: fixed N
    assert l.tcu_b2b_gemm_f16_algo(p, p, p, p, 64, 256, 128, 128, 1, 1, 5, 0) == tcu.TCU_ERR_INVALID_ARGUMENT
    assert l.tcu_lstm_f16(p, p, p, 0, 0, p, p, 1, 64, 100, 128, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert l.tcu_lstm_f16(p, p, p, 0, 0, p, p, 1, 10, 128, 128, 0) == tcu.TCU_ERR_UNSUPPORTED_SHAPE


def test_python_wrappers_validate_before_calling(tcu):
    import torch

    a = torch.zeros(64, 64, dtype=torch.float16)
    with pytest.raises(ValueError, match="device memory"):
        tcu.gemm(a, a)
    with pytest.raises(ValueError, match="mismatched K"):
        tcu.gemm(a, torch.zeros(64, 32, dtype=torch.float16))
    with pytest.raises(ValueError, match="W must be"):
        tcu.lstm(torch.zeros(1, 64, 128, dtype=torch.float16), torch.zeros(512, 100, dtype=torch.float16),
                 torch.zeros(512, dtype=torch.float16))
    err = tcu.TcuError(-2, "x")
    assert isinstance(err, RuntimeError) and err.status == -2


def test_python_wrappers_check_operand_shapes_against_each_other(tcu):
    """A key/value tensor with fewer leading dimensions than the query (the MQA/GQA habit), a mismatched key count,
    a wrongly shaped output or initial state would make a kernel read or write past an allocation: all of them are
    refused on the host, before any pointer is taken (so CPU tensors suffice here)."""
    import torch

    f16 = torch.float16
    q = torch.zeros(2, 4, 128, 64, dtype=f16)
    kv = torch.zeros(2, 4, 256, 64, dtype=f16)
    with pytest.raises(ValueError, match="k must be"):
        tcu.flash_attention(q, torch.zeros(2, 1, 256, 64, dtype=f16), kv)
    with pytest.raises(ValueError, match="k must be"):
        tcu.flash_attention(q, torch.zeros(256, 64, dtype=f16), kv)
    with pytest.raises(ValueError, match="k must be"):
        tcu.flash_attention(q, torch.zeros(2, 4, 256, 128, dtype=f16), kv)
    with pytest.raises(ValueError, match="v must be"):
        tcu.flash_attention(q, kv, torch.zeros(2, 4, 128, 64, dtype=f16))
    with pytest.raises(ValueError, match="v must be"):
        tcu.flash_attention(q, kv, torch.zeros(4, 256, 64, dtype=f16))
    with pytest.raises(ValueError, match="out must be"):
        tcu.flash_attention(q, kv, kv, out=torch.zeros(2, 4, 64, 64, dtype=f16))
    with pytest.raises(ValueError, match="device memory"):  # consistent shapes get as far as the device check
        tcu.flash_attention(q, kv, kv)

    # the reference's flattened call shape: every tensor must hold exactly batch * rows * cols elements
    Q, K, V, O = (torch.zeros(n, dtype=f16) for n in (64 * 128, 256 * 128, 128 * 256, 64 * 128))
    with pytest.raises(ValueError, match="K must hold"):
        tcu.flash_attention_fwd(Q, K[:-128], V, O, 64, 256, 128, 128)
    with pytest.raises(ValueError, match="V must hold"):
        tcu.flash_attention_fwd(Q, K, V, O, 64, 256, 128, 64)
    with pytest.raises(ValueError, match="Q must hold"):
        tcu.flash_attention_fwd(Q, K, V, O, 64, 256, 128, 128, batch=2)
    with pytest.raises(ValueError, match="O must hold"):
        tcu.flash_attention_fwd(Q, K, V, O[:100], 64, 256, 128, 128)
    with pytest.raises(ValueError, match="positive"):
        tcu.flash_attention_fwd(Q, K, V, O, 64, 0, 128, 128)
    with pytest.raises(ValueError, match="device memory"):
        tcu.flash_attention_fwd(Q, K, V, O, 64, 256, 128, 128)

    a, b, c = torch.zeros(64, 64, dtype=f16), torch.zeros(128, 64, dtype=f16), torch.zeros(32, 128, dtype=f16)
    with pytest.raises(ValueError, match="out must be"):
        tcu.b2b_gemm(a, b, c, out=torch.zeros(1, 64, 64, dtype=f16))
    with pytest.raises(ValueError, match="out must be"):
        tcu.b2b_gemm(a.unsqueeze(0), b.unsqueeze(0), c.unsqueeze(0), out=torch.zeros(64, 32, dtype=f16))
    with pytest.raises(ValueError, match="2-D or all be 3-D"):
        tcu.b2b_gemm(a.unsqueeze(0), b, c)
    with pytest.raises(ValueError, match="do not chain"):
        tcu.b2b_gemm(a, b, torch.zeros(32, 64, dtype=f16))
    with pytest.raises(ValueError, match="device memory"):
        tcu.b2b_gemm(a, b, c, out=torch.zeros(64, 32, dtype=f16))

    x, W, bias = torch.zeros(2, 64, 128, dtype=f16), torch.zeros(512, 256, dtype=f16), torch.zeros(512, dtype=f16)
    with pytest.raises(ValueError, match="h0 must be"):
        tcu.lstm(x, W, bias, h0=torch.zeros(32, 128, dtype=f16))
    with pytest.raises(ValueError, match="c0 must be"):
        tcu.lstm(x, W, bias, c0=torch.zeros(64, 64))
    with pytest.raises(ValueError, match="x must be"):
        tcu.lstm(x[0], W, bias)


def test_tile_test_library_loads():
    path = os.path.join(ROOT, "tests", "device", "_build", "libtcu_tile_tests.so")
    if not os.path.exists(path):
        pytest.skip("device test library not built")
    import torch  # noqa: F401  (load torch's HIP runtime first, as every user of the library does)

    handle = ctypes.CDLL(path)
    assert handle.tt_num_cases() > 50
