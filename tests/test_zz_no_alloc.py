"""tcu_lstm_f16_noalloc: the LSTM layer with the hoisted input projection whose [T, B, 4H] f32 pre-activations go to
a buffer that is part of the library's device image, for callers that cannot allocate. Called through the C-ABI
(ctypes, raw pointers) and compared bit for bit with tcu_lstm_f16_ws on a caller-owned workspace (the two run the
same kernels), and against the CPU oracle to the LSTM tolerance; two calls in a row, the second with a smaller input,
so that whatever the first left in the shared buffer is seen not to matter. Collected last: a failure here must not
hide the other tests behind `pytest -x`."""
import numpy as np
import pytest

ABS_TOL = 1e-2  # max absolute error against the f32 oracle (the tolerance the LSTM configuration states)


def _layer(oracle, T, B, I, H, seed):
    x = oracle.fill_normal(T * B * I, seed, 0, 0.5).reshape(T, B, I)
    W = oracle.fill_normal(4 * H * (I + H), seed + 1, 0, 0.05).reshape(4 * H, I + H)
    b = oracle.fill_normal(4 * H, seed + 2, 0, 0.1)
    h0 = oracle.fill_normal(B * H, seed + 3, 0, 0.5).reshape(B, H)
    c0 = oracle.fill_normal(B * H, seed + 4, 0, 0.5).reshape(B, H).astype(np.float32)
    return x, W, b, h0, c0


@pytest.mark.gpu
def test_no_alloc_entry_matches_workspace_entry(tcu, oracle, device):
    import torch

    lib = tcu.lib()
    limit = int(lib.tcu_lstm_noalloc_max_bytes())
    assert limit == 64 << 20
    stream = torch.cuda.current_stream().cuda_stream
    # first the largest layer that fits (the C5 shape: exactly the limit), then a much smaller one
    for T, B, I, H, seed, ref_rows in ((16, 256, 1024, 1024, 900, (100, 102)), (4, 64, 128, 128, 910, None)):
        print(f"lstm noalloc T{T} B{B} I{I} H{H}", flush=True)
        x, W, b, h0, c0 = _layer(oracle, T, B, I, H, seed)
        dx, dW, db, dh0, dc0 = (torch.from_numpy(np.ascontiguousarray(a)).to(device) for a in (x, W, b, h0, c0))
        need = int(lib.tcu_lstm_workspace_bytes(T, B, I, H))
        assert 0 < need <= limit
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        h_ws = torch.empty(T, B, H, dtype=torch.float16, device=device)
        c_ws = torch.empty(B, H, dtype=torch.float32, device=device)
        h_na = torch.full((T, B, H), float("nan"), dtype=torch.float16, device=device)
        c_na = torch.full((B, H), float("nan"), dtype=torch.float32, device=device)
        torch.cuda.synchronize()  # every output buffer exists before the entry point under test runs
        rc = lib.tcu_lstm_f16_ws(dx.data_ptr(), dW.data_ptr(), db.data_ptr(), dh0.data_ptr(), dc0.data_ptr(),
                                 h_ws.data_ptr(), c_ws.data_ptr(), T, B, I, H, ws.data_ptr(), need, stream)
        assert rc == 0, tcu.last_error()
        before = torch.cuda.memory_allocated()
        # free device memory as the driver sees it (hipMemGetInfo): a hipMalloc inside the library would move this one,
        # which torch's own counter cannot see. Compared from the second layer on: by then the scratch array's address
        # has been looked up and every kernel of the call has run once (tcu_lstm_f16_ws above runs the same ones).
        free_before = torch.cuda.mem_get_info()[0]
        rc = lib.tcu_lstm_f16_noalloc(dx.data_ptr(), dW.data_ptr(), db.data_ptr(), dh0.data_ptr(), dc0.data_ptr(),
                                      h_na.data_ptr(), c_na.data_ptr(), T, B, I, H, stream)
        assert rc == 0, tcu.last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        if seed != 900:
            assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(h_na, h_ws) and torch.equal(c_na, c_ws)  # same kernels, same operands: bit-identical
        rows = ref_rows or (0, B)
        h_ref, c_ref = oracle.lstm(x, W, b, h0, c0, rows=rows) if ref_rows else oracle.lstm(x, W, b, h0, c0)
        sl = slice(rows[0], rows[1])
        assert oracle.max_abs_err(h_na[:, sl].float().cpu().numpy(), h_ref[:, sl]) <= ABS_TOL
        assert oracle.max_abs_err(c_na[sl].cpu().numpy(), c_ref[sl]) <= ABS_TOL


@pytest.mark.gpu
def test_no_alloc_entry_rejects_layers_beyond_its_buffer(tcu, device):
    import torch

    lib = tcu.lib()
    T, B, I, H = 32, 256, 1024, 1024  # 128 MiB of pre-activations
    t = torch.zeros(16, dtype=torch.float16, device=device)  # never dereferenced: the size check comes first
    p = t.data_ptr()
    rc = lib.tcu_lstm_f16_noalloc(p, p, p, 0, 0, p, p, T, B, I, H, 0)
    assert rc == tcu.TCU_ERR_UNSUPPORTED_SHAPE
    assert "static scratch buffer" in tcu.last_error()
