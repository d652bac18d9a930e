"""Writes the small golden fixtures in this directory.

Nothing here imports the reference or the oracle: expected outputs come from numpy float64
arithmetic (and, for the LSTM, torch.nn.LSTM on the CPU), i.e. from implementations that
share no code with oracle/oracle.c.  Inputs reuse the deterministic ramps of the
reference's own tests where it has them:
  * A[i] = (i % 2048) / 1000       tests/cpp/cell/test_single_wmma.cu:58-62
  * src[i] = i % 2048              tests/cpp/cell/test_g2s_load.cu:40
Run: python tests/golden/make_golden.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def ramp(n, div=1000.0):
    return ((np.arange(n) % 2048) / div).astype(np.float16)


def softmax64(s):
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=-1, keepdims=True)


def main():
    rng = np.random.default_rng(20240830)
    out = {}

    # GEMM on the reference's ramp, shapes of its test list (16^3 and 96x48x80)
    for (M, N, K) in [(16, 16, 16), (96, 48, 80), (128, 64, 256)]:
        A = ramp(M * K).reshape(M, K)
        Bt = ramp(N * K).reshape(N, K)[::-1].copy()  # asymmetric so a transposed operand is caught
        out[f"gemm_{M}x{N}x{K}_A"] = A
        out[f"gemm_{M}x{N}x{K}_Bt"] = Bt
        out[f"gemm_{M}x{N}x{K}_C"] = (A.astype(np.float64) @ Bt.astype(np.float64).T)

    # b2b: intermediate rounded to f16 by numpy
    M, N, K, P = 32, 64, 48, 16
    A = (rng.standard_normal((M, K)) * 0.1).astype(np.float16)
    Bt = (rng.standard_normal((N, K)) * 0.1).astype(np.float16)
    Ct = (rng.standard_normal((P, N)) * 0.1).astype(np.float16)
    acc = (A.astype(np.float64) @ Bt.astype(np.float64).T).astype(np.float32).astype(np.float16)
    out["b2b_A"], out["b2b_Bt"], out["b2b_Ct"] = A, Bt, Ct
    out["b2b_D"] = acc.astype(np.float64) @ Ct.astype(np.float64).T

    # attention, float64 softmax
    M, N, K, P = 16, 48, 32, 24
    Q = rng.standard_normal((M, K)).astype(np.float16)
    Kn = rng.standard_normal((N, K)).astype(np.float16)
    V = rng.standard_normal((N, P)).astype(np.float16)
    scale = 1.0 / np.sqrt(K)
    out["attn_Q"], out["attn_Kn"], out["attn_V"] = Q, Kn, V
    out["attn_scale"] = np.float32(scale)
    out["attn_O"] = softmax64(np.float64(np.float32(scale)) * (Q.astype(np.float64) @ Kn.astype(np.float64).T)) @ V.astype(np.float64)

    # LSTM via torch.nn.LSTM on the CPU (gate order i, f, g, o; separate input/hidden weights)
    import torch

    T, B, I, H = 4, 3, 8, 6
    x = (rng.standard_normal((T, B, I)) * 0.5).astype(np.float16)
    W = (rng.standard_normal((4 * H, I + H)) * 0.3).astype(np.float16)
    b = (rng.standard_normal(4 * H) * 0.3).astype(np.float16)
    h0 = (rng.standard_normal((B, H)) * 0.3).astype(np.float16)
    c0 = (rng.standard_normal((B, H)) * 0.3).astype(np.float32)
    m = torch.nn.LSTM(I, H, num_layers=1, bias=True).double()
    with torch.no_grad():
        m.weight_ih_l0.copy_(torch.from_numpy(W[:, :I].astype(np.float64)))
        m.weight_hh_l0.copy_(torch.from_numpy(W[:, I:].astype(np.float64)))
        m.bias_ih_l0.copy_(torch.from_numpy(b.astype(np.float64)))
        m.bias_hh_l0.zero_()
        y, (hT, cT) = m(torch.from_numpy(x.astype(np.float64)),
                        (torch.from_numpy(h0.astype(np.float64))[None], torch.from_numpy(c0.astype(np.float64))[None]))
    out["lstm_x"], out["lstm_W"], out["lstm_b"], out["lstm_h0"], out["lstm_c0"] = x, W, b, h0, c0
    out["lstm_h_all"] = y.numpy()  # float64, h never rounded to f16 between steps
    out["lstm_cT"] = cT[0].numpy()

    np.savez_compressed(os.path.join(HERE, "golden_small.npz"), **out)
    print("wrote", os.path.join(HERE, "golden_small.npz"), os.path.getsize(os.path.join(HERE, "golden_small.npz")), "bytes")


if __name__ == "__main__":
    main()
