"""Run-time compiled GEMM instantiations (the reference's examples/python/gemm: compile.py, entry.py, gemm.py,
main.py). CPU part: the generated translation units compile for gfx950 and export the reference's
`kernel_entry`; a tile that does not fit raises instead of producing a library. GPU part: compile, launch,
compare with the oracle; a two-candidate sweep."""
import ctypes
import os

import pytest
import torch


@pytest.fixture(scope="module")
def jit(tcu):
    from tiledcuda_amd import jit as module

    return module


def test_generated_sources_compile_and_export_kernel_entry(jit, tmp_path):
    for kind, cfg in (("tile_library", (256, 256, 256, 64, 64, 32, 2, 2)), ("pipelined", (256, 256, 256, 128, 128, 64, 2, 2)),
                      ("tile_wave128", (512, 256, 192, 256, 256, 64, 2, 2))):
        builder = jit.Compile(file_prefix="t", tmp_dir=str(tmp_path), kernel=kind)
        path = builder.compile(*cfg)
        assert path and os.path.exists(path)
        assert builder.compile(*cfg) == path  # cached by name
        text = open(path[:-3] + ".hip").read()
        assert 'extern "C" int kernel_entry(__half* parameter1, __half* parameter2, float* parameter3)' in text
        # symbol presence without loading the HIP runtime: look the name up in the file
        assert b"kernel_entry_stream" in open(path, "rb").read()


def test_cache_key_follows_the_source_and_cache_dir_is_private(jit, tmp_path, monkeypatch):
    """The library name carries a digest of the generated source and of the headers: a changed kernel header must
    not resolve to the library built from the old one. The default cache directory is private to the user."""
    import stat
    import subprocess

    calls = []

    def fake_run(cmd, **kw):
        calls.append(cmd)
        open(cmd[-1], "wb").close()
        return subprocess.CompletedProcess(cmd, 0, "", "")

    monkeypatch.setattr(jit.subprocess, "run", fake_run)
    builder = jit.Compile(file_prefix="k", tmp_dir=str(tmp_path))
    cfg = (256, 256, 256, 64, 64, 32, 2, 2)
    first = builder.compile(*cfg)
    assert builder.compile(*cfg) == first and len(calls) == 1
    monkeypatch.setattr(jit, "_headers_digest", lambda: "a different set of headers")
    second = builder.compile(*cfg)
    assert second != first and len(calls) == 2

    monkeypatch.setenv("XDG_CACHE_HOME", str(tmp_path / "cache"))
    path = jit.Compile().tmp_dir
    assert path.startswith(str(tmp_path / "cache"))
    assert stat.S_IMODE(os.stat(path).st_mode) == 0o700


def test_bad_instantiation_raises(jit, tmp_path):
    builder = jit.Compile(file_prefix="bad", tmp_dir=str(tmp_path))
    with pytest.raises(RuntimeError, match="Compilation failed"):
        builder.compile(256, 256, 256, 96, 64, 32, 2, 2)  # 96 does not divide 256


@pytest.mark.gpu
@pytest.mark.parametrize("kind,cfg", [("tile_library", (64, 64, 32, 2, 2)), ("pipelined", (128, 128, 64, 2, 2)),
                                      ("tile_wave128", (256, 256, 64, 2, 2))])
def test_jit_gemm_matches_oracle(jit, oracle, device, tmp_path, kind, cfg):
    M = N = K = 256
    A = oracle.fill_uniform(M * K, 41).reshape(M, K)
    Bt = oracle.fill_uniform(N * K, 42).reshape(N, K)
    a, b = torch.from_numpy(A).to(device), torch.from_numpy(Bt).to(device)
    c = torch.full((M, N), float("nan"), dtype=torch.float32, device=device)
    jit.gemm_func(a, b, c, M, N, K, *cfg, kernel=kind, tmp_dir=str(tmp_path))
    assert oracle.max_rel_err(c.cpu().numpy(), oracle.gemm(A, Bt)) <= 1e-3  # fp32 accumulate, fp32 out


@pytest.mark.gpu
def test_sweep_orders_candidates(jit, device, tmp_path):
    res = jit.sweep(512, 512, 512, [(64, 64, 32, (2, 2)), (128, 128, 64, (2, 2)), (96, 64, 32, (2, 2))],
                    kernel="tile_library", iters=5, warmup=1, tmp_dir=str(tmp_path))
    assert len(res) == 3
    assert res[-1]["ms"] is None and "Compilation failed" in res[-1]["error"]
    assert all(r["ok"] for r in res[:2]) and res[0]["ms"] <= res[1]["ms"]
