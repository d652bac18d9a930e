"""Runs the host-only C++ checks of the type layer (layouts, iterators, shapes, LDS swizzle,
workgroup->tile map): tests/host/host_tests.hip, which restates the reference's
tests/cpp/cell/test_layout.cu and test_global_tile_iterator.cu. Needs hipcc, not a GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "host", "host_tests.hip")
EXE = os.path.join(ROOT, "tests", "host", "_build", "host_tests")


def _newest_header_mtime():
    newest = os.path.getmtime(SRC)
    for d, _, files in os.walk(os.path.join(ROOT, "include")):
        for f in files:
            newest = max(newest, os.path.getmtime(os.path.join(d, f)))
    return newest


def test_host_type_layer():
    if not os.path.exists(EXE) or os.path.getmtime(EXE) < _newest_header_mtime():
        if shutil.which("hipcc") is None:
            pytest.skip("hipcc not available and no prebuilt host test binary")
        os.makedirs(os.path.dirname(EXE), exist_ok=True)
        subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-std=c++20", "-O1", "-I" + os.path.join(ROOT, "include"),
                               SRC, "-o", EXE], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    proc = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "OK (0 failed checks)" in proc.stdout
