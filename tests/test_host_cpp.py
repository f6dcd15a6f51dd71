"""The C++ host layer (vulkanforge_amd/host/vfkv_host.hpp) through its self-test binary: layout
arithmetic on any machine, closed-form decode checks when a GPU is present."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "vulkanforge_amd", "host", "selftest")


def _run():
    if not os.path.exists(BIN):
        pytest.skip("host self-test binary not built (make -C vulkanforge_amd/host)")
    return subprocess.run([BIN], capture_output=True, text=True, timeout=120)


def test_host_layer_layout_checks():
    r = _run()
    assert r.returncode == 0, r.stdout + r.stderr
    assert "passed" in r.stdout


@pytest.mark.gpu
def test_host_layer_decode_closed_forms_on_gpu():
    r = _run()
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout, r.stdout
