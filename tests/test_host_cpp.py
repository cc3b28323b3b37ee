"""Runs the C++ tests of the host-side operator mirror (ane-fieldfare_amd/host/fieldfare_host.hpp).

The binaries are built by __graft_entry__.build() (tests/host/build.sh): the host-logic test needs no
GPU; the GPU test drives the mirrored classes against the library and checks against the CPU oracle."""
import subprocess
from pathlib import Path

import pytest

HOST = Path(__file__).resolve().parent / "host"


def _run(name, timeout):
    exe = HOST / name
    if not exe.exists():
        subprocess.run(["bash", str(HOST / "build.sh")], check=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=timeout)
    print(res.stdout, res.stderr)
    assert res.returncode == 0, res.stdout + res.stderr
    return res.stdout


def test_host_logic_cpp():
    assert "host logic ok" in _run("test_host_logic", 60)


@pytest.mark.gpu
def test_host_operators_on_gpu_cpp():
    assert "host gpu ok" in _run("test_host_gpu", 120)
