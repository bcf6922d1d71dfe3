"""The ABI consumed from plain C (tests/c_client/abi_client.c, built by __graft_entry__.build()):
no Python between the caller and the library, as with cgo."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CLIENT = os.path.join(HERE, "c_client", "abi_client.bin")


def run_client():
    return subprocess.run([CLIENT], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)


def test_c_client_links_and_reports_a_missing_gpu_cleanly():
    r = run_client()
    assert r.returncode in (0, 2), r.stdout          # 2: create_metal_device() returned nil, nothing crashed
    if r.returncode == 2:
        assert "no usable GPU" in r.stdout


@pytest.mark.gpu
def test_c_client_is_bit_identical_on_the_gpu():
    r = run_client()
    assert r.returncode == 0, r.stdout
    assert "bit-identical" in r.stdout
