"""A consumer of the library that is neither Python nor torch: the native program
of tests/native/abi_roundtrip_driver.cpp drives every engine through the C ABI
and checks each byte against its own host model.  Built beforehand by
``make -C tests/native`` (``__graft_entry__.build()`` does it)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BUILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "build")


def test_native_consumer_of_the_c_abi(gpu_device):
    exe = os.path.join(BUILD, "abi_roundtrip_driver")
    assert os.path.exists(exe), f"{exe} is missing: run make -C tests/native"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert "ok: 36 cases through the C ABI" in r.stdout, r.stdout


def test_two_threads_of_a_native_program_put_and_get_at_once(gpu_device):
    """tests/native/two_way_driver.cpp: concurrent calls from plain C++ threads,
    every block compared afterwards.  The rates it prints are reported, not asserted."""
    exe = os.path.join(BUILD, "two_way_driver")
    assert os.path.exists(exe), f"{exe} is missing: run make -C tests/native"
    r = subprocess.run([exe, "0.4", "64"], capture_output=True, text=True, timeout=120)
    print(r.stdout)
    assert r.returncode == 0 and r.stdout.startswith("ok:"), r.stdout + r.stderr
