"""A consumer of the library that is neither Python nor torch: the native program
of tests/native/abi_roundtrip_driver.cpp drives every engine through the C ABI
and checks each byte against its own host model.  It runs twice: against the
shipped library, and against a build of the library whose host code is under
AddressSanitizer (the device code is the same).  Both are built beforehand by
``make -C tests/native`` (``__graft_entry__.build()`` does it)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BUILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "build")


def run(exe, **env):
    assert os.path.exists(exe), f"{exe} is missing: run make -C tests/native"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300,
                       env=dict(os.environ, **env))
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert "ok: 32 cases through the C ABI" in r.stdout, r.stdout
    return r


def test_native_consumer_of_the_c_abi(gpu_device):
    run(os.path.join(BUILD, "abi_roundtrip_driver"))


def test_host_code_under_address_sanitizer(gpu_device):
    r = run(os.path.join(BUILD, "asan", "abi_roundtrip_driver"),
            ASAN_OPTIONS="protect_shadow_gap=0:detect_leaks=0:verify_asan_link_order=0")
    assert "AddressSanitizer" not in r.stderr


@pytest.mark.parametrize("asan", [False, True], ids=["plain", "asan"])
def test_two_threads_of_a_native_program_put_and_get_at_once(gpu_device, asan):
    """tests/native/two_way_driver.cpp: concurrent calls from plain C++ threads,
    every block compared afterwards; both directions together move more than
    either alone.  Also against the library whose host code is under
    AddressSanitizer, with the lane streams forced on."""
    exe = os.path.join(BUILD, "asan" if asan else "", "two_way_driver")
    assert os.path.exists(exe), f"{exe} is missing: run make -C tests/native"
    env = dict(os.environ)
    if asan:
        env.update(ASAN_OPTIONS="protect_shadow_gap=0:detect_leaks=0:verify_asan_link_order=0",
                   FKV_LANE_STREAMS="1")
    r = subprocess.run([exe, "0.4", "64"], capture_output=True, text=True, timeout=120, env=env)
    assert r.returncode == 0 and r.stdout.startswith("ok:"), r.stdout + r.stderr
    assert "AddressSanitizer" not in r.stderr
    import re
    nums = [float(x) for x in re.findall(r"([0-9.]+) GB/s", r.stdout)]
    assert len(nums) == 3 and nums[2] > 1.2 * max(nums[0], nums[1]), r.stdout


def test_link_gap_probe_runs(gpu_device):
    """tests/native/link_gap_probe.hip, the stand-alone measurement behind the XCD
    split and the event flags: it has to build and run; its figures are for reading."""
    exe = os.path.join(BUILD, "link_gap_probe")
    assert os.path.exists(exe), f"{exe} is missing: run make -C tests/native"
    r = subprocess.run([exe, "--between", "event-nofence"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0 and "mean gap" in r.stdout, r.stdout + r.stderr
