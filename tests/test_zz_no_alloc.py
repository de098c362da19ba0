"""fkv_transfer_kv_blocks_noalloc, the entry point that allocates nothing, against
fkv_transfer_kv_blocks on the same inputs: two calls in a row through the C ABI,
the second with a smaller input (the fixed device array then still holds the tail
of the first call's plan), both directions, and the oracle on top."""
import ctypes

import numpy as np
import pytest

from kvsetup import KVSetup, SGLANG, TRTLLM, VLLM

pytestmark = pytest.mark.gpu
NOALLOC = "fkv_transfer_kv_blocks_noalloc"


def both_ways(gpu_device, backend, kv_dim, layout, chunk, sizes, seed, sync=True):
    """The same transfers through the two entry points on two copies of the same
    bytes; host pools and device tensors must agree after every call."""
    import torch
    L, NG, NC = 5, 700, 640
    a = KVSetup(backend, L, kv_dim, NG, NC, chunk, layout, seed=seed)
    b = KVSetup(backend, L, kv_dim, NG, NC, chunk, layout, seed=seed)
    da, db = a.to_device(gpu_device), b.to_device(gpu_device)
    rng = np.random.default_rng(seed)
    st = torch.cuda.Stream()
    for k, n in enumerate(sizes):
        h2d = k % 2 == 1
        g, c = rng.permutation(NG)[:n], rng.permutation(NC)[:n]
        assert da.transfer_raw(g, c, h2d) == 0
        rc = db.transfer_raw(g, c, h2d, entry=NOALLOC, sync=sync, stream=st.cuda_stream)
        assert rc == 0, _error()
        if not sync:
            st.synchronize()
        a.oracle_transfer(g, c, h2d)
        np.testing.assert_array_equal(db.host_bytes(), da.host_bytes(), err_msg=f"host, call {k}")
        for i, (x, y) in enumerate(zip(db.gpu_bytes(), da.gpu_bytes())):
            np.testing.assert_array_equal(x, y, err_msg=f"GPU tensor {i}, call {k}")
        da.assert_matches_reference(f"call {k} ({n} blocks, h2d={h2d})")


def _error():
    from flexkv_amd import _lib
    return _lib.load().fkv_last_error().decode()


@pytest.mark.parametrize("backend,kv_dim,layout,chunk", [
    (VLLM, 2, "BLOCKFIRST", 32768), (TRTLLM, 2, "BLOCKFIRST", 4096), (SGLANG, 2, "LAYERFIRST", 1152),
    (VLLM, 1, "BLOCKFIRST", 73728)])
def test_two_calls_in_a_row_the_second_smaller(gpu_device, backend, kv_dim, layout, chunk):
    both_ways(gpu_device, backend, kv_dim, layout, chunk, sizes=[600, 600, 37, 37, 1, 1], seed=chunk)


def test_asynchronous_calls_on_one_stream(gpu_device):
    both_ways(gpu_device, VLLM, 2, "BLOCKFIRST", 8192, sizes=[300, 120, 64, 9], seed=5, sync=False)


def test_limits_are_reported(gpu_device):
    from flexkv_amd import _lib
    s = KVSetup(VLLM, 2, 2, 16, 16, 64, "BLOCKFIRST", seed=1)
    dev = s.to_device(gpu_device)
    ids = np.arange(8)
    assert dev.transfer_raw(ids, ids, False, entry=NOALLOC, use_ce=True) == _lib.FKV_ERR_UNSUPPORTED
    assert "kernel path only" in _error()
    many = np.zeros(70000, dtype=np.int64)   # 16 B per block: beyond the 1 MiB plan
    assert dev.transfer_raw(many, many, False, entry=NOALLOC) == _lib.FKV_ERR_INVALID_ARG
    assert "fixed scratch" in _error()
    # and the entry point still works afterwards
    assert dev.transfer_raw(ids, ids[::-1].copy(), False, entry=NOALLOC) == 0
    s.oracle_transfer(ids, ids[::-1].copy(), False)
    dev.assert_matches_reference("after the refused calls")


def test_first_library_call_of_a_process(gpu_device):
    """In a fresh process the entry point is the first thing the library does on
    the device: nothing has been probed or allocated by another entry point."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = (
        "import sys; sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + '/tests')\n"
        "import numpy as np\n"
        "from kvsetup import KVSetup\n"
        "s = KVSetup(0, 6, 2, 300, 300, 32768, 'BLOCKFIRST', seed=2)\n"
        "dev = s.to_device('cuda:0')\n"
        "rng = np.random.default_rng(1)\n"
        "for n, h2d in ((250, False), (250, True), (20, False), (20, True)):\n"
        "    g, c = rng.permutation(300)[:n], rng.permutation(300)[:n]\n"
        "    assert dev.transfer_raw(g, c, h2d, entry='fkv_transfer_kv_blocks_noalloc') == 0\n"
        "    s.oracle_transfer(g, c, h2d)\n"
        "    dev.assert_matches_reference(f'{n} blocks, h2d={h2d}')\n"
        "print('ok')\n")
    r = subprocess.run([sys.executable, "-c", script, root], capture_output=True, text=True,
                       timeout=110)
    assert r.returncode == 0 and r.stdout.split()[-1:] == ["ok"], r.stdout + r.stderr
