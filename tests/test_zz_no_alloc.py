"""fkv_transfer_kv_blocks_noalloc, the entry point that allocates nothing, against
fkv_transfer_kv_blocks on the same inputs: two calls in a row through the C ABI,
the second with a smaller input (the fixed device array then still holds the tail
of the first call's plan), both directions, and the oracle on top; the call recorded
into a graph and replayed; calls on streams that are destroyed afterwards."""
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


def raw_call(dev, g, c, h2d, stream, sync):
    """The entry point with id arrays the caller owns (any torch or numpy memory)."""
    import torch
    from flexkv_amd import _lib
    s = dev.s
    ptrs = np.ascontiguousarray([t.data_ptr() for t in dev.gpu], dtype=np.uint64)
    d = _lib.TransferDesc()
    d.backend, d.num_layers_total = s.backend, s.num_layers_total
    d.gpu_tensor_ptrs, d.num_gpu_tensor_ptrs, d.device = ptrs.ctypes.data, ptrs.size, -1
    d.gpu_kv_stride, d.gpu_block_stride = s.gpu_kv_stride, s.gpu_block_stride
    d.gpu_layer_stride = s.gpu_layer_stride
    d.cpu_ptr = dev.host.data_ptr()
    d.cpu_kv_stride, d.cpu_layer_stride = s.cpu_kv_stride, s.cpu_layer_stride
    d.cpu_block_stride, d.chunk_size = s.cpu_block_stride, s.chunk
    d.start_layer_id, d.num_layers, d.kv_dim = 0, s.num_layers, s.kv_dim
    d.num_blocks = int(g.numel())
    d.gpu_block_ids, d.cpu_block_ids = g.data_ptr(), c.data_ptr()
    d.is_host_to_device, d.use_ce_transfer, d.transfer_num_cta, d.sync = int(h2d), 0, 4, int(sync)
    d.ce = _lib.default_ce_config()
    d.ce.is_blockfirst = int(s.cpu_layout == "BLOCKFIRST")
    return int(getattr(_lib.load(), NOALLOC)(ctypes.byref(d), stream))


@pytest.mark.parametrize("ids_where", ["pinned", "pageable", "device"])
def test_recorded_into_a_graph_and_replayed(gpu_device, ids_where):
    """The call enqueues kernel launches only, so a stream capture can record it.  The
    graph is replayed four times with eager work and synchronisations between the
    replays: fresh host bytes before every replay (a replay must move the bytes of its
    own time, not of the capture's), and, where the kernel reads the id lists in place
    (pinned or device memory), other block ids before the last two.  Every replay is
    held to the oracle."""
    import torch
    L, NG, NC, n, chunk = 4, 200, 160, 90, 8192
    s = KVSetup(VLLM, L, 2, NG, NC, chunk, "BLOCKFIRST", seed=77)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(3)
    gids, cids = rng.permutation(NG)[:n].astype(np.int64), rng.permutation(NC)[:n].astype(np.int64)
    make = {"pinned": lambda a: torch.from_numpy(a.copy()).pin_memory(),
            "pageable": lambda a: torch.from_numpy(a.copy()),
            "device": lambda a: torch.from_numpy(a.copy()).to(gpu_device)}[ids_where]
    # id lists at an offset inside their allocation: the device view must follow
    room_g, room_c = make(np.concatenate([np.full(5, -1), gids])), make(np.concatenate([np.full(3, -1), cids]))
    g_t, c_t = room_g[5:], room_c[3:]
    st = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=st, capture_error_mode="relaxed"):
        rc = raw_call(dev, g_t, c_t, True, st.cuda_stream, sync=False)
    assert rc == 0, _error()
    dev.assert_matches_reference("recording moves nothing")
    for rep in range(4):
        fresh = rng.integers(0, 256, s.host_bytes, dtype=np.uint8)
        s.host_ref[:] = fresh
        dev.host.copy_(torch.from_numpy(fresh))
        if rep == 2 and ids_where != "pageable":   # read in place: the graph follows the lists
            gids, cids = rng.permutation(NG)[:n].astype(np.int64), rng.permutation(NC)[:n].astype(np.int64)
            g_t.copy_(torch.from_numpy(gids))
            c_t.copy_(torch.from_numpy(cids))
            torch.cuda.synchronize()
        elif rep == 2:                             # copied into the launches: changes do not reach it
            g_t.zero_()
            c_t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        s.oracle_transfer(gids, cids, True)
        dev.assert_matches_reference(f"replay {rep}, ids {ids_where}")
        # eager work of the same entry point between the replays (it shares the array)
        eg, ec = rng.permutation(NG)[:17], rng.permutation(NC)[:17]
        assert dev.transfer_raw(eg, ec, rep % 2 == 0, entry=NOALLOC, stream=st.cuda_stream) == 0
        s.oracle_transfer(eg, ec, rep % 2 == 0)
        dev.assert_matches_reference(f"eager call after replay {rep}")


def test_the_stream_of_an_earlier_call_may_be_gone(gpu_device):
    """The entry point keeps no stream handle: a call on a stream that the caller
    destroys afterwards leaves nothing behind that a later call would touch."""
    import torch
    hip = ctypes.CDLL("libamdhip64.so")
    s = KVSetup(VLLM, 3, 2, 64, 64, 4096, "BLOCKFIRST", seed=6)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(9)
    torch.cuda.synchronize()
    for rep in range(3):
        stream = ctypes.c_void_p()
        assert hip.hipStreamCreateWithFlags(ctypes.byref(stream), 1) == 0   # non-blocking
        g, c = rng.permutation(64)[:40], rng.permutation(64)[:40]
        assert dev.transfer_raw(g, c, rep % 2 == 1, entry=NOALLOC, sync=False, stream=stream.value) == 0
        assert hip.hipStreamSynchronize(stream) == 0
        assert hip.hipStreamDestroy(stream) == 0
        s.oracle_transfer(g, c, rep % 2 == 1)
        dev.assert_matches_reference(f"call {rep} on a stream of its own")


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
