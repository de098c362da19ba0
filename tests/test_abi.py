"""The C-ABI library loads without a GPU, exports every function the header
declares, and rejects bad descriptors with the reference's exception classes
before touching the device."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest
import torch

from flexkv_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fkv_transfer.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fkv_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    names = declared_functions()
    assert len(names) >= 25
    dyn = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True,
                         text=True, check=True).stdout
    exported = set(re.findall(r" T (fkv_\w+)", dyn))
    for n in names:
        assert n in exported, f"{n} declared in the header but not exported"
        assert hasattr(lib, n)
        assert n in _lib.SIGNATURES, f"{n} has no ctypes prototype"
    assert exported == set(names), "exports that the header does not declare"


def test_header_compiles_as_c_and_struct_sizes_match():
    src = r'''
#include "fkv_transfer.h"
#include <stdio.h>
int main(void){ printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(fkv_ce_config),
  sizeof(fkv_transfer_desc), sizeof(fkv_ce_analysis), sizeof(fkv_tp_rank_plan),
  sizeof(fkv_tp_group_params), sizeof(fkv_layerwise_params), sizeof(fkv_stats),
  sizeof(fkv_launch_policy), sizeof(fkv_staging_transfer_desc), sizeof(fkv_chunk_ptrs_desc));
  return 0; }
'''
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        open(c, "w").write(src)
        exe = os.path.join(d, "t")
        subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Werror", "-I",
                               os.path.join(ROOT, "include"), c, "-o", exe])
        sizes = list(map(int, subprocess.check_output([exe]).split()))
    want = [ctypes.sizeof(x) for x in (_lib.CEConfig, _lib.TransferDesc, _lib.CEAnalysis,
                                       _lib.TPRankPlan, _lib.TPGroupParams, _lib.LayerwiseParams,
                                       _lib.Stats, _lib.LaunchPolicy, _lib.StagingTransferDesc,
                                       _lib.ChunkPtrsDesc)]
    assert sizes == want


def test_defaults_of_ce_config():
    cfg = _lib.default_ce_config()   # csrc/ce_transfer.h:18-41
    assert (cfg.segment_threshold, cfg.path_opt_enabled, cfg.force_path, cfg.enable_memcpy2d,
            cfg.is_blockfirst, cfg.num_kv_heads, cfg.gather_threads, cfg.gather_nt) == \
        (8, 1, -1, 0, 0, 1, 4, 1)


def _call(**over):
    from flexkv_amd.c_ext import transfer_kv_blocks
    ids = torch.arange(2, dtype=torch.int64)
    args = dict(gpu_block_id_tensor=ids, gpu_tensor_ptrs_tensor=torch.zeros(4, dtype=torch.int64),
                gpu_kv_stride_in_bytes=64, gpu_block_stride_in_bytes=16,
                gpu_layer_stride_in_bytes=128, cpu_block_id_tensor=ids,
                cpu_tensor=torch.zeros(1024, dtype=torch.uint8), cpu_kv_stride_in_bytes=16,
                cpu_layer_stride_in_bytes=32, cpu_block_stride_in_bytes=128,
                chunk_size_in_bytes=16, start_layer_id=0, num_layers=4)
    args.update(over)
    transfer_kv_blocks(**args)


def test_bad_descriptors_are_rejected_on_the_host():
    with pytest.raises(RuntimeError, match="Unsupported gpu_block_type: 7"):  # bindings.cpp:91-94
        _call(gpu_block_type=7)
    with pytest.raises(ValueError, match="differ in length"):
        _call(cpu_block_id_tensor=torch.arange(3, dtype=torch.int64))
    with pytest.raises(TypeError):
        _call(gpu_block_id_tensor=torch.arange(2, dtype=torch.int32))
    with pytest.raises(ValueError, match="negative block id"):
        _call(gpu_block_id_tensor=torch.tensor([0, -1], dtype=torch.int64))
    with pytest.raises(ValueError, match="GPU tensor pointers"):
        _call(num_layers=5)                                   # vLLM needs 5 pointers, 4 given
    with pytest.raises(ValueError, match="GPU tensor pointers"):
        _call(gpu_block_type=2, num_layers=4, kv_dim=2)       # SGLang needs K and V tables
    with pytest.raises(ValueError, match="chunk_size_in_bytes"):
        _call(chunk_size_in_bytes=0)


def test_empty_transfer_is_a_no_op_without_a_gpu():
    empty = torch.empty(0, dtype=torch.int64)
    _call(gpu_block_id_tensor=empty, cpu_block_id_tensor=empty)   # no device call is made
    _call(num_layers=0)


def _multi(*overs):
    """transfer_kv_blocks_multi with one descriptor per dict of overrides."""
    from flexkv_amd.c_ext import transfer_kv_blocks_multi
    ids = torch.arange(2, dtype=torch.int64)
    calls = []
    for over in overs:
        kw = dict(gpu_block_id_tensor=ids, gpu_tensor_ptrs_tensor=torch.zeros(4, dtype=torch.int64),
                  gpu_kv_stride_in_bytes=64, gpu_block_stride_in_bytes=16,
                  gpu_layer_stride_in_bytes=128, cpu_block_id_tensor=ids,
                  cpu_tensor=torch.zeros(1024, dtype=torch.uint8), cpu_kv_stride_in_bytes=16,
                  cpu_layer_stride_in_bytes=32, cpu_block_stride_in_bytes=128,
                  chunk_size_in_bytes=16, start_layer_id=0, num_layers=4)
        kw.update(over)
        calls.append(((), kw))
    transfer_kv_blocks_multi(calls)


def test_multi_descriptor_call_checks_every_descriptor_on_the_host():
    empty = torch.empty(0, dtype=torch.int64)
    none = dict(gpu_block_id_tensor=empty, cpu_block_id_tensor=empty)
    _multi()                       # no descriptors, or only empty ones: no device call
    _multi(none, none, none)
    # a bad descriptor behind good ones is found before anything runs
    with pytest.raises(ValueError, match="chunk_size_in_bytes"):
        _multi(none, dict(none, chunk_size_in_bytes=0))
    with pytest.raises(RuntimeError, match="Unsupported gpu_block_type: 9"):
        _multi(none, none, dict(none, gpu_block_type=9))
    with pytest.raises(ValueError, match="differ in length"):
        _multi(none, dict(cpu_block_id_tensor=torch.arange(3, dtype=torch.int64)))
    with pytest.raises(ValueError, match="negative block id"):
        _multi(none, dict(gpu_block_id_tensor=torch.tensor([0, -1], dtype=torch.int64)))
    # the C entry point itself refuses a bad array
    lib = _lib.load()
    assert lib.fkv_transfer_kv_blocks_multi(None, 2, None) == _lib.FKV_ERR_INVALID_ARG
    assert b"descriptor array" in lib.fkv_last_error()
    assert lib.fkv_transfer_kv_blocks_multi(None, 0, None) == _lib.FKV_OK


def test_status_codes_map_to_exception_classes():
    lib = _lib.load()
    out = _lib.TPRankPlan()
    rc = lib.fkv_tp_rank_plan_compute(5, 4, 1, 0, b"sharded", 0, 0, 0, 1, 1, 64, 64, 16,
                                      ctypes.byref(out))
    assert rc == _lib.FKV_ERR_INVALID_ARG and "bad rank" in _lib.last_error()
    with pytest.raises(ValueError):
        _lib.check(rc)
    with pytest.raises(RuntimeError):
        _lib.check(_lib.FKV_ERR_RUNTIME)


def test_host_registration_chunking():
    """flexkv/transfer/host_buffer.py:57-98: chunk size from GiB with a 4 KiB
    margin rounded down to a page; pieces cover the buffer exactly once."""
    lib = _lib.load()
    from oracle import fkv_oracle as O
    for gb in (0, -1, 0.5, 1, 2.5, 0.001):
        assert lib.fkv_host_chunk_bytes_from_gb(gb) == O.lib().fkv_oracle_host_chunk_bytes(gb)
    assert lib.fkv_host_chunk_bytes_from_gb(1.0) == (1 << 30) - 4096
    assert lib.fkv_host_chunk_bytes_from_gb(0.0) == 0
    for total, chunk in ((10 << 20, 0), (10 << 20, 16 << 20), (10 << 20, 3 << 20), (4096, 4096),
                         ((3 << 20) * 4, 3 << 20), (1, 4096)):
        n = lib.fkv_host_register_plan(total, chunk, None, None, 0)
        off = np.zeros(n, dtype=np.uint64)
        sz = np.zeros(n, dtype=np.uint64)
        assert lib.fkv_host_register_plan(total, chunk, off.ctypes.data, sz.ctypes.data, n) == n
        want_off = list(range(0, total, chunk)) if chunk and total > chunk else [0]
        assert off.tolist() == want_off               # range(0, total, chunk) of the reference
        assert int(sz.sum()) == total and (sz > 0).all()
        assert all(int(o + s) == int(o2) for o, s, o2 in zip(off, sz, off[1:]))
        if chunk and total > chunk:
            assert (sz[:-1] == chunk).all() and sz[-1] <= chunk


def test_profiler_ranges_are_off_unless_asked_for():
    """fkv_range_push / fkv_range_pop forward to the ROCm marker library only with
    FKV_ROCTX=1 (read once per process, so each case runs in its own process)."""
    import subprocess
    import sys
    code = ("from flexkv_amd import _lib; L = _lib.load(); "
            "print(L.fkv_range_push(b'x'), L.fkv_range_pop())")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = {k: v for k, v in os.environ.items() if k != "FKV_ROCTX"}
    off = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True,
                         text=True, check=True).stdout.split()
    assert off == ["0", "0"]
    on = subprocess.run([sys.executable, "-c", code], cwd=root, env=dict(env, FKV_ROCTX="1"),
                        capture_output=True, text=True, check=True).stdout.split()
    assert on in (["1", "1"], ["0", "0"])       # 0 0 only where no marker library is installed


def test_link_activity_board_is_shared_between_processes():
    """The board on which processes post their link-bound launches: what one
    process posts, another one sees for that direction and GPU only, until it has
    ended `window_ms` ago; a process never sees its own postings, and the posting
    of a process that is gone is dropped."""
    import subprocess
    import sys
    key = f"abitest{os.getpid()}"
    env = dict(os.environ, FKV_LINK_BOARD_KEY=key)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    head = ("import ctypes, sys, time; sys.path.insert(0, sys.argv[1])\n"
            "from flexkv_amd import _lib\n"
            "L = _lib.load()\n"
            "b = ctypes.c_int32(7)\n"
            "def busy(dev, h2d, win):\n"
            "    assert L.fkv_link_activity_elsewhere(dev, h2d, win, ctypes.byref(b)) == 0\n"
            "    return b.value\n")
    poster = subprocess.Popen(
        [sys.executable, "-c", head +
         "assert L.fkv_link_activity_post(0, 1, 400000) == 0\n"      # host->GPU, 0.4 s
         "assert busy(0, 1, 20) == 0\n"                               # not its own
         "print('posted', flush=True); sys.stdin.readline()\n", root],
        env=env, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        assert poster.stdout.readline().strip() == "posted"
        probe = subprocess.run(
            [sys.executable, "-c", head +
             "print(busy(0, 1, 20), busy(0, 0, 20), busy(1, 1, 20))\n"
             "time.sleep(0.6)\n"
             "print(busy(0, 1, 20), busy(0, 1, 5000))\n"
             "print(L.fkv_link_activity_post(0, 0, -1) != 0)\n", root],
            env=env, capture_output=True, text=True, timeout=120)
        assert probe.returncode == 0, probe.stderr
        # busy host->GPU on device 0 only; over 20 ms after its 0.4 s, still within 5 s of
        # its end; a negative duration is refused
        assert probe.stdout.split("\n")[:3] == ["1 0 0", "0 1", "True"], probe.stdout
    finally:
        poster.stdin.write("\n")
        poster.stdin.close()
        assert poster.wait(30) == 0
    gone = subprocess.run([sys.executable, "-c", head + "print(busy(0, 1, 5000))\n", root],
                          env=env, capture_output=True, text=True, timeout=120)
    assert gone.stdout.strip() == "0", gone.stdout + gone.stderr   # its slot was taken over
    for dev in (0, 1):
        path = f"/dev/shm/fkv_link_{os.getuid()}_{key}_{dev}"
        if os.path.exists(path):
            os.unlink(path)
