"""The committed golden vectors (tests/golden/*.npz, written by
tests/golden/make_vectors.py from the closed-form fixtures of the reference's own
tests): the oracle must reproduce them, and so must the HIP path."""
import os

import numpy as np
import pytest
import torch

from flexkv_amd.layout import LayerGroupSpec
from mgsetup import INDEXER_HEAD_SIZE, MAIN_HEAD_SIZE, MGCase
from oracle import fkv_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


# ---- tp1 fill pattern: a put of four blocks into a host pool --------------------------------

def _tp1(kind):
    g = load("tp1_fill_pattern.npz")
    L, KV, N, T, H, D, NH = (int(x) for x in g["shape"])
    chunk = T * H * D * 2
    gpu = [np.ascontiguousarray(g["gpu"][l]).view(np.uint8).reshape(-1) for l in range(L)]
    if kind == "blockfirst":
        want, cks, cls, cbs = g["host_blockfirst"], chunk, KV * chunk, L * KV * chunk
    else:
        want, cbs, cks, cls = g["host_layerfirst"], chunk, NH * chunk, KV * NH * chunk
    strides = dict(gks=N * chunk, gbs=chunk, gls=KV * N * chunk, cks=cks, cls=cls, cbs=cbs)
    return g, (L, KV, N, NH, chunk), gpu, want.view(np.uint8).reshape(-1), strides


@pytest.mark.parametrize("kind", ["blockfirst", "layerfirst"])
def test_oracle_reproduces_the_fill_pattern_image(kind):
    g, (L, KV, N, NH, chunk), gpu, want, s = _tp1(kind)
    host = np.zeros(want.size, dtype=np.uint8)
    O.transfer_c(O.BACKEND_VLLM, [a.ctypes.data for a in gpu], L, s["gks"], s["gbs"], s["gls"], 0,
                 host.ctypes.data, s["cks"], s["cls"], s["cbs"], 0, chunk, 0, L, KV,
                 g["gpu_ids"], g["cpu_ids"], False)
    assert np.array_equal(host, want)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["blockfirst", "layerfirst"])
@pytest.mark.parametrize("use_ce", [False, True], ids=["kernel", "ce"])
def test_device_reproduces_the_fill_pattern_image(gpu_device, kind, use_ce):
    from flexkv_amd.c_ext import transfer_kv_blocks
    g, (L, KV, N, NH, chunk), gpu, want, s = _tp1(kind)
    dev = [torch.from_numpy(a.copy()).to(gpu_device) for a in gpu]
    ptrs = torch.tensor([t.data_ptr() for t in dev], dtype=torch.int64)
    host = torch.zeros(want.size, dtype=torch.uint8, pin_memory=True)
    transfer_kv_blocks(torch.from_numpy(g["gpu_ids"]), ptrs, s["gks"], s["gbs"], s["gls"],
                       torch.from_numpy(g["cpu_ids"]), host, s["cks"], s["cls"], s["cbs"], chunk, 0,
                       L, is_host_to_device=False, kv_dim=KV, use_ce_transfer=use_ce,
                       ce_path_opt=True, is_blockfirst=kind == "blockfirst")
    assert np.array_equal(host.numpy(), want)
    # and back: erase the blocks on the device, restore them from the golden host image
    for t in dev:
        t.view(KV, N, chunk)[:, torch.from_numpy(g["gpu_ids"]).to(gpu_device)] = 0
    host.copy_(torch.from_numpy(want))
    transfer_kv_blocks(torch.from_numpy(g["gpu_ids"]), ptrs, s["gks"], s["gbs"], s["gls"],
                       torch.from_numpy(g["cpu_ids"]), host, s["cks"], s["cls"], s["cbs"], chunk, 0,
                       L, is_host_to_device=True, kv_dim=KV, use_ce_transfer=use_ce,
                       ce_path_opt=True, is_blockfirst=kind == "blockfirst")
    for l in range(L):
        assert np.array_equal(dev[l].cpu().numpy(), gpu[l]), l


# ---- multi-group restore with a sliding-window sidecar (case T6) ------------------------------

def _t6_case():
    main = LayerGroupSpec(4, 1, MAIN_HEAD_SIZE, (0, 1, 2, 3), itemsize=1)
    indexer = LayerGroupSpec(3, 1, INDEXER_HEAD_SIZE, (1, 2, 3), itemsize=1)
    return MGCase([main, indexer], 4)


def test_oracle_reproduces_the_multi_group_vectors():
    g = load("multi_group_t6.npz")
    cpu_src, gpu_dst, swa_src, swa_dst = (int(x) for x in g["ids"])
    case = _t6_case()
    assert case.block_stride == int(g["block_stride"][0])
    case.host[:] = g["host"]
    case.swa_host[:] = g["swa_host"]
    O.layerwise_multi_group(1, case.oracle_groups(), case.members, case.host, [gpu_dst],
                            [cpu_src], 1, 1, "sharded", case.oracle_swa([swa_src], [swa_dst]))
    for local in range(4):
        assert np.array_equal(case.gpu[0][local], g["gpu_main"][local]), local
    for local in range(3):
        assert np.array_equal(case.gpu[1][local], g["gpu_indexer"][local]), local
    for orig in range(4):
        assert np.array_equal(case.swa_gpu[orig], g["swa_gpu"][orig]), orig


@pytest.mark.gpu
@pytest.mark.parametrize("engine", [False, True], ids=["kernel", "ce"])
def test_device_reproduces_the_multi_group_vectors(gpu_device, engine):
    g = load("multi_group_t6.npz")
    cpu_src, gpu_dst, swa_src, swa_dst = (int(x) for x in g["ids"])
    case = _t6_case()
    case.host[:] = g["host"]
    case.swa_host[:] = g["swa_host"]
    dev = case.to_device(gpu_device)
    dev.run_h2d(cpu_ids=[cpu_src], gpu_ids=[gpu_dst], swa=([swa_src], [swa_dst]),
                use_ce_transfer=engine)
    for local in range(4):
        assert np.array_equal(dev.gpu[0][local].cpu().numpy(), g["gpu_main"][local]), local
    for local in range(3):
        assert np.array_equal(dev.gpu[1][local].cpu().numpy(), g["gpu_indexer"][local]), local
    for orig in range(4):
        assert np.array_equal(dev.swa_gpu[orig].cpu().numpy(), g["swa_gpu"][orig]), orig
    dev.group.close()
