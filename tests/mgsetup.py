"""Multi-group + sliding-window fixtures shared by the oracle and the GPU tests.

Geometry, block ids and byte seeds are those of the reference's own
known-answer tests (tests/test_layerwise_multi_group_swa.py:24-37, 188-236;
tests/test_layerwise_dsv4_multi_group_swa_roundtrip.py:85-131, 143-181), so an
expected byte never depends on the code under test.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from flexkv_amd.layout import (KVCacheLayout, KVCacheLayoutType, LayerGroupSpec,
                               MultiGroupBlockLayout, TransferStrides, multi_group_tables)

NUM_GPU_BLOCKS = 8
NUM_CPU_BLOCKS = 8
TOKENS_PER_BLOCK = 16
MAIN_HEAD_SIZE = 32
INDEXER_HEAD_SIZE = 16
SWA_BYTES_PER_TOKEN = 64
CPU_SRC, GPU_DST = 2, 5
SWA_CPU_SRC, SWA_GPU_DST = 3, 6


def gpu_layout_of(g: LayerGroupSpec, num_blocks: int, tpb: int) -> KVCacheLayout:
    """test_layerwise_multi_group_swa.py:65-76"""
    return KVCacheLayout(KVCacheLayoutType.LAYERFIRST, g.num_layers, num_blocks,
                         tpb // g.compress_ratio, g.num_kv_heads, g.head_size,
                         kv_dim=1 if g.num_kv_heads == 1 else 2, num_kv_heads=g.num_kv_heads)


def swa_layout_of(num_layers: int, num_blocks: int, tpb: int, width: int) -> KVCacheLayout:
    """test_layerwise_multi_group_swa.py:99-109"""
    return KVCacheLayout(KVCacheLayoutType.LAYERFIRST, num_layers, num_blocks, tpb, 1, width,
                         kv_dim=1, num_kv_heads=1)


def main_seed(orig: int, gi: int, local: int, tpb_g: int, heads: int, width: int,
              mul=(100, 10, 3)) -> np.ndarray:
    """Bytes of one (group member, block): ((orig*100 + gi*10 + local*3 + tok) ^ b) & 0xFF
    at [tok, head, b] (test_layerwise_multi_group_swa.py:214-224); the DSv4 round
    trip uses the multipliers (97, 13, 7)."""
    tok = np.arange(tpb_g)[:, None, None]
    b = np.arange(width)[None, None, :]
    v = ((orig * mul[0] + gi * mul[1] + local * mul[2] + tok) ^ b) & 0xFF
    return np.broadcast_to(v, (tpb_g, heads, width)).astype(np.uint8)


def swa_seed(orig: int, tpb: int, width: int, salt: int = 0xB2) -> np.ndarray:
    """((orig*31 + tok + salt) ^ b) & 0xFF at [tok, 0, b]
    (test_layerwise_multi_group_swa.py:227-236; salt 0xD4 in the DSv4 round trip)."""
    tok = np.arange(tpb)[:, None, None]
    b = np.arange(width)[None, None, :]
    return (((orig * 31 + tok + salt) ^ b) & 0xFF).astype(np.uint8)


@dataclass
class MGCase:
    """Host-memory model of a multi-group pool with a uniform SWA sidecar."""
    layer_groups: List[LayerGroupSpec]
    num_original_layers: int
    tpb: int = TOKENS_PER_BLOCK
    num_gpu_blocks: int = NUM_GPU_BLOCKS
    num_cpu_blocks: int = NUM_CPU_BLOCKS
    swa_width: int = SWA_BYTES_PER_TOKEN
    tables: Dict[str, object] = field(init=False)

    def __post_init__(self) -> None:
        self.cpu_layout = MultiGroupBlockLayout(self.num_cpu_blocks, self.tpb,
                                                tuple(self.layer_groups), kv_dim=1)
        self.gpu_layouts = [gpu_layout_of(g, self.num_gpu_blocks, self.tpb)
                            for g in self.layer_groups]
        self.tables = multi_group_tables(self.cpu_layout, self.num_original_layers,
                                         [[l] for l in self.gpu_layouts])
        self.block_stride = int(self.tables["cpu_block_stride"])
        self.host = np.zeros(self.num_cpu_blocks * self.block_stride, dtype=np.uint8)
        # one byte buffer per layer of every group, shaped [block, token, head, dim]
        self.gpu: List[List[np.ndarray]] = [
            [np.zeros((self.num_gpu_blocks, self.tpb // g.compress_ratio, g.num_kv_heads,
                       g.head_size * g.itemsize), dtype=np.uint8) for _ in range(g.num_layers)]
            for g in self.layer_groups]
        self.swa_cpu_layout = swa_layout_of(self.num_original_layers, self.num_cpu_blocks,
                                            self.tpb, self.swa_width)
        self.swa_gpu_layout = swa_layout_of(self.num_original_layers, self.num_gpu_blocks,
                                            self.tpb, self.swa_width)
        self.swa_host = np.zeros(self.swa_cpu_layout.kv_shape, dtype=np.uint8)
        self.swa_gpu = [np.zeros((self.num_gpu_blocks, self.tpb, 1, self.swa_width),
                                 dtype=np.uint8) for _ in range(self.num_original_layers)]
        self.swa_cpu_strides = TransferStrides.from_layout(self.swa_cpu_layout, 1)
        self.swa_gpu_strides = TransferStrides.from_layout(self.swa_gpu_layout, 1)

    @property
    def members(self) -> Sequence[Sequence[Tuple[int, int]]]:
        return self.tables["layer_members"]  # type: ignore[return-value]

    # ---- seeding of the host pools (known answers) ------------------------------
    def seed_main(self, cpu_block: int, orig: int, gi: int, local: int) -> np.ndarray:
        g = self.layer_groups[gi]
        exp = main_seed(orig, gi, local, self.tpb // g.compress_ratio, g.num_kv_heads,
                        g.head_size * g.itemsize)
        base = (cpu_block * self.block_stride + self.tables["group_cpu_offset_bytes"][gi]
                + local * self.tables["group_cpu_layer_strides"][gi])
        self.host[base:base + exp.size] = exp.reshape(-1)
        return exp

    def seed_all_main(self, cpu_block: int = CPU_SRC) -> Dict[Tuple[int, int, int], np.ndarray]:
        return {(orig, gi, local): self.seed_main(cpu_block, orig, gi, local)
                for orig in range(self.num_original_layers) for gi, local in self.members[orig]}

    def seed_all_swa(self, cpu_block: int = SWA_CPU_SRC) -> Dict[int, np.ndarray]:
        out = {}
        for orig in range(self.num_original_layers):
            exp = swa_seed(orig, self.tpb, self.swa_width)
            self.swa_host[orig, 0, cpu_block] = exp
            out[orig] = exp
        return out

    # ---- oracle view ---------------------------------------------------------------
    def oracle_groups(self):
        from oracle import fkv_oracle as O
        t = self.tables
        return [O.GroupRef(g.num_layers, [self.gpu[gi]], [t["group_gpu_kv_strides"][gi]],
                           [t["group_gpu_block_strides"][gi]], [t["group_gpu_layer_strides"][gi]],
                           [t["group_gpu_chunk_sizes"][gi]], t["group_cpu_offset_bytes"][gi],
                           t["group_h2d_cpu_kv_strides"][gi], t["group_h2d_cpu_layer_strides"][gi],
                           t["group_cpu_block_strides"][gi], t["group_cpu_tp_strides"][gi])
                for gi, g in enumerate(self.layer_groups)]

    def oracle_swa(self, cpu_ids, gpu_ids) -> dict:
        from oracle import fkv_oracle as O
        s = self.swa_gpu_strides
        grp = O.GroupRef(self.num_original_layers, [self.swa_gpu], [s.kv], [s.block], [s.layer],
                         [s.chunk])
        c = self.swa_cpu_strides
        return {"kind": "uniform", "group": grp, "host": self.swa_host.reshape(-1),
                "gpu_ids": list(gpu_ids), "cpu_ids": list(cpu_ids), "kv_stride": c.kv,
                "layer_stride": c.layer, "block_stride": c.block}

    # ---- device view ---------------------------------------------------------------
    def to_device(self, device: str = "cuda:0", eventfds=None, tp_size: int = 1,
                  has_swa: bool = True, ssd_files=None, swa_ssd_files=None,
                  iouring_entries: int = 512):
        """Builds the library's group over device copies of the (zeroed or seeded)
        buffers.  Returns a DeviceMG."""
        import torch
        from flexkv_amd.c_ext import LayerwiseTransferGroup
        host = torch.zeros(self.host.size, dtype=torch.uint8, pin_memory=True)
        host.copy_(torch.from_numpy(self.host))
        gpu = [[torch.from_numpy(a.copy()).to(device) for a in grp] for grp in self.gpu]
        swa_host = torch.zeros(self.swa_host.shape, dtype=torch.uint8, pin_memory=True)
        swa_host.copy_(torch.from_numpy(self.swa_host))
        swa_gpu = [torch.from_numpy(a.copy()).to(device) for a in self.swa_gpu]
        t = self.tables
        ctor = {k: t[k] for k in t if k.startswith("group_")}
        s = self.swa_gpu_strides
        swa_kw = {}
        if has_swa:
            swa_kw = dict(
                has_swa=True, swa_gpu_blocks=[swa_gpu], swa_cpu_blocks=swa_host,
                swa_ssd_files=swa_ssd_files or {},
                swa_gpu_kv_strides_tensor=torch.tensor([s.kv], dtype=torch.int64),
                swa_gpu_block_strides_tensor=torch.tensor([s.block], dtype=torch.int64),
                swa_gpu_layer_strides_tensor=torch.tensor([s.layer], dtype=torch.int64),
                swa_gpu_chunk_sizes_tensor=torch.tensor([s.chunk], dtype=torch.int64))
        group = LayerwiseTransferGroup(
            num_gpus=1, gpu_blocks_per_group=[[g] for g in gpu], cpu_blocks=host,
            ssd_files=ssd_files or {},
            num_original_layers=self.num_original_layers, layer_members=t["layer_members"],
            iouring_entries=iouring_entries, iouring_flags=0,
            layer_eventfds_tensor=(eventfds if eventfds is not None
                                   else torch.empty(0, dtype=torch.int32)),
            tp_size=tp_size, is_blockfirst=True, **ctor, **swa_kw)
        return DeviceMG(self, group, host, gpu, swa_host, swa_gpu)


class DeviceMG:
    def __init__(self, case: MGCase, group, host, gpu, swa_host, swa_gpu) -> None:
        self.case, self.group = case, group
        self.host, self.gpu, self.swa_host, self.swa_gpu = host, gpu, swa_host, swa_gpu

    def swa_call_kwargs(self, cpu_ids, gpu_ids) -> dict:
        import torch
        c = self.case.swa_cpu_strides
        empty = torch.empty(0, dtype=torch.int64)
        return dict(
            swa_h2d_src=torch.tensor(list(cpu_ids), dtype=torch.int64),
            swa_h2d_dst=torch.tensor(list(gpu_ids), dtype=torch.int64),
            swa_disk2h_src=empty, swa_disk2h_dst=empty,
            swa_cpu_kv_stride_in_bytes=c.kv, swa_cpu_layer_stride_in_bytes=c.layer,
            swa_cpu_block_stride_in_bytes=c.block, swa_cpu_chunk_size_in_bytes=c.chunk,
            swa_h2d_cpu_kv_stride_in_bytes=c.kv, swa_h2d_cpu_layer_stride_in_bytes=c.layer,
            swa_cpu_tp_stride_in_bytes=c.block, swa_ssd_layer_stride_in_bytes=0,
            swa_ssd_kv_stride_in_bytes=0, swa_num_blocks_per_file=0)

    def run_h2d(self, cpu_ids=(CPU_SRC,), gpu_ids=(GPU_DST,), swa: Optional[tuple] = None,
                use_ce_transfer=True, **kw) -> None:
        """The call of test_layerwise_multi_group_swa.py:409-457; ``swa`` is
        (host block ids, device block ids) or None."""
        import torch
        empty = torch.empty(0, dtype=torch.int64)
        extra = self.swa_call_kwargs(*swa) if swa is not None else {}
        self.group.layerwise_transfer_multi_group(
            empty, empty, num_blocks_per_file=0, round_robin=1, num_threads_per_device=4,
            gpu_block_id_tensor=torch.tensor(list(gpu_ids), dtype=torch.int64),
            cpu_block_id_tensor=torch.tensor(list(cpu_ids), dtype=torch.int64),
            transfer_cta_num=4, use_ce_transfer=use_ce_transfer, kv_dim=1, num_kv_heads=1,
            counter_id=kw.pop("counter_id", 0), **extra, **kw)
        if kw.get("notify_mode") == "polling":
            self.group.synchronize()
        torch.cuda.synchronize()

    def main_block(self, gi: int, local: int, block: int) -> np.ndarray:
        return self.gpu[gi][local][block].cpu().numpy()

    def swa_block(self, orig: int, block: int) -> np.ndarray:
        return self.swa_gpu[orig][block].cpu().numpy()
