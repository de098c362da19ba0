"""Shared scaffolding for the transfer tests: engine-shaped KV tensors, host
pools and the strides that describe them, as seeded bytes.

Everything is built on the CPU first (numpy), so the oracle can run on the very
same bytes; ``to_device()`` uploads a copy for the HIP path.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

VLLM, TRTLLM, SGLANG = 0, 1, 2


@dataclass
class KVSetup:
    backend: int
    num_layers: int
    kv_dim: int
    num_gpu_blocks: int
    num_cpu_blocks: int
    chunk: int                      # bytes of one (layer, k-or-v, block)
    cpu_layout: str = "BLOCKFIRST"  # or "LAYERFIRST"
    gpu_layout: str = "LAYERFIRST"  # vLLM only: "LAYERFIRST" [kv,N,chunk] or "LAYERBLOCK" [N,kv,chunk]
    seed: int = 0
    gpu_block_pad: int = 0          # extra bytes between GPU blocks (non-dense engine tensors)
    cpu_copies: int = 1             # host pool holds this many block regions (all_write mode)

    gpu_ref: List[np.ndarray] = field(default_factory=list, repr=False)
    host_ref: Optional[np.ndarray] = field(default=None, repr=False)

    def __post_init__(self) -> None:
        L, K, N, C = self.num_layers, self.kv_dim, self.num_gpu_blocks, self.chunk
        rng = np.random.default_rng(self.seed)
        bs = C + self.gpu_block_pad
        if self.backend == VLLM:
            if self.gpu_layout == "LAYERFIRST":       # per layer [kv, N, chunk]
                self.gpu_block_stride, self.gpu_kv_stride = bs, N * bs
            else:                                      # per layer [N, kv, chunk]
                self.gpu_kv_stride, self.gpu_block_stride = bs, K * bs
            self.gpu_layer_stride = K * N * bs
            sizes = [K * N * bs] * L
        elif self.backend == TRTLLM:                   # one tensor [N, L, kv, chunk]
            self.gpu_kv_stride = bs
            self.gpu_layer_stride = K * bs
            self.gpu_block_stride = L * K * bs
            sizes = [N * L * K * bs]
        elif self.backend == SGLANG:                   # K_0..K_{L-1}, V_0..V_{L-1}, each [N, chunk]
            self.gpu_block_stride = bs
            self.gpu_kv_stride = 0
            self.gpu_layer_stride = N * bs
            sizes = [N * bs] * (K * L)
        else:
            raise ValueError(self.backend)
        self.gpu_ref = [rng.integers(0, 256, size=s, dtype=np.uint8) for s in sizes]

        NH = self.num_cpu_blocks * self.cpu_copies
        if self.cpu_layout == "BLOCKFIRST":            # [NH, L, kv, chunk]
            self.cpu_kv_stride, self.cpu_layer_stride, self.cpu_block_stride = C, K * C, L * K * C
        elif self.cpu_layout == "LAYERFIRST":          # [L, kv, NH, chunk]
            self.cpu_block_stride, self.cpu_kv_stride, self.cpu_layer_stride = C, NH * C, K * NH * C
        else:
            raise ValueError(self.cpu_layout)
        self.host_bytes = NH * L * K * C
        self.host_ref = rng.integers(0, 256, size=self.host_bytes, dtype=np.uint8)

    # ---- oracle side -------------------------------------------------------
    @property
    def num_layers_total(self) -> int:
        return self.num_layers

    def ref_ptrs(self) -> List[int]:
        return [a.ctypes.data for a in self.gpu_ref]

    def oracle_transfer(self, gpu_ids, cpu_ids, is_h2d: bool, start_layer: int = 0,
                        num_layers: Optional[int] = None, gpu_off: int = 0, cpu_off: int = 0,
                        chunk: Optional[int] = None, use_index_form: bool = False) -> None:
        from oracle import fkv_oracle as O
        nl = self.num_layers - start_layer if num_layers is None else num_layers
        ch = self.chunk if chunk is None else chunk
        if use_index_form:
            O.transfer_index(self.backend, self.gpu_ref, self.num_layers_total,
                             self.gpu_kv_stride, self.gpu_block_stride, self.gpu_layer_stride,
                             gpu_off, self.host_ref, self.cpu_kv_stride, self.cpu_layer_stride,
                             self.cpu_block_stride, cpu_off, ch, start_layer, nl, self.kv_dim,
                             gpu_ids, cpu_ids, is_h2d)
        else:
            O.transfer_c(self.backend, self.ref_ptrs(), self.num_layers_total,
                         self.gpu_kv_stride, self.gpu_block_stride, self.gpu_layer_stride,
                         gpu_off, self.host_ref.ctypes.data, self.cpu_kv_stride,
                         self.cpu_layer_stride, self.cpu_block_stride, cpu_off, ch,
                         start_layer, nl, self.kv_dim, gpu_ids, cpu_ids, is_h2d)

    # ---- device side -------------------------------------------------------
    def to_device(self, device: str = "cuda:0"):
        """Upload copies of the current reference bytes; returns a DeviceSide."""
        import torch
        gpu = [torch.from_numpy(a.copy()).to(device) for a in self.gpu_ref]
        host = torch.empty(self.host_bytes, dtype=torch.uint8, pin_memory=True)
        host.copy_(torch.from_numpy(self.host_ref))
        ptrs = torch.tensor([t.data_ptr() for t in gpu], dtype=torch.int64).pin_memory()
        return DeviceSide(self, gpu, host, ptrs)


class DeviceSide:
    def __init__(self, setup: KVSetup, gpu, host, ptrs) -> None:
        self.s, self.gpu, self.host, self.ptrs = setup, gpu, host, ptrs

    def transfer(self, gpu_ids, cpu_ids, is_h2d: bool, start_layer: int = 0,
                 num_layers: Optional[int] = None, **kw) -> None:
        import torch
        from flexkv_amd.c_ext import transfer_kv_blocks
        s = self.s
        nl = s.num_layers - start_layer if num_layers is None else num_layers
        kw.setdefault("is_blockfirst", s.cpu_layout == "BLOCKFIRST")
        transfer_kv_blocks(
            torch.as_tensor(np.asarray(gpu_ids, dtype=np.int64)), self.ptrs,
            s.gpu_kv_stride, s.gpu_block_stride, s.gpu_layer_stride,
            torch.as_tensor(np.asarray(cpu_ids, dtype=np.int64)), self.host,
            s.cpu_kv_stride, s.cpu_layer_stride, s.cpu_block_stride, s.chunk,
            start_layer, nl, is_host_to_device=is_h2d, kv_dim=s.kv_dim,
            gpu_block_type=s.backend, **kw)

    def transfer_raw(self, gpu_ids, cpu_ids, is_h2d: bool, start_layer: int = 0,
                     num_layers: Optional[int] = None, gpu_off: int = 0, cpu_off: int = 0,
                     chunk: Optional[int] = None, use_ce: bool = False, num_cta: int = 4,
                     sync: bool = True, stream: int = 0, ce: Optional[dict] = None,
                     entry: str = "fkv_transfer_kv_blocks") -> int:
        """Straight through the C ABI (fkv_transfer_kv_blocks), including the
        in-chunk offsets the Python operator does not expose.  Returns the status."""
        import ctypes
        from flexkv_amd import _lib
        s = self.s
        L = _lib.load()
        g = np.ascontiguousarray(gpu_ids, dtype=np.int64)
        c = np.ascontiguousarray(cpu_ids, dtype=np.int64)
        ptrs = np.ascontiguousarray([t.data_ptr() for t in self.gpu], dtype=np.uint64)
        d = _lib.TransferDesc()
        d.backend, d.num_layers_total = s.backend, s.num_layers_total
        d.gpu_tensor_ptrs, d.num_gpu_tensor_ptrs, d.device = ptrs.ctypes.data, ptrs.size, -1
        d.gpu_kv_stride, d.gpu_block_stride = s.gpu_kv_stride, s.gpu_block_stride
        d.gpu_layer_stride, d.gpu_startoff_inside_chunks = s.gpu_layer_stride, gpu_off
        d.cpu_ptr = self.host.data_ptr()
        d.cpu_kv_stride, d.cpu_layer_stride = s.cpu_kv_stride, s.cpu_layer_stride
        d.cpu_block_stride, d.cpu_startoff_inside_chunks = s.cpu_block_stride, cpu_off
        d.chunk_size = s.chunk if chunk is None else chunk
        d.start_layer_id = start_layer
        d.num_layers = s.num_layers - start_layer if num_layers is None else num_layers
        d.kv_dim, d.num_blocks = s.kv_dim, g.size
        d.gpu_block_ids, d.cpu_block_ids = g.ctypes.data, c.ctypes.data
        d.is_host_to_device, d.use_ce_transfer = int(is_h2d), int(use_ce)
        d.transfer_num_cta, d.sync = num_cta, int(sync)
        d.ce = _lib.default_ce_config()
        d.ce.is_blockfirst = int(s.cpu_layout == "BLOCKFIRST")
        for k, v in (ce or {}).items():
            setattr(d.ce, k, v)
        return int(getattr(L, entry)(ctypes.byref(d), stream))

    def gpu_bytes(self) -> List[np.ndarray]:
        return [t.cpu().numpy() for t in self.gpu]

    def host_bytes(self) -> np.ndarray:
        return self.host.numpy()

    def assert_matches_reference(self, what: str = "") -> None:
        """Device tensors and pinned host pool equal the oracle's, byte for byte."""
        s = self.s
        np.testing.assert_array_equal(self.host_bytes(), s.host_ref,
                                      err_msg=f"host pool differs {what}")
        for i, (got, want) in enumerate(zip(self.gpu_bytes(), s.gpu_ref)):
            np.testing.assert_array_equal(got, want, err_msg=f"GPU tensor {i} differs {what}")


def block_ids(rng: np.random.Generator, pool: int, n: int, pattern: str = "scattered"):
    """n distinct ids out of range(pool): 'contiguous', 'few_seg' (quarters in
    the order 0,2,1,3) or 'scattered' (random permutation prefix)."""
    if pattern == "contiguous":
        start = int(rng.integers(0, pool - n + 1))
        return np.arange(start, start + n, dtype=np.int64)
    if pattern == "few_seg":
        start = int(rng.integers(0, pool - n + 1))
        base = np.arange(start, start + n, dtype=np.int64)
        q = n // 4
        return np.concatenate([base[0:q], base[2 * q:3 * q], base[q:2 * q], base[3 * q:]])
    return rng.permutation(pool)[:n].astype(np.int64)
