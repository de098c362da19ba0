"""fkv_staging_transfer / fkv_build_gpu_chunk_ptrs on the GPU against the oracle:
variable-size payloads between a device staging buffer and a pinned host cache with a
host-side size table, and the table of chunk addresses."""
import numpy as np
import pytest
import torch

from kvsetup import KVSetup, SGLANG, TRTLLM, VLLM
from oracle import fkv_oracle as O

pytestmark = pytest.mark.gpu


def pinned(arr):
    t = torch.empty(arr.shape, dtype=torch.from_numpy(arr[:0].copy()).dtype, pin_memory=True)
    t.copy_(torch.from_numpy(arr))
    return t


class Case:
    """Host cache [layout], size table [N, L, kv], staging [bsz, stride] as numpy
    references and their device / pinned twins."""

    def __init__(self, device, rng, L, kv_dim, NB, N, cap, stride, layout, size_range, bsz_total):
        self.L, self.kv, self.NB, self.N, self.cap, self.stride = L, kv_dim, NB, N, cap, stride
        if layout == "BLOCKFIRST":
            self.strides = (cap, kv_dim * cap, L * kv_dim * cap)   # kv, layer, block
        else:
            self.strides = (N * cap, kv_dim * N * cap, cap)
        self.host_ref = rng.integers(0, 256, N * L * kv_dim * cap, dtype=np.uint8)
        self.table_ref = rng.integers(0, 7, N * L * kv_dim).astype(np.uint32)
        self.ids = rng.permutation(N)[:NB].astype(np.int64)
        self.staging_ref = rng.integers(0, 256, bsz_total * stride, dtype=np.uint8)
        lo, hi = size_range
        self.sizes_ref = rng.integers(lo, hi + 1, bsz_total).astype(np.uint64)
        self.host = pinned(self.host_ref)
        self.table = pinned(self.table_ref.view(np.int32))
        self.staging = torch.from_numpy(self.staging_ref.copy()).to(device)
        self.sizes = torch.from_numpy(self.sizes_ref.view(np.int64).copy()).to(device)
        self.overflow = torch.zeros(1, dtype=torch.int32, device=device)

    def run(self, start_layer, batch_start, bsz, write, slot0=0):
        from flexkv_amd.c_ext import staging_transfer
        ks, ls, bs = self.strides
        staging_transfer(self.staging[slot0 * self.stride:], self.stride, self.sizes[slot0:],
                         self.host, self.cap, self.overflow, ks, ls, bs,
                         torch.from_numpy(self.ids), self.table, self.L * self.kv, self.kv,
                         start_layer, self.kv, batch_start, bsz, write, sync=True)
        return O.staging_transfer(self.staging_ref[slot0 * self.stride:], self.stride,
                                  self.sizes_ref[slot0:], self.host_ref, self.cap, ks, ls, bs,
                                  self.ids, self.table_ref, self.L * self.kv, self.kv, start_layer,
                                  self.kv, self.NB, batch_start, bsz, write)

    def check(self, what):
        np.testing.assert_array_equal(self.host.numpy(), self.host_ref, err_msg=f"host cache {what}")
        np.testing.assert_array_equal(self.table.numpy().view(np.uint32), self.table_ref,
                                      err_msg=f"size table {what}")
        np.testing.assert_array_equal(self.staging.cpu().numpy(), self.staging_ref,
                                      err_msg=f"staging {what}")
        np.testing.assert_array_equal(self.sizes.cpu().numpy().view(np.uint64), self.sizes_ref,
                                      err_msg=f"sizes {what}")


@pytest.mark.parametrize("layout", ["BLOCKFIRST", "LAYERFIRST"])
@pytest.mark.parametrize("cap,stride,size_range", [
    (32768, 33280, (9000, 33000)),   # Llama-shaped chunk, some payloads do not fit
    (4608, 4608, (0, 4608)),         # everything fits, empty payloads included
    (1000, 1040, (1, 1040)),         # capacity no multiple of 16
    (73728, 73728, (50000, 73728)),
])
def test_write_then_read_matches_the_oracle(gpu_device, layout, cap, stride, size_range):
    rng = np.random.default_rng(cap + len(layout))
    L, kv_dim, NB, N, start_layer, nl = 6, 2, 23, 40, 1, 4
    total = nl * kv_dim * NB
    c = Case(gpu_device, rng, L, kv_dim, NB, N, cap, stride, layout, size_range, total)
    # three batches that start and end inside a layer
    over = 0
    for bs, n in ((0, 50), (50, 77), (127, total - 127)):
        over += c.run(start_layer, bs, n, True, slot0=bs)
    c.check("after the writes")
    assert int(c.overflow.item()) == over
    assert (over > 0) == (size_range[1] > cap)
    # read everything back into scrubbed staging: sizes come from the table
    c.staging.fill_(0xEE)
    c.staging_ref[:] = 0xEE
    c.sizes.zero_()
    c.sizes_ref[:] = 0
    for bs, n in ((0, 99), (99, total - 99)):
        c.run(start_layer, bs, n, False, slot0=bs)
    c.check("after the reads")


def test_unaligned_addresses_take_the_byte_path(gpu_device):
    """A staging stride and a host slot that are no multiples of 16."""
    rng = np.random.default_rng(4)
    c = Case(gpu_device, rng, 3, 1, 9, 12, 1001, 1003, "BLOCKFIRST", (0, 1001), 27)
    c.run(0, 0, 27, True)
    c.check("unaligned write")
    c.staging.fill_(1)
    c.staging_ref[:] = 1
    c.run(0, 0, 27, False)
    c.check("unaligned read")


def test_read_entry_beyond_the_staging_slot(gpu_device):
    rng = np.random.default_rng(6)
    c = Case(gpu_device, rng, 2, 1, 4, 4, 4096, 2048, "BLOCKFIRST", (0, 0), 8)
    c.table_ref[:] = [100, 2049, 2048, 5000, 0, 16, 17, 4096]
    c.table.copy_(torch.from_numpy(c.table_ref.view(np.int32)))
    over = c.run(0, 0, 8, False)
    c.check("entries beyond the slot")
    assert over == int(c.overflow.item()) == 3


def test_errors(gpu_device):
    from flexkv_amd.c_ext import staging_transfer
    rng = np.random.default_rng(8)
    c = Case(gpu_device, rng, 2, 1, 4, 4, 256, 256, "BLOCKFIRST", (0, 256), 8)
    ks, ls, bs = c.strides
    pageable = torch.zeros(c.host.numel(), dtype=torch.uint8)
    with pytest.raises(ValueError, match="device-visible"):
        staging_transfer(c.staging, 256, c.sizes, pageable, 256, c.overflow, ks, ls, bs,
                         torch.from_numpy(c.ids), c.table, 2, 1, 0, 1, 0, 8, True)
    with pytest.raises(ValueError, match="shorter|must hold bsz"):
        staging_transfer(c.staging, 256, c.sizes, c.host, 256, c.overflow, ks, ls, bs,
                         torch.from_numpy(c.ids), c.table, 2, 1, 0, 1, 0, 9, True)
    staging_transfer(c.staging, 256, c.sizes, c.host, 256, c.overflow, ks, ls, bs,
                     torch.from_numpy(c.ids), c.table, 2, 1, 0, 1, 3, 0, True)   # empty batch


@pytest.mark.parametrize("backend,gpu_layout", [(VLLM, "LAYERFIRST"), (VLLM, "LAYERBLOCK"),
                                                (TRTLLM, "LAYERFIRST"), (SGLANG, "LAYERFIRST")])
def test_chunk_ptrs_match_the_oracle_and_address_the_chunks(gpu_device, backend, gpu_layout):
    """The addresses equal the oracle's on the device tensors' own pointers, and
    reading 16 bytes at each of them gives the chunk the numbering names."""
    from flexkv_amd.c_ext import build_gpu_chunk_ptrs
    L, kv_dim, NG, NB, chunk = 5, 2, 31, 11, 512
    s = KVSetup(backend, L, kv_dim, NG, 4, chunk, "BLOCKFIRST", gpu_layout, seed=backend + 20)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(backend)
    ids = rng.permutation(NG)[:NB].astype(np.int64)
    start_layer, batch_start = 1, 7
    bsz = (L - start_layer) * kv_dim * NB - batch_start
    out = torch.zeros(bsz, dtype=torch.int64, device=gpu_device)
    build_gpu_chunk_ptrs(out, dev.ptrs, s.gpu_kv_stride, s.gpu_block_stride, s.gpu_layer_stride,
                         torch.from_numpy(ids), start_layer, kv_dim, batch_start, bsz, L,
                         gpu_block_type=backend, sync=True)
    dev_ptrs = [t.data_ptr() for t in dev.gpu]
    want = O.chunk_ptrs(backend, dev_ptrs, L, s.gpu_kv_stride, s.gpu_block_stride,
                        s.gpu_layer_stride, ids, start_layer, kv_dim, batch_start, bsz)
    got = out.cpu().numpy().view(np.uint64)
    np.testing.assert_array_equal(got, want)
    # the same numbering on the reference bytes: first 16 bytes of every chunk
    ref = O.chunk_ptrs(backend, s.ref_ptrs(), L, s.gpu_kv_stride, s.gpu_block_stride,
                       s.gpu_layer_stride, ids, start_layer, kv_dim, batch_start, bsz)
    import ctypes
    for i in (0, 1, bsz // 2, bsz - 1):
        off = None
        for t, base in zip(dev.gpu, dev_ptrs):
            if base <= int(got[i]) < base + t.numel():
                off = (t, int(got[i]) - base)
        assert off is not None
        dev_bytes = off[0][off[1]:off[1] + 16].cpu().numpy()
        ref_bytes = np.frombuffer((ctypes.c_uint8 * 16).from_address(int(ref[i])), dtype=np.uint8)
        np.testing.assert_array_equal(dev_bytes, ref_bytes)
