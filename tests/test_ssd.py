"""Host pool <-> SSD files: block placement, the oracle against the reference's own
fixture, the library against the oracle (file images and read-back), request
coalescing, both I/O engines, error behaviour.  No GPU involved."""
import ctypes
import os

import numpy as np
import pytest
import torch

from flexkv_amd import _lib
from flexkv_amd.c_ext import SSDIOCTX, transfer_kv_blocks_ssd
from flexkv_amd.layout import KVCacheLayout, KVCacheLayoutType, TransferStrides

L = _lib.load()
ES = 2  # bytes per element of the reference's fixture dtype (fp16)


def lib_locate(ssd_id, rr, ndev, nfiles):
    d, f, b = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int64()
    assert L.fkv_ssd_locate(ssd_id, rr, ndev, nfiles, ctypes.byref(d), ctypes.byref(f),
                            ctypes.byref(b)) == 0
    return d.value, f.value, b.value


# ---- where a block id lives -------------------------------------------------------

@pytest.mark.parametrize("rr,ndev,nfiles", [(1, 1, 1), (1, 2, 3), (4, 3, 2), (8, 2, 1), (3, 4, 4)])
def test_locate_closed_forms_and_bijection(rr, ndev, nfiles):
    from oracle import fkv_oracle as O
    n = rr * ndev * nfiles * 7
    seen = set()
    for i in range(n):
        got = lib_locate(i, rr, ndev, nfiles)
        assert got == O.ssd_locate(i, rr, ndev, nfiles)
        # the reference's own second statement of the mapping,
        # flexkv/transfer/nixlutil.py:351-385
        in_dev = (i // rr) // ndev * rr + i % rr
        assert got == ((i // rr) % ndev, in_dev % nfiles, in_dev // nfiles)
        seen.add(got)
    # n ids fill a dense grid: every (device, file) holds blocks 0 .. n/(ndev*nfiles)-1
    per_file = n // (ndev * nfiles)
    assert seen == {(d, f, b) for d in range(ndev) for f in range(nfiles) for b in range(per_file)}
    # stripes of `rr` consecutive ids stay on one device, the next stripe on the next
    assert all(lib_locate(i, rr, ndev, nfiles)[0] == (i // rr) % ndev for i in range(n))


# ---- fixtures ----------------------------------------------------------------------------

class SsdCase:
    """Host pool of a given layout, files with the per-file layout the reference's
    workers derive (same kind, block axis divided over the files with padding,
    flexkv/transfer/worker.py:1576-1584)."""

    def __init__(self, tmp_path, kind, layers, blocks, tpb, heads, dim, kv_dim, ndev=1, nfiles=1,
                 rr=1, ssd_blocks=None, fill="arange"):
        self.layout = KVCacheLayout(KVCacheLayoutType[kind], layers, blocks, tpb, heads, dim,
                                    kv_dim=kv_dim, num_kv_heads=heads)
        self.kv_dim, self.layers, self.ndev, self.nfiles, self.rr = kv_dim, layers, ndev, nfiles, rr
        self.ssd_blocks = ssd_blocks or blocks
        total_files = ndev * nfiles
        ssd_layout = KVCacheLayout(KVCacheLayoutType[kind], layers, self.ssd_blocks, tpb, heads,
                                   dim, kv_dim=kv_dim, num_kv_heads=heads)
        self.file_layout = ssd_layout.div_block(total_files, padding=True)
        self.c = TransferStrides.from_layout(self.layout, ES)
        self.s = TransferStrides.from_layout(self.file_layout, ES)
        n = self.layout.get_total_elements()
        if fill == "arange":  # tests/test_kv_transfer_correctness.py:1999-2004
            vals = (np.arange(n, dtype=np.int64) % 9973).astype(np.float16)
        else:
            vals = np.random.default_rng(3).integers(0, 65536, n, dtype=np.uint16).view(np.float16)
        self.host = vals.view(np.uint8).copy()
        self.file_bytes = self.file_layout.get_total_elements() * ES
        self.paths = {}
        for d in range(ndev):
            os.makedirs(tmp_path / f"dev{d}", exist_ok=True)
            self.paths[d] = []
            for f in range(nfiles):
                p = str(tmp_path / f"dev{d}" / f"ssd_cache_{d}_{f}.bin")
                with open(p, "wb") as fh:
                    fh.truncate(self.file_bytes)
                self.paths[d].append(p)
        self.ref_files = [np.zeros(self.file_bytes, dtype=np.uint8) for _ in range(total_files)]

    def file_images(self):
        return [np.fromfile(p, dtype=np.uint8) for d in range(self.ndev) for p in self.paths[d]]

    def run(self, ctx, ssd_ids, cpu_ids, is_read, host=None, start_layer=0, num_layers=None,
            threads=4, opt=True):
        host = self.host if host is None else host
        nl = self.layers - start_layer if num_layers is None else num_layers
        transfer_kv_blocks_ssd(
            ctx, torch.arange(start_layer, start_layer + nl, dtype=torch.int32), host.ctypes.data,
            torch.as_tensor(np.asarray(ssd_ids, dtype=np.int64)),
            torch.as_tensor(np.asarray(cpu_ids, dtype=np.int64)), self.c.layer, self.c.kv,
            self.s.layer, self.s.kv, self.c.chunk, self.c.block, is_read, self.ssd_blocks,
            round_robin=self.rr, num_threads_per_device=threads, kv_dim=self.kv_dim,
            ssd_io_opt=opt)

    def oracle(self, ssd_ids, cpu_ids, is_read, host=None, start_layer=0, num_layers=None):
        from oracle import fkv_oracle as O
        host = self.host if host is None else host
        nl = self.layers - start_layer if num_layers is None else num_layers
        O.ssd_transfer(self.ref_files, self.ndev, self.nfiles, start_layer, nl, host, ssd_ids,
                       cpu_ids, self.c.layer, self.c.kv, self.s.layer, self.s.kv, self.c.chunk,
                       self.c.block, is_read, self.rr, self.kv_dim)


SIZES = [pytest.param((4, 8, 16, 1, 512), id="mla-mini"),
         pytest.param((16, 16, 16, 1, 512), id="mla-multi-layer"),
         pytest.param((4, 8, 16, 8, 128), id="mha-mini"),
         pytest.param((2, 4, 1, 8, 128), id="mha-edge")]
ENGINES = [pytest.param(0, id="threads"), pytest.param(64, id="iouring")]


# ---- the oracle against the reference's fixture -------------------------------------------------

@pytest.mark.parametrize("size", SIZES)
@pytest.mark.parametrize("kv_dim", [1, 2])
@pytest.mark.parametrize("kind", ["LAYERFIRST", "BLOCKFIRST"])
def test_oracle_file_image_equals_pool_image(tmp_path, size, kv_dim, kind):
    """tests/test_kv_transfer_correctness.py:2022-2131: one file with the pool's own
    layout and identity ids — the file must become a byte copy of the pool, and
    reading it back must restore the pool."""
    case = SsdCase(tmp_path, kind, *size, kv_dim)
    ids = np.arange(size[1])
    case.oracle(ids, ids, False)
    assert np.array_equal(case.ref_files[0], case.host)
    back = np.zeros_like(case.host)
    case.oracle(ids, ids, True, host=back)
    assert np.array_equal(back, case.host)
    # block 3 of the pool into block 1 of the file: only that block's chunks change
    case2 = SsdCase(tmp_path / "b", kind, *size, kv_dim)
    case2.oracle([1], [3], False)
    shape = case2.layout.kv_shape
    pool = case2.host.view(np.float16).reshape(shape)
    img = case2.ref_files[0].view(np.float16).reshape(shape)
    blk_axis = 2 if kind == "LAYERFIRST" else 0
    assert np.array_equal(np.take(img, 1, axis=blk_axis), np.take(pool, 3, axis=blk_axis))
    assert not np.delete(img, 1, axis=blk_axis).any()


# ---- the library against the oracle ----------------------------------------------------------------

@pytest.mark.parametrize("size", SIZES)
@pytest.mark.parametrize("kv_dim", [1, 2])
@pytest.mark.parametrize("kind", ["LAYERFIRST", "BLOCKFIRST"])
@pytest.mark.parametrize("entries", ENGINES)
@pytest.mark.parametrize("opt", [False, True], ids=["baseline", "optimized"])
def test_round_trip_like_the_reference(tmp_path, size, kv_dim, kind, entries, opt):
    case = SsdCase(tmp_path, kind, *size, kv_dim)
    ctx = SSDIOCTX(case.paths, 1, entries, 0)
    ids = np.arange(size[1])
    for threads in (1, 4):
        case.run(ctx, ids, ids, False, threads=threads, opt=opt)
        assert np.array_equal(case.file_images()[0], case.host)  # same layout: a byte copy
        back = np.zeros_like(case.host)
        case.run(ctx, ids, ids, True, host=back, threads=threads, opt=opt)
        assert np.array_equal(back, case.host)
    ctx.close()


@pytest.mark.parametrize("kind", ["LAYERFIRST", "BLOCKFIRST"])
@pytest.mark.parametrize("kv_dim", [1, 2])
@pytest.mark.parametrize("entries", ENGINES)
@pytest.mark.parametrize("opt", [False, True], ids=["baseline", "optimized"])
def test_partial_blocks_like_the_reference(tmp_path, kind, kv_dim, entries, opt):
    """tests/test_kv_transfer_correctness.py:2139-2262: write blocks [0,2,4,6], zero
    them in the pool, read them back into [1,3,5,7]; the odd blocks then hold what
    the even ones held, everything else is as the zeroing left it."""
    layers, blocks, tpb, heads, dim = 4, 8, 16, 8, 128
    case = SsdCase(tmp_path, kind, layers, blocks, tpb, heads, dim, kv_dim)
    shape = tuple(case.layout.kv_shape)
    orig = case.host.view(np.float16).reshape(shape).copy()
    pool = case.host.view(np.float16).reshape(shape)
    ctx = SSDIOCTX(case.paths, 1, entries, 0)
    even, odd = [0, 2, 4, 6], [1, 3, 5, 7]
    case.run(ctx, even, even, False, opt=opt)
    if kind == "LAYERFIRST":
        pool[:, :, even] = 0
    else:
        pool[even] = 0
    case.run(ctx, even, odd, True, opt=opt)
    for src, dst in zip(even, odd):
        if kind == "LAYERFIRST":
            assert np.array_equal(pool[:, :, dst], orig[:, :, src])
            assert not pool[:, :, src].any()
        else:
            assert np.array_equal(pool[dst], orig[src])
            assert not pool[src].any()
    ctx.close()


@pytest.mark.parametrize("kind", ["LAYERFIRST", "BLOCKFIRST"])
@pytest.mark.parametrize("kv_dim", [1, 2])
@pytest.mark.parametrize("ndev,nfiles,rr", [(1, 1, 1), (2, 2, 1), (3, 2, 4), (1, 3, 2)])
@pytest.mark.parametrize("entries", ENGINES)
def test_striped_files_match_the_oracle(tmp_path, kind, kv_dim, ndev, nfiles, rr, entries):
    """Random ids over several devices and files, both optimisation modes: the file
    images and the pool after reading back must equal the oracle's byte for byte."""
    blocks, ssd_blocks = 24, 48
    rng = np.random.default_rng(ndev * 10 + nfiles)
    for opt in (True, False):
        sub = tmp_path / f"opt{int(opt)}"
        os.makedirs(sub)
        case = SsdCase(sub, kind, 5, blocks, 8, 2, 64, kv_dim, ndev, nfiles, rr, ssd_blocks,
                       fill="random")
        ctx = SSDIOCTX(case.paths, ndev, entries, 0)
        assert ctx.uses_iouring == (entries > 0)
        ssd_ids = rng.permutation(ssd_blocks)[:17]
        cpu_ids = rng.permutation(blocks)[:17]
        case.run(ctx, ssd_ids, cpu_ids, False, opt=opt)
        case.oracle(ssd_ids, cpu_ids, False)
        for got, want in zip(case.file_images(), case.ref_files):
            assert np.array_equal(got, want)
        # a layer range in the middle, other blocks: read into a scratch pool
        ssd2, cpu2 = ssd_ids[:9], rng.permutation(blocks)[:9]
        got_pool, want_pool = np.zeros_like(case.host), np.zeros_like(case.host)
        case.run(ctx, ssd2, cpu2, True, host=got_pool, start_layer=1, num_layers=3, opt=opt)
        case.oracle(ssd2, cpu2, True, host=want_pool, start_layer=1, num_layers=3)
        assert np.array_equal(got_pool, want_pool) and want_pool.any()
        ctx.close()


def test_modes_and_engines_write_identical_files(tmp_path):
    """tests/test_kv_transfer_correctness.py:2291-2340: optimisation on/off (and here
    also threads / io_uring) must leave byte-identical files."""
    images = []
    for k, (entries, opt) in enumerate([(0, False), (0, True), (32, False), (32, True)]):
        sub = tmp_path / str(k)
        os.makedirs(sub)
        case = SsdCase(sub, "LAYERFIRST", 6, 16, 16, 4, 64, 2, 1, 2, 1, 32, fill="random")
        ctx = SSDIOCTX(case.paths, 1, entries, 0)
        case.run(ctx, [0, 1, 2, 3, 10, 12, 14, 31, 30], [5, 6, 7, 8, 0, 1, 2, 3, 4], False, opt=opt)
        images.append(np.concatenate(case.file_images()))
        ctx.close()
    assert all(np.array_equal(images[0], im) for im in images[1:]) and images[0].any()


def test_multi_group_blocks_move_as_opaque_blobs(tmp_path):
    """flexkv/transfer/worker.py:1637-1668: one 'layer' whose stride and chunk are
    the whole block, kv_dim 1 — block sizes that are not a multiple of anything."""
    block_bytes, blocks = 3 * 1152 + 40, 12
    rng = np.random.default_rng(5)
    host = rng.integers(0, 256, blocks * block_bytes, dtype=np.uint8)
    p = str(tmp_path / "mg.bin")
    with open(p, "wb") as fh:
        fh.truncate(20 * block_bytes)
    for entries in (0, 16):
        ctx = SSDIOCTX({0: [p]}, 1, entries, 0)
        ssd_ids, cpu_ids = torch.tensor([4, 5, 6, 19, 0]), torch.tensor([11, 3, 4, 5, 0])
        one = torch.tensor([0], dtype=torch.int32)
        transfer_kv_blocks_ssd(ctx, one, host.ctypes.data, ssd_ids, cpu_ids, block_bytes, 0,
                               block_bytes, 0, block_bytes, block_bytes, False, 20, 1, 32, 1)
        img = np.fromfile(p, dtype=np.uint8).reshape(20, block_bytes)
        pool = host.reshape(blocks, block_bytes)
        assert np.array_equal(img[ssd_ids.numpy()], pool[cpu_ids.numpy()])
        back = np.zeros_like(host)
        transfer_kv_blocks_ssd(ctx, one, back.ctypes.data, ssd_ids, cpu_ids, block_bytes, 0,
                               block_bytes, 0, block_bytes, block_bytes, True, 20, 1, 32, 1)
        assert np.array_equal(back.reshape(blocks, block_bytes)[cpu_ids.numpy()],
                              pool[cpu_ids.numpy()])
        ctx.close()


def test_direct_io_when_everything_is_page_aligned(tmp_path):
    """4 KiB-aligned chunk, strides and base: the O_DIRECT descriptors are used where
    the file system has them; the bytes are the same either way."""
    kind, layers, blocks, tpb, heads, dim = "BLOCKFIRST", 3, 8, 16, 2, 64  # chunk 4096 B
    case = SsdCase(tmp_path, kind, layers, blocks, tpb, heads, dim, 2, fill="random")
    assert case.c.chunk == 4096
    buf = np.zeros(case.host.size + 4096, dtype=np.uint8)
    off = (-buf.ctypes.data) % 4096
    pool = buf[off:off + case.host.size]
    pool[:] = case.host
    for entries in (0, 16):
        ctx = SSDIOCTX(case.paths, 1, entries, 0)
        ids = np.arange(blocks)
        case.run(ctx, ids[::-1].copy(), ids, False, host=pool)
        case.oracle(ids[::-1].copy(), ids, False)
        assert np.array_equal(case.file_images()[0], case.ref_files[0])
        back = np.zeros(case.host.size + 4096, dtype=np.uint8)[off:off + case.host.size]
        case.run(ctx, ids[::-1].copy(), ids, True, host=back)
        assert np.array_equal(back, case.host)
        ctx.close()


# ---- what the requests look like -------------------------------------------------------------------

def plan(case, ssd_ids, cpu_ids, opt=True, start_layer=0, num_layers=None):
    s = np.ascontiguousarray(ssd_ids, dtype=np.int64)
    c = np.ascontiguousarray(cpu_ids, dtype=np.int64)
    nl = case.layers - start_layer if num_layers is None else num_layers
    args = (case.ndev, case.nfiles, start_layer, nl, s.ctypes.data, c.ctypes.data, s.size,
            case.c.layer, case.c.kv, case.s.layer, case.s.kv, case.c.chunk, case.c.block, case.rr,
            case.kv_dim, int(opt))
    rows = L.fkv_ssd_plan(*args, None, 0)
    out = np.zeros((max(rows, 1), 5), dtype=np.int64)
    assert L.fkv_ssd_plan(*args, out.ctypes.data, rows) == rows
    return out[:rows]


def covered(rows):
    """(file id, file offset, host offset, length) per iovec, from the plan rows."""
    out, pos = [], {}
    for req, fd, foff, hoff, ln in rows.tolist():
        at = pos.get(req, foff)
        out.append((fd, at, hoff, ln))
        pos[req] = at + ln
    return out


def test_requests_are_coalesced(tmp_path):
    bf = SsdCase(tmp_path / "bf", "BLOCKFIRST", 4, 16, 16, 2, 64, 2)
    ids = np.arange(16)
    rows = plan(bf, ids, ids)
    assert len(rows) == 1 and rows[0, 4] == bf.host.size          # the whole pool in one extent
    rows = plan(bf, ids, ids[::-1].copy())                         # file in order, pool reversed
    assert len(set(rows[:, 0])) == 1 and len(rows) == 16 and set(rows[:, 4]) == {bf.c.block}
    rows = plan(bf, ids, ids, opt=False)                           # baseline: one chunk each
    assert len(rows) == 16 * 4 * 2 and set(rows[:, 4]) == {bf.c.chunk}
    assert len(set(rows[:, 0])) == len(rows)
    lf = SsdCase(tmp_path / "lf", "LAYERFIRST", 4, 16, 16, 2, 64, 2)
    rows = plan(lf, ids, ids)
    assert len(rows) == 1                                          # same layout, identity: all adjacent
    rows = plan(lf, ids[:8], ids[:8])                              # half the blocks: one run per (layer, kv)
    assert len(rows) == 8 and set(rows[:, 4]) == {8 * lf.c.chunk}
    rows = plan(lf, [0, 1, 2, 5, 6], [9, 10, 3, 4, 5])
    # per (layer, kv): file runs {0,1,2} and {5,6}; pool runs {9,10},{3} and {4,5}
    assert len(set(rows[:, 0])) == 16 and len(rows) == 24
    # whatever the grouping, the extents are exactly the oracle's chunks
    want = set()
    for b_ssd, b_cpu in zip([0, 1, 2, 5, 6], [9, 10, 3, 4, 5]):
        for l in range(4):
            for kv in range(2):
                want.add((0, b_ssd * lf.c.block + l * lf.s.layer + kv * lf.s.kv,
                          b_cpu * lf.c.block + l * lf.c.layer + kv * lf.c.kv))
    got = set()
    for fd, foff, hoff, ln in covered(rows):
        for k in range(ln // lf.c.chunk):
            got.add((fd, foff + k * lf.c.chunk, hoff + k * lf.c.chunk))
    assert got == want


def test_large_requests_are_split_and_iovecs_bounded(tmp_path):
    case = SsdCase(tmp_path, "LAYERFIRST", 1, 4096, 16, 1, 64, 1)  # 2 KiB chunks
    ids = np.arange(4096)
    rows = plan(case, ids, ids[::-1].copy())                       # 4096 iovecs of one chunk
    per_req = np.bincount(rows[:, 0])
    assert per_req.max() <= 1024 and len(per_req) == 4
    big = SsdCase(tmp_path / "big", "BLOCKFIRST", 32, 40, 64, 8, 128, 2, fill="random")  # 8 MiB blocks
    rows = plan(big, np.arange(40), np.arange(40))
    sizes = {}
    for req, _fd, _f, _h, ln in rows.tolist():
        sizes[req] = sizes.get(req, 0) + ln
    assert max(sizes.values()) <= 16 << 20 and sum(sizes.values()) == big.host.size


@pytest.mark.parametrize("entries", [0, 32], ids=["threads", "iouring"])
def test_few_large_requests_are_cut_up_for_the_workers(tmp_path, entries):
    """Six 8 MiB blocks make three 16 MiB requests; the engines cut them into pieces
    (in the middle of iovecs too) so that every worker has some.  Same bytes."""
    case = SsdCase(tmp_path, "BLOCKFIRST", 32, 6, 64, 8, 128, 2, fill="random")
    assert case.c.block == 8 << 20
    ids = np.arange(6)
    rows = plan(case, ids, ids[::-1].copy())
    assert len(set(rows[:, 0])) == 3 and len(rows) == 6
    ctx = SSDIOCTX(case.paths, 1, entries, 0)
    case.run(ctx, ids, ids[::-1].copy(), False, threads=5)
    case.oracle(ids, ids[::-1].copy(), False)
    assert np.array_equal(case.file_images()[0], case.ref_files[0])
    back = np.zeros_like(case.host)
    case.run(ctx, ids, [3, 4, 5, 0, 1, 2], True, host=back, threads=5)
    want = np.zeros_like(case.host)
    case.oracle(ids, [3, 4, 5, 0, 1, 2], True, host=want)
    assert np.array_equal(back, want)
    ctx.close()


# ---- errors -----------------------------------------------------------------------------------------------

def test_error_behaviour(tmp_path):
    with pytest.raises(RuntimeError, match="Failed to open file"):
        SSDIOCTX({0: [str(tmp_path / "missing.bin")]}, 1, 0, 0)
    with pytest.raises(RuntimeError, match="same, non-zero number of files"):
        SSDIOCTX({0: ["a"], 1: []}, 2, 0, 0)
    case = SsdCase(tmp_path, "BLOCKFIRST", 2, 4, 16, 1, 64, 2)
    for entries in (0, 8):
        ctx = SSDIOCTX(case.paths, 1, entries, 0)
        back = np.zeros(case.host.size * 4, dtype=np.uint8)
        with pytest.raises(RuntimeError, match="Failed to transfer data"):
            case.run(ctx, [9], [1], True, host=back)               # beyond the end of the file
        with pytest.raises(ValueError, match="negative block id"):
            case.run(ctx, [-1], [1], True, host=back)
        with pytest.raises(ValueError, match="differ in length"):
            case.run(ctx, [1, 2], [1], True, host=back)
        case.run(ctx, [], [], True, host=back)                     # nothing to do
        ctx.close()
