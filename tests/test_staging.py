"""The oracle's restatement of the compressed-staging helpers
(csrc/compression/common/staging_transfer.cuh) against a second, shaped statement:
the host cache as a numpy array [N, L, kv, capacity] and the size table as
[N, L, kv], indexed by (layer, kv, block id) in plain Python loops, so that the
stride arithmetic of the C loop is checked by something that has none."""
import numpy as np
import pytest

from oracle import fkv_oracle as O


def shaped_case(rng, L, kv_dim, NB, N, cap, stride, start_layer, nl, batch_start, bsz):
    host = rng.integers(0, 256, (N, L, kv_dim, cap), dtype=np.uint8)
    table = rng.integers(0, 1000, (N, L, kv_dim), dtype=np.uint32)
    ids = rng.permutation(N)[:NB].astype(np.int64)
    staging = rng.integers(0, 256, (bsz, stride), dtype=np.uint8)
    return host, table, ids, staging


def chunk_of(g, kv_dim, NB):
    return g // (kv_dim * NB), (g % (kv_dim * NB)) // NB, g % NB


@pytest.mark.parametrize("batch_start,bsz", [(0, 40), (7, 23), (39, 1), (13, 0)])
@pytest.mark.parametrize("kv_dim", [1, 2])
def test_write_matches_the_shaped_statement(kv_dim, batch_start, bsz):
    rng = np.random.default_rng(10 * kv_dim + batch_start)
    L, NB, N, cap, stride, start_layer, nl = 6, 5, 9, 96, 128, 2, 4   # nl*kv*NB chunks in the call
    batch_start = min(batch_start, nl * kv_dim * NB - 1)
    bsz = min(bsz, nl * kv_dim * NB - batch_start)
    host, table, ids, staging = shaped_case(rng, L, kv_dim, NB, N, cap, stride, start_layer, nl,
                                            batch_start, bsz)
    sizes = rng.integers(0, cap + 1, bsz).astype(np.uint64)
    if bsz > 3:
        sizes[1], sizes[3] = cap + 1, stride   # do not fit the host slot
        sizes[2] = cap                          # fits exactly
    want_host, want_table = host.copy(), table.copy()
    want_overflow = 0
    for i in range(bsz):
        layer, kv, b = chunk_of(batch_start + i, kv_dim, NB)
        if sizes[i] > cap:
            want_overflow += 1
            want_table[ids[b], start_layer + layer, kv] = 0
            continue
        want_table[ids[b], start_layer + layer, kv] = sizes[i]
        want_host[ids[b], start_layer + layer, kv, :int(sizes[i])] = staging[i, :int(sizes[i])]
    flat_host, flat_table = host.reshape(-1), table.reshape(-1)
    got = O.staging_transfer(staging.reshape(-1), stride, sizes, flat_host, cap, cap, kv_dim * cap,
                             L * kv_dim * cap, ids, flat_table, L * kv_dim, kv_dim, start_layer,
                             kv_dim, NB, batch_start, bsz, True)
    assert got == want_overflow
    assert np.array_equal(host, want_host) and np.array_equal(table, want_table)


@pytest.mark.parametrize("layout", ["blockfirst", "layerfirst"])
def test_read_matches_the_shaped_statement_and_round_trips(layout):
    rng = np.random.default_rng(3)
    L, kv_dim, NB, N, cap, stride, start_layer, nl = 5, 2, 4, 7, 80, 96, 1, 3
    total = nl * kv_dim * NB
    if layout == "blockfirst":      # [N, L, kv, cap]
        shape, strides = (N, L, kv_dim, cap), (cap, kv_dim * cap, L * kv_dim * cap)  # kv, layer, block
        at = lambda a, n, l, k: a[n, l, k]
    else:                            # [L, kv, N, cap]
        shape, strides = (L, kv_dim, N, cap), (N * cap, kv_dim * N * cap, cap)
        at = lambda a, n, l, k: a[l, k, n]
    host = rng.integers(0, 256, shape, dtype=np.uint8)
    table = np.zeros((N, L, kv_dim), dtype=np.uint32)
    ids = rng.permutation(N)[:NB].astype(np.int64)
    payload = rng.integers(0, 256, (total, stride), dtype=np.uint8)
    sizes = rng.integers(1, cap + 1, total).astype(np.uint64)
    O.staging_transfer(payload.reshape(-1), stride, sizes, host.reshape(-1), cap, *strides, ids,
                       table.reshape(-1), L * kv_dim, kv_dim, start_layer, kv_dim, NB, 0, total, True)
    for g in range(total):
        layer, kv, b = chunk_of(g, kv_dim, NB)
        assert table[ids[b], start_layer + layer, kv] == sizes[g]
        assert np.array_equal(at(host, ids[b], start_layer + layer, kv)[:int(sizes[g])],
                              payload[g, :int(sizes[g])])
    # read back in two batches that split a layer
    back = np.full((total, stride), 0xEE, dtype=np.uint8)
    got_sizes = np.zeros(total, dtype=np.uint64)
    for bs, n in ((0, 11), (11, total - 11)):
        O.staging_transfer(back[bs:].reshape(-1), stride, got_sizes[bs:], host.reshape(-1), cap,
                           *strides, ids, table.reshape(-1), L * kv_dim, kv_dim, start_layer, kv_dim,
                           NB, bs, n, False)
    assert np.array_equal(got_sizes, sizes)
    for g in range(total):
        n = int(sizes[g])
        assert np.array_equal(back[g, :n], payload[g, :n]) and (back[g, n:] == 0xEE).all()


def test_read_entry_beyond_the_staging_slot_is_counted_not_copied():
    L, kv_dim, NB, N, cap, stride = 1, 1, 3, 3, 64, 32
    host = np.arange(N * cap, dtype=np.uint8)
    table = np.array([10, 33, 32], dtype=np.uint32)     # 33 > stride
    staging = np.zeros(NB * stride, dtype=np.uint8)
    sizes = np.full(NB, 7, dtype=np.uint64)
    over = O.staging_transfer(staging, stride, sizes, host, cap, cap, cap, cap, np.arange(3), table,
                              1, 1, 0, 1, NB, 0, NB, False)
    assert over == 1 and sizes.tolist() == [10, 0, 32]
    assert not staging[stride:2 * stride].any()
    assert np.array_equal(staging[2 * stride:3 * stride], host[2 * cap:2 * cap + 32])


@pytest.mark.parametrize("backend", [O.BACKEND_VLLM, O.BACKEND_TRTLLM, O.BACKEND_SGLANG])
def test_chunk_ptrs_enumerate_layer_then_kv_then_block(backend):
    rng = np.random.default_rng(backend)
    L, kv_dim, NB = 5, 2, 4
    n_ptrs = {O.BACKEND_VLLM: L, O.BACKEND_TRTLLM: 1, O.BACKEND_SGLANG: 2 * L}[backend]
    ptrs = (rng.integers(1, 1 << 30, n_ptrs) * 4096).astype(np.uint64)
    kvs, bs, ls = 1 << 20, 4096, 1 << 24
    ids = rng.permutation(50)[:NB].astype(np.int64)
    start_layer, batch_start, bsz = 1, 5, 21
    got = O.chunk_ptrs(backend, ptrs, L, kvs, bs, ls, ids, start_layer, kv_dim, batch_start, bsz)
    want = []
    for layer in range(L - start_layer):
        for kv in range(kv_dim):
            for b in range(NB):
                want.append(O.chunk_addr(backend, ptrs, L, kvs, bs, ls, start_layer + layer, kv,
                                         int(ids[b])))
    assert got.tolist() == want[batch_start:batch_start + bsz]
