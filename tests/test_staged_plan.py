"""The arithmetic that decides which way a layerwise restore goes
(fkv_staged_restore_plan, no device involved): runs of consecutive host block ids,
holes that are read along, the staging row of every position, and the choice among
the kernel path, one copy command per run, and rows gathered by host threads with
one copy command per batch.  Checked by invariants and by a brute-force statement of
the same rules on small id sets."""
import ctypes

import numpy as np
import pytest

from flexkv_amd import _lib

L = _lib.load()


def policy(**kw):
    p = _lib.LaunchPolicy()
    p.staged_restore, p.staged_ring = 1, 3
    p.staged_copy_overhead_us, p.staged_overhead_pct = 10, 10
    p.staged_bridge_kb, p.staged_max_mb, p.link_gbps_estimate = 512, 512, 45
    for k, v in kw.items():
        setattr(p, k, v)
    return p


def plan(ids, row_bytes, pieces, pol):
    ids = np.ascontiguousarray(ids, dtype=np.int64)
    staged, nruns, rows = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int64()
    runs = (_lib.StagedRun * max(1, ids.size))()
    row_of = np.full(ids.size, -1, dtype=np.int64)
    _lib.check(L.fkv_staged_restore_plan(ids.ctypes.data, ids.size, row_bytes, pieces,
                                         ctypes.byref(pol), ctypes.byref(staged),
                                         ctypes.byref(nruns), ctypes.byref(rows), runs, ids.size,
                                         row_of.ctypes.data))
    return staged.value, [(r.first_id, r.rows, r.row0) for r in runs[:nruns.value]], \
        rows.value, row_of


KERNEL, RUNS, GATHERED = 0, 1, 2


def brute_force(ids, row_bytes, pieces, pol):
    """The rules restated on Python sets: bridge holes smallest first while one hole
    stays within the bridge size and all together within the allowed waste."""
    u = sorted(set(int(x) for x in ids))
    holes = sorted((b - a - 1, a) for a, b in zip(u, u[1:]) if b != a + 1)
    useful = len(u) * row_bytes
    waste, bridged = 0, set()
    for rows, after in holes:
        if rows * row_bytes > pol.staged_bridge_kb * 1024 or \
                waste + rows * row_bytes > useful * pol.staged_overhead_pct / 100:
            break
        waste += rows * row_bytes
        bridged.add(after)
    runs, start, prev = [], u[0], u[0]
    for x in u[1:]:
        if x != prev + 1 and prev not in bridged:
            runs.append((start, prev - start + 1))
            start = x
        prev = x
    runs.append((start, prev - start + 1))
    total = sum(r for _, r in runs)
    chosen = total * row_bytes <= pol.staged_max_mb << 20
    if pol.staged_restore == 1:
        batch_us = useful / (pol.link_gbps_estimate * 1e3)
        chosen = chosen and len(runs) * pieces * pol.staged_copy_overhead_us <= \
            batch_us * pol.staged_overhead_pct / 100
    chosen = chosen and len(runs) * pieces <= 4096   # never thousands of commands per batch
    return chosen and pol.staged_restore != 0, runs, total


@pytest.mark.parametrize("seed", range(12))
def test_runs_and_rows_against_brute_force(seed):
    rng = np.random.default_rng(seed)
    pool = int(rng.integers(8, 400))
    n = int(rng.integers(1, pool + 1))
    ids = rng.permutation(pool)[:n]
    if seed % 3 == 0:   # a few long runs with small holes
        ids = np.concatenate([np.arange(a, a + int(rng.integers(1, 40)))
                              for a in rng.integers(0, pool, 4)])
        ids = rng.permutation(ids)          # duplicates and any order are allowed
    row_bytes = int(rng.choice([4096, 73728, 1 << 20]))
    pieces = int(rng.choice([1, 2, 8]))
    pol = policy(staged_restore=2)          # the layout itself, whatever the cost rule says
    staged, runs, total, row_of = plan(ids, row_bytes, pieces, pol)
    want_staged, want_runs, want_total = brute_force(ids, row_bytes, pieces, pol)
    assert staged == (RUNS if want_staged else KERNEL)
    if not staged:
        return
    assert [(f, r) for f, r, _ in runs] == want_runs and total == want_total
    # runs ascend, do not touch, and their staging rows follow each other without gaps
    for (f0, r0, s0), (f1, r1, s1) in zip(runs, runs[1:]):
        assert f0 + r0 < f1 and s1 == s0 + r0
    assert runs[0][2] == 0 and runs[-1][2] + runs[-1][1] == total
    # every position lands on the row of its own host block, equal ids on equal rows
    for pos, i in enumerate(ids):
        f, r, s = next(x for x in runs if x[0] <= i < x[0] + x[1])
        assert row_of[pos] == s + (i - f)
    # what is read beyond the wanted blocks stays within the allowance
    assert (total - len(set(ids.tolist()))) * row_bytes <= \
        len(set(ids.tolist())) * row_bytes * pol.staged_overhead_pct / 100


def test_the_choice():
    one_run = np.arange(100, 612)
    scattered = np.random.default_rng(1).permutation(4096)[:512]
    pol = policy()
    assert plan(one_run, 73728, 1, pol)[0]                       # c3: 512 blocks of 72 KiB, one run
    assert not plan(scattered, 73728, 1, pol)[0]                 # hundreds of runs
    assert not plan(one_run[:4], 4096, 1, pol)[0]                # 16 KiB per batch: a command costs more
    assert plan(one_run[:4], 4096, 1, policy(staged_restore=2))[0]
    assert not plan(one_run, 73728, 1, policy(staged_restore=0))[0]
    assert not plan(one_run, 2 << 20, 1, policy(staged_max_mb=512))[0]   # 1 GiB of staging per batch
    # K and V apart on the host: twice the commands per run
    few = np.concatenate([np.arange(0, 200), np.arange(300, 500), np.arange(700, 900)])
    assert plan(few, 73728, 1, pol)[0] and not plan(few, 73728, 4, pol)[0]


def gather_policy(**kw):
    kw.setdefault("staged_gather", 1)
    kw.setdefault("gather_threads", 4)
    kw.setdefault("model_gather_thread_mbps", 20000)
    kw.setdefault("model_link_mbps", 57200)
    return policy(**kw)


def route_by_the_rules(ids, row_bytes, pieces, pol, cores):
    """The three-way choice restated: runs first; else the gather when the one copy
    command of a batch is cheap against the batch's link time and the threads finish
    a batch in 80 % of that time."""
    if brute_force(ids, row_bytes, pieces, pol)[0]:
        return RUNS
    n = len(ids)
    nbytes = n * row_bytes
    if pol.staged_gather == 0 or nbytes > pol.staged_max_mb << 20:
        return KERNEL
    if pol.staged_gather == 2:
        return GATHERED
    link_us = nbytes / pol.model_link_mbps
    if pol.staged_copy_overhead_us > link_us * pol.staged_overhead_pct / 100:
        return KERNEL
    threads = max(1, min(pol.gather_threads, max(1, cores - 1)))
    gather_us = nbytes / (threads * pol.model_gather_thread_mbps) + n * pieces * 0.05 / threads
    return GATHERED if gather_us <= 0.8 * link_us else KERNEL


@pytest.mark.parametrize("seed", range(40))
def test_the_three_way_choice_against_its_rules(seed):
    import os
    rng = np.random.default_rng(100 + seed)
    pool = int(rng.integers(64, 5000))
    n = int(rng.integers(1, min(pool, 600) + 1))
    ids = rng.permutation(pool)[:n] if seed % 4 else np.arange(7, 7 + n)
    row_bytes = int(rng.choice([2048, 73728, 262144, 1 << 20]))
    pieces = int(rng.choice([1, 2, 16, 64]))
    pol = gather_policy(staged_restore=int(rng.choice([0, 1, 1, 2])),
                        staged_gather=int(rng.choice([0, 1, 1, 2])),
                        gather_threads=int(rng.choice([1, 2, 4, 6])),
                        model_link_mbps=int(rng.choice([14000, 28600, 57200])))
    got, runs, total, row_of = plan(ids, row_bytes, pieces, pol)
    assert got == route_by_the_rules(ids, row_bytes, pieces, pol, os.cpu_count() or 1), \
        (n, row_bytes, pieces, pol.staged_restore, pol.staged_gather, pol.gather_threads)
    if got == GATHERED:   # no runs; position p is staged on row p
        assert runs == [] and total == n and (row_of == np.arange(n)).all()


def test_scattered_host_blocks_are_gathered_when_the_threads_keep_up():
    scattered = np.random.default_rng(1).permutation(4096)[:512]
    one_run = np.arange(100, 612)
    c3 = (scattered, 73728, 1)                                    # 36 MiB per batch, 512 runs
    assert plan(*c3, gather_policy())[0] == GATHERED
    assert plan(one_run, 73728, 1, gather_policy())[0] == RUNS    # a run needs no host pass
    assert plan(*c3, gather_policy(staged_gather=0))[0] == KERNEL
    # two threads at 20 GB/s each do not finish 36 MiB inside 80 % of its link time ...
    assert plan(*c3, gather_policy(gather_threads=2))[0] == KERNEL
    # ... unless the link is half as fast: the choice follows the link figure
    assert plan(*c3, gather_policy(gather_threads=2, model_link_mbps=28600))[0] == GATHERED
    # a batch of 16 KiB: one copy command costs more than the batch's time on the link
    assert plan(scattered[:4], 4096, 1, gather_policy())[0] == KERNEL
    assert plan(scattered[:4], 4096, 1, gather_policy(staged_gather=2))[0] == GATHERED
    # rows cut into 64 small pieces each: the per-piece cost eats the margin
    assert plan(scattered, 73728, 64, gather_policy())[0] == KERNEL
    # forced routes for tests: runs wins where both are forced
    assert plan(*c3, gather_policy(staged_restore=2, staged_gather=2))[0] == RUNS
    assert plan(*c3, gather_policy(staged_restore=0, staged_gather=2))[0] == GATHERED
    # a batch beyond the largest staging buffer stays on the kernel path
    assert plan(scattered, 2 << 20, 1, gather_policy(staged_gather=2))[0] == KERNEL


def test_holes_are_bridged_smallest_first_within_the_allowance():
    # runs of 50 blocks with holes of 1, 2 and 30 blocks; rows of 64 KiB: the allowance is
    # 10 % of 200 rows = 20 rows, the bridge size 512 KiB = 8 rows
    ids = np.concatenate([np.arange(0, 50), np.arange(51, 101), np.arange(103, 153),
                          np.arange(183, 233)])
    staged, runs, total, _ = plan(ids, 65536, 1, policy(staged_restore=2))
    assert staged and [(f, r) for f, r, _ in runs] == [(0, 153), (183, 50)] and total == 203
    # a smaller allowance takes the 1-block hole only
    staged, runs, total, _ = plan(ids, 65536, 1, policy(staged_restore=2, staged_overhead_pct=1))
    assert [(f, r) for f, r, _ in runs] == [(0, 101), (103, 50), (183, 50)] and total == 201
    # no bridging at all
    staged, runs, total, _ = plan(ids, 65536, 1, policy(staged_restore=2, staged_bridge_kb=0))
    assert len(runs) == 4 and total == 200


def test_bad_arguments():
    ids = np.arange(4, dtype=np.int64)
    out = ctypes.c_int32()
    assert L.fkv_staged_restore_plan(ids.ctypes.data, 4, 4096, 1, None, ctypes.byref(out), None,
                                     None, None, 0, None) == _lib.FKV_ERR_INVALID_ARG
    pol = policy()
    assert L.fkv_staged_restore_plan(None, 0, 4096, 1, ctypes.byref(pol), ctypes.byref(out), None,
                                     None, None, 0, None) == _lib.FKV_OK and out.value == 0
