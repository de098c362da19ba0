"""Random puts and gets from several threads and streams at once, each thread on
its own share of the blocks, replayed on the CPU oracle and compared byte for
byte at the end.  Every launch meets launches of the other direction, so the
XCD split, the claim counters, the plan memory and the lane streams are all in
play."""
import threading
import time

import numpy as np
import pytest
import torch

from kvsetup import KVSetup, VLLM

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("chunk", [16384, 1152, 73728], ids=["16k", "packed", "72k"])
def test_random_transfers_from_six_threads(gpu_device, chunk):
    threads, per, seconds = 6, 128, 1.5
    s = KVSetup(VLLM, 4, 2, threads * per, threads * per, chunk, "BLOCKFIRST", seed=chunk)
    dev = s.to_device(gpu_device)
    errors, counts, lock = [], [0] * threads, threading.Lock()

    def work(t):
        try:
            rng = np.random.default_rng(100 + t)
            streams = [torch.cuda.Stream() for _ in range(3)]
            base, end = t * per, time.time() + seconds
            while time.time() < end:
                n = int(rng.integers(1, per))
                g, c = base + rng.permutation(per)[:n], base + rng.permutation(per)[:n]
                h2d, sync = bool(rng.integers(0, 2)), bool(rng.integers(0, 4))
                st = streams[int(rng.integers(0, 3))]
                with torch.cuda.stream(st):
                    dev.transfer(g, c, is_h2d=h2d, sync=sync)
                    if not sync:
                        st.synchronize()
                with lock:   # the oracle replays this thread's transfers in its order
                    s.oracle_transfer(g, c, h2d)
                counts[t] += 1
        except Exception as e:  # noqa: BLE001
            errors.append(repr(e))
    workers = [threading.Thread(target=work, args=(t,)) for t in range(threads)]
    [w.start() for w in workers]
    [w.join() for w in workers]
    torch.cuda.synchronize()
    assert not errors, errors
    assert min(counts) > 5, counts
    dev.assert_matches_reference(f"{sum(counts)} concurrent transfers, chunk {chunk}")
    # every plan went back to the pool, and the pool never made a request wait for a slot
    from flexkv_amd.c_ext import get_stats
    st = get_stats()
    assert st["plan_slots"] > 0 and st["plan_slots_in_use"] == 0, st



@pytest.mark.parametrize("dirty", ["0", "1"], ids=["zeroed", "garbage"])
def test_first_launches_of_a_fresh_process(gpu_device, dirty):
    """The claim counters of a plan slot are created with the slot.  The very
    first launches of a process, on non-blocking streams, must hand out all their
    work whatever the counters hold at that moment: zeroes, or (with the test
    switch FKV_TEST_DIRTY_COUNTERS) the leftovers of something else.  A launch
    that mistook leftovers for claims would copy nothing."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = (
        "import sys; sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + '/tests')\n"
        "import numpy as np, torch\n"
        "from kvsetup import KVSetup\n"
        "from flexkv_amd.c_ext import get_stats\n"
        "s = KVSetup(0, 8, 2, 400, 400, 32768, 'BLOCKFIRST', seed=1)\n"
        "dev = s.to_device('cuda:0')\n"
        "st = [torch.cuda.Stream(), torch.cuda.Stream()]\n"
        "rng = np.random.default_rng(5)\n"
        "for k in range(12):\n"
        "    g, c = rng.permutation(400)[:300], rng.permutation(400)[:300]\n"
        "    with torch.cuda.stream(st[k % 2]):\n"
        "        dev.transfer(g, c, is_h2d=(k % 2 == 1), sync=True)\n"
        "    s.oracle_transfer(g, c, k % 2 == 1)\n"
        "torch.cuda.synchronize()\n"
        "print('confined launches:', get_stats()['confined_launches'])\n"
        "dev.assert_matches_reference('first launches')\n"
        "print('ok')\n")
    env = dict(os.environ, FKV_TEST_DIRTY_COUNTERS=dirty)
    for _ in range(2):
        r = subprocess.run([sys.executable, "-c", script, root], capture_output=True, text=True,
                           timeout=170, env=env)
        assert r.returncode == 0 and r.stdout.split()[-1:] == ["ok"], r.stdout + r.stderr


def test_waiting_requests_leave_the_cores_alone(gpu_device):
    """The runtime's waits keep a core busy each.  With eight threads waiting for their
    synchronous transfers at once the library lets two of them wait that way and the others
    poll with sleeps: the process uses well under half of the eight cores it would otherwise
    (with quiet_wait_us = 0, the runtime's wait for everybody, it uses most of them: printed,
    the box decides).  The bytes are checked against the oracle afterwards."""
    from flexkv_amd.c_ext import launch_policy
    threads, per, rounds = 8, 64, 12
    s = KVSetup(VLLM, 4, 2, threads * per, threads * per, 65536, "BLOCKFIRST", seed=5)
    dev = s.to_device(gpu_device)
    ids = [np.arange(t * per, (t + 1) * per, dtype=np.int64) for t in range(threads)]

    def burst(h2d):
        barrier = threading.Barrier(threads + 1)

        def work(t):
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                barrier.wait()
                for _ in range(rounds):
                    dev.transfer(ids[t], ids[t], is_h2d=h2d, sync=True)
        workers = [threading.Thread(target=work, args=(t,)) for t in range(threads)]
        [w.start() for w in workers]
        barrier.wait()
        cpu0, t0 = time.process_time(), time.perf_counter()
        [w.join() for w in workers]
        return (time.process_time() - cpu0) / (time.perf_counter() - t0)

    burst(False)                                   # streams, plans, lanes
    cores = max(burst(False), burst(True))
    with launch_policy(quiet_wait_us=0):
        spinning = max(burst(False), burst(True))
    print("cores busy with eight waiting threads: %.1f, with the runtime's wait for all: %.1f"
          % (cores, spinning))
    assert cores < 4.0, (cores, spinning)
    # a negative setting makes every waiter poll: one thread waiting for its transfers then
    # leaves its core alone too
    with launch_policy(quiet_wait_us=-100):
        cpu0, t0 = time.process_time(), time.perf_counter()
        for _ in range(40):
            dev.transfer(np.arange(threads * per, dtype=np.int64),
                         np.arange(threads * per, dtype=np.int64), is_h2d=False, sync=True)
        alone = (time.process_time() - cpu0) / (time.perf_counter() - t0)
    print("one waiting thread, every waiter polling: %.2f cores" % alone)
    assert alone < 0.6, alone
    for t in range(threads):
        s.oracle_transfer(ids[t], ids[t], False)
        s.oracle_transfer(ids[t], ids[t], True)
    dev.assert_matches_reference("eight threads of synchronous transfers")
