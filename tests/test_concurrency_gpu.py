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
