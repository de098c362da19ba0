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
    from flexkv_amd.c_ext import plan_counters_dirty
    assert plan_counters_dirty() == 0   # every launch left its claim counters zeroed


def test_first_launches_of_a_fresh_process_leave_clean_counters(gpu_device):
    """The claim counters of a plan slot are created with the slot.  The very
    first launches of a process, on non-blocking streams, must find them zeroed
    and leave them zeroed (a clear that is still under way when the first kernel
    claims from them leaves them dirty, and a later launch to a single
    workgroup).  Several fresh processes, each checked after a dozen transfers."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = (
        "import sys; sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + '/tests')\n"
        "import numpy as np, torch\n"
        "from kvsetup import KVSetup\n"
        "from flexkv_amd.c_ext import get_stats, plan_counters_dirty\n"
        "s = KVSetup(0, 8, 2, 400, 400, 32768, 'BLOCKFIRST', seed=1)\n"
        "dev = s.to_device('cuda:0')\n"
        "st = [torch.cuda.Stream(), torch.cuda.Stream()]\n"
        "ids = np.arange(300)\n"
        "for k in range(12):\n"
        "    with torch.cuda.stream(st[k % 2]):\n"
        "        dev.transfer(ids, ids, is_h2d=(k % 2 == 1), sync=False)\n"
        "torch.cuda.synchronize()\n"
        "assert get_stats()['confined_launches'] == 12\n"
        "print('dirty', plan_counters_dirty())\n")
    for _ in range(3):
        r = subprocess.run([sys.executable, "-c", script, root], capture_output=True, text=True,
                           timeout=170)
        assert r.returncode == 0 and r.stdout.split()[-2:] == ["dirty", "0"], r.stdout + r.stderr
