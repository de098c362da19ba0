#!/usr/bin/env python3
"""Benchmark of the GPU<->CPU KV-block transfer path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c0..c4]

A step is one pass of the hot path over one batch of block ids: a GPU->host
gather of the selected blocks into the host cache followed by the host->GPU
scatter of the same blocks (c0, c1, c2), one layer-by-layer restore (c3), or
one burst of 64 concurrent requests (c4).  Inputs are resident in HBM / pinned
host memory before the timed region starts.  One JSON line is printed.

Configurations (BASELINE.json "configs"):
  c0  Llama-3-8B, vLLM layout, bf16: 32 x [2,4096,16,8,128]; 256 random blocks
  c1  SGLang token-major, bf16, page 64: 64 x [262144,8,128]; 1024 pages
      (64 runs of 8 + 512 isolated)                      <- default, the metric's config
  c2  TRT-LLM layout, fp8 e4m3: [4096,80,2,8,32,128]; 2048 random blocks
  c3  DeepSeek-V3 MLA, bf16: 61 x [16384,64,576]; layerwise restore of 512 blocks
  c4  64 concurrent requests on the c0 shape with a 32768-block pool
Beyond BASELINE.json (the rows next to the path):
  mg      layerwise restore of heterogeneous layer groups + sliding-window sidecar
          (DeepSeek-V4-like: 61 layers, two compressed latent groups, an indexer group)
  worker  c0-shaped put/get ops through a transfer worker process (pipe + shared op pool)
  groups  whole-block ops of a model with three layer groups: one call per group against
          one call for all; chunk sizes that are no whole number of slices
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth
METRIC = "KV block transfer GB/s (D2H, H2D) on 1 GPU; % of measured host-link peak"

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs of this script scaled by plain copy kernels of known size
# (profiles/fkv_copy_chunks_kernel_c1_pmc.md).  None where no such run was made.
MEASURED_TRAFFIC_BYTES = {("c1", "kernel"): 8590414848, ("transform-c0", "kernel"): 8590474240}


def _median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


# ---------------------------------------------------------------------------
# workloads
# ---------------------------------------------------------------------------
class Workload:
    """GPU tensors, pinned host cache, ids and strides of one configuration."""

    def __init__(self, name, torch, device, scale=1.0):
        self.name, self.torch, self.device = name, torch, device
        t = torch
        g = lambda seed: t.Generator().manual_seed(seed)
        if name in ("c0", "c4"):
            L, N, T, H, D = 32, (4096 if name == "c0" else 32768), 16, 8, 128
            self.desc = ("Llama-3-8B vLLM layout bf16: 32 x [2,%d,16,8,128], host [NH,32,2,16,8,128]"
                         % N)
            self.backend, self.kv_dim, self.L = 0, 2, L
            self.chunk = T * H * D * 2
            gen = t.Generator(device=device).manual_seed(0)
            self.tensors = [t.randn(2, N, T, H, D, device=device, dtype=t.bfloat16, generator=gen)
                            for _ in range(L)]
            self.gks, self.gbs, self.gls = N * self.chunk, self.chunk, 2 * N * self.chunk
            self.num_gpu_blocks = N
            if name == "c0":
                gg = g(1)
                n = 256
                self.NH = 1024
                self.gpu_ids = t.randperm(N, generator=gg)[:n].to(t.int64)
                self.cpu_ids = t.randperm(self.NH, generator=gg)[:n].to(t.int64)
            else:
                # 64 requests, sizes min(512, Geometric(p=1/48)), disjoint random ids
                gg = g(5)
                sizes = t.empty(64).geometric_(1.0 / 48, generator=gg).clamp(1, 512).to(t.int64)
                total = int(sizes.sum())
                self.NH = total
                perm_g = t.randperm(N, generator=gg)[:total].to(t.int64)
                perm_c = t.randperm(self.NH, generator=gg)[:total].to(t.int64)
                offs = [0] + list(t.cumsum(sizes, 0).tolist())
                self.requests = [(perm_g[offs[i]:offs[i + 1]].contiguous(),
                                  perm_c[offs[i]:offs[i + 1]].contiguous()) for i in range(64)]
                self.gpu_ids, self.cpu_ids = perm_g, perm_c
        elif name == "c1":
            L, tokens, H, D, page = 32, 262144, 8, 128, 64
            self.desc = ("SGLang token-major bf16 page 64: 64 x [262144,8,128] (K then V, 32 layers), "
                         "1024 pages = 64 runs of 8 + 512 isolated, host [1024,32,2,64,8,128]")
            self.backend, self.kv_dim, self.L = 2, 2, L
            self.chunk = page * H * D * 2
            gen = t.Generator(device=device).manual_seed(2)
            self.tensors = [t.randn(tokens, H, D, device=device, dtype=t.bfloat16, generator=gen)
                            for _ in range(2 * L)]
            N = tokens // page
            self.num_gpu_blocks = N
            self.gks, self.gbs, self.gls = 0, self.chunk, N * self.chunk
            self.NH = 1024
            self.gpu_ids = sglang_page_ids(t, N, seed=2)
            self.cpu_ids = t.arange(self.NH, dtype=t.int64)
        elif name == "c2":
            N, L, H, T, D = 4096, 80, 8, 32, 128
            self.desc = ("TRT-LLM layout fp8 e4m3: one [4096,80,2,8,32,128] tensor, 2048 random "
                         "blocks, host [2048,80,2,8,32,128]")
            self.backend, self.kv_dim, self.L = 1, 2, L
            self.chunk = H * T * D
            gen = t.Generator(device=device).manual_seed(3)
            codes = t.randint(0, 254, (N, L, 2, H, T, D), device=device, dtype=t.uint8,
                              generator=gen)
            codes += (codes >= 0x7F).to(t.uint8)  # skip 0x7F; 0xFF is never produced
            self.tensors = [codes]
            self.num_gpu_blocks = N
            self.gks, self.gls, self.gbs = self.chunk, 2 * self.chunk, L * 2 * self.chunk
            self.NH = 2048
            gg = g(3)
            self.gpu_ids = t.randperm(N, generator=gg)[:2048].to(t.int64)
            self.gpu_ids_reload = t.randperm(N, generator=gg)[:2048].to(t.int64)
            self.cpu_ids = t.arange(2048, dtype=t.int64)
        elif name == "c3":
            L, N, T, D = 61, 16384, 64, 576
            self.desc = ("DeepSeek-V3 MLA latent KV bf16: 61 x [16384,64,576], layerwise restore of "
                         "512 blocks, host [512,61,1,64,1,576]")
            self.backend, self.kv_dim, self.L = 0, 1, L
            self.chunk = T * D * 2
            gen = t.Generator(device=device).manual_seed(4)
            self.tensors = [(t.randn(N, T, D, device=device, dtype=t.bfloat16, generator=gen) * 0.5)
                            for _ in range(L)]
            self.num_gpu_blocks = N
            self.gks, self.gbs, self.gls = N * self.chunk, self.chunk, N * self.chunk
            self.NH = 512
            gg = g(4)
            self.gpu_ids = t.randperm(N, generator=gg)[:512].to(t.int64)
            self.cpu_ids = t.randperm(self.NH, generator=gg)[:512].to(t.int64)
        else:
            raise ValueError(name)
        # host cache, block-first: [NH, L, kv, chunk]
        self.cks = self.chunk
        self.cls = self.kv_dim * self.chunk
        self.cbs = self.L * self.kv_dim * self.chunk
        self.host = t.empty(self.NH * self.cbs, dtype=t.uint8, pin_memory=True)
        self.ptrs = t.tensor([x.data_ptr() for x in self.tensors], dtype=t.int64).pin_memory()
        self.num_blocks = int(self.gpu_ids.numel())
        self.bytes_per_direction = self.num_blocks * self.L * self.kv_dim * self.chunk

    def transfer(self, gpu_ids, cpu_ids, h2d, **kw):
        from flexkv_amd.c_ext import transfer_kv_blocks
        kw.setdefault("sync", False)
        transfer_kv_blocks(gpu_ids, self.ptrs, self.gks, self.gbs, self.gls, cpu_ids, self.host,
                           self.cks, self.cls, self.cbs, self.chunk, 0, self.L,
                           is_host_to_device=h2d, kv_dim=self.kv_dim, gpu_block_type=self.backend,
                           is_blockfirst=True, **kw)

    # block rows of one (layer, kv) as a [N, chunk] uint8 view of the engine tensor
    def gpu_rows(self, layer, kv):
        t = self.torch
        if self.backend == 0:
            x = self.tensors[layer]
            x = x[kv] if self.kv_dim == 2 else x
            return x.reshape(self.num_gpu_blocks, -1).view(t.uint8)
        if self.backend == 2:
            return self.tensors[kv * self.L + layer].view(self.num_gpu_blocks, -1).view(t.uint8)
        return self.tensors[0][:, layer, kv].reshape(self.num_gpu_blocks, -1)  # strided view

    def host_rows(self, layer, kv):
        return self.host.view(self.NH, self.L, self.kv_dim, self.chunk)[:, layer, kv]

    def verify_host_image(self, gpu_ids, cpu_ids):
        """host[cpu_ids, l, kv] == engine rows [gpu_ids], compared on the GPU
        against torch's own index_select."""
        t = self.torch
        gi, ci = gpu_ids.to(self.device), cpu_ids
        for l in range(self.L):
            for kv in range(self.kv_dim):
                want = self.gpu_rows(l, kv).index_select(0, gi)
                got = self.host_rows(l, kv).index_select(0, ci).to(self.device)
                if not t.equal(want, got):
                    return False
        return True


def sglang_page_ids(t, num_pages, seed, runs=64, run_len=8, isolated=512):
    """64 non-overlapping runs of 8 consecutive pages + 512 isolated pages not
    adjacent to any chosen page, order shuffled; everything from one generator."""
    g = t.Generator().manual_seed(seed)
    taken = t.zeros(num_pages + 2, dtype=t.bool)  # index shifted by one, guards at both ends
    pieces = []
    while len(pieces) < runs:
        s = int(t.randint(0, num_pages - run_len + 1, (1,), generator=g))
        if not taken[s:s + run_len + 2].any():   # the run and one page on either side are free
            taken[s + 1:s + 1 + run_len] = True
            pieces.append(t.arange(s, s + run_len, dtype=t.int64))
    singles = 0
    while singles < isolated:
        s = int(t.randint(0, num_pages, (1,), generator=g))
        if not taken[s:s + 3].any():
            taken[s + 1] = True
            pieces.append(t.tensor([s], dtype=t.int64))
            singles += 1
    order = t.randperm(len(pieces), generator=g).tolist()
    return t.cat([pieces[i] for i in order]).contiguous()


# ---------------------------------------------------------------------------
# measurements
# ---------------------------------------------------------------------------
def measure_link(device_index=0, nbytes=1 << 30, reps=10):
    from flexkv_amd import _lib
    L = _lib.load()
    out = {}
    for name, direction in (("d2h", 0), ("h2d", 1)):
        best, med = ctypes.c_double(), ctypes.c_double()
        _lib.check(L.fkv_measure_link_peak(device_index, nbytes, reps, direction,
                                           ctypes.byref(best), ctypes.byref(med)))
        out[name] = best.value
    return out


def measure_link_bidirectional(torch, device, nbytes=1 << 30, reps=6):
    """Plain pinned copies in both directions at once (two streams), best of `reps`:
    the yardstick for puts running next to gets."""
    hd = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
    hu = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
    dd = torch.empty(nbytes, dtype=torch.uint8, device=device)
    du = torch.empty(nbytes, dtype=torch.uint8, device=device)
    s_up, s_down = torch.cuda.Stream(), torch.cuda.Stream()
    best = float("inf")
    for _ in range(reps + 1):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        with torch.cuda.stream(s_up):
            hu.copy_(du, non_blocking=True)
        with torch.cuda.stream(s_down):
            dd.copy_(hd, non_blocking=True)
        torch.cuda.synchronize()
        best = min(best, time.perf_counter() - t0)
    return 2 * nbytes / best / 1e9


def run_gather_scatter(w, torch, steps, warmup, num_cta, use_ce):
    """c0 / c1 / c2: D2H gather then H2D scatter per step."""
    st = torch.cuda.Stream()
    kw = dict(transfer_num_cta=num_cta, use_ce_transfer=use_ce, ce_path_opt=True)
    reload_ids = getattr(w, "gpu_ids_reload", w.gpu_ids)
    ev = lambda: torch.cuda.Event(enable_timing=True)
    d2h_ms, h2d_ms = [], []
    torch.cuda.synchronize()   # the tensors were filled on another stream
    with torch.cuda.stream(st):
        for _ in range(warmup):
            w.transfer(w.gpu_ids, w.cpu_ids, False, **kw)
            w.transfer(reload_ids, w.cpu_ids, True, **kw)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        marks = []
        for _ in range(steps):
            a, b, c = ev(), ev(), ev()
            a.record(st)
            w.transfer(w.gpu_ids, w.cpu_ids, False, **kw)
            b.record(st)
            w.transfer(reload_ids, w.cpu_ids, True, **kw)
            c.record(st)
            marks.append((a, b, c))
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    for a, b, c in marks:
        d2h_ms.append(a.elapsed_time(b))
        h2d_ms.append(b.elapsed_time(c))
    return wall, d2h_ms, h2d_ms


def verify_round_trip(w, torch, num_cta):
    """Bit-exactness at full size through size-independent properties:
    (1) the host image equals torch's own index_select of the engine tensors;
    (2) gather -> erase the blocks on the GPU -> scatter restores every byte."""
    from flexkv_amd.c_ext import transfer_kv_blocks  # noqa: F401
    w.host.zero_()
    w.transfer(w.gpu_ids, w.cpu_ids, False, transfer_num_cta=num_cta, sync=True)
    ok = w.verify_host_image(w.gpu_ids, w.cpu_ids)
    gi = w.gpu_ids.to(w.device)
    saved = [[w.gpu_rows(l, kv).index_select(0, gi) for kv in range(w.kv_dim)] for l in range(w.L)]
    for l in range(w.L):
        for kv in range(w.kv_dim):
            w.gpu_rows(l, kv).index_fill_(0, gi, 0)
    w.transfer(w.gpu_ids, w.cpu_ids, True, transfer_num_cta=num_cta, sync=True)
    for l in range(w.L):
        for kv in range(w.kv_dim):
            ok = ok and torch.equal(w.gpu_rows(l, kv).index_select(0, gi), saved[l][kv])
    return bool(ok)


def run_layerwise(w, torch, steps, warmup, num_cta, notify, dummy, layer_spans=False):
    """c3: per-layer restore with a dummy per-layer compute kernel on a second
    stream gated on each layer's event.  `layer_spans` brackets every layer's
    compute with two timing events; torch creates them with default flags, and
    next to a transfer over the host link each such event idles the compute
    stream for 0.1 ms or more, so the spans are off unless asked for."""
    from flexkv_amd.c_ext import LayerwiseTransferGroup
    i64 = lambda v: torch.tensor([v], dtype=torch.int64)
    grp = LayerwiseTransferGroup(
        num_gpus=1, gpu_blocks=[w.tensors], cpu_blocks=w.host, ssd_files={}, num_layers=w.L,
        gpu_kv_strides_tensor=i64(w.gks), gpu_block_strides_tensor=i64(w.gbs),
        gpu_layer_strides_tensor=i64(w.gls), gpu_chunk_sizes_tensor=i64(w.chunk),
        iouring_entries=0, iouring_flags=0,
        layer_eventfds_tensor=torch.empty(0, dtype=torch.int32), tp_size=1, is_blockfirst=True)
    empty = torch.empty(0, dtype=torch.int64)

    def restore():
        grp.layerwise_transfer(
            empty, empty, 0, 0, 0, 0, 0, w.gpu_ids, w.cpu_ids, w.cks, w.cls, w.cbs, w.chunk,
            w.cks, w.cls, w.cbs, num_cta, False, w.L, 1, w.kv_dim, 1, counter_id=0,
            kv_shared_across_ranks_mode="sharded", notify_mode=notify)

    layer_bytes = w.num_blocks * w.kv_dim * w.chunk
    # Dummy per-layer compute on a second stream, sized to about one layer's copy
    # time: fused attention (default; what a restored layer feeds), a 2048^3 GEMM
    # chain, or a streaming elementwise kernel.
    comp = torch.cuda.Stream()
    ev = lambda: torch.cuda.Event(enable_timing=True)
    target_ms = layer_bytes / 55e9 * 1e3
    if dummy == "sdpa":
        q = torch.randn(1, 32, 2048, 128, device=w.device, dtype=torch.bfloat16)
        unit = lambda: torch.nn.functional.scaled_dot_product_attention(q, q, q)
    elif dummy in ("gemm", "gemm4k"):
        # 2048^3: one round of workgroups on 256 CUs, so a single CU held by a copy
        # wavefront costs a second round; 4096^3: several rounds, the loss is the
        # share of CUs the copy holds
        n = 2048 if dummy == "gemm" else 4096
        a = torch.randn(n, n, device=w.device, dtype=torch.bfloat16)
        b = torch.randn(n, n, device=w.device, dtype=torch.bfloat16)
        c = torch.empty(n, n, device=w.device, dtype=torch.bfloat16)
        unit = lambda: torch.matmul(a, b, out=c)
    else:
        x = torch.randn(16 << 20, device=w.device)
        unit = lambda: x.mul_(1.0001)

    def layer_compute(reps):
        for _ in range(reps):
            unit()

    def compute_only(reps):
        with torch.cuda.stream(comp):
            s, e = ev(), ev()
            s.record(comp)
            for _ in range(w.L):
                layer_compute(reps)
            e.record(comp)
        e.synchronize()
        return s.elapsed_time(e)

    compute_only(1)
    per_unit = compute_only(4) / (4 * w.L)
    reps = max(1, int(round(target_ms / per_unit)))
    compute_ms = _median([compute_only(reps) for _ in range(3)])

    alone = []
    for _ in range(max(2, warmup + 1)):   # restore with nobody computing next to it
        torch.cuda.synchronize()
        restore()
        grp.synchronize()
        alone.append(grp.batch_times_ms()[-1])
    restore_alone_ms = min(alone[1:]) if len(alone) > 1 else alone[0]

    totals, restores, firsts, stalls, busy = [], [], [], [], []
    for it in range(warmup + steps):
        torch.cuda.synchronize()
        s, e = ev(), ev()
        spans = []
        with torch.cuda.stream(comp):
            s.record(comp)
        restore()  # polling: returns right after the launches
        with torch.cuda.stream(comp):
            for l in range(w.L):
                grp.wait_layer(l, comp)
                if layer_spans:
                    a0, a1 = ev(), ev()
                    a0.record(comp)        # stamped once layer l has landed
                layer_compute(reps)
                if layer_spans:
                    a1.record(comp)
                    spans.append((a0, a1))
            e.record(comp)
        e.synchronize()
        grp.synchronize()
        if it >= warmup:
            bt = grp.batch_times_ms()
            total = s.elapsed_time(e)
            # without spans: what the compute stream needs alone, i.e. every ms beyond
            # that counts as stalled (waiting for a layer, or slowed down by the copies)
            computing = sum(x.elapsed_time(y) for x, y in spans) if layer_spans else compute_ms
            totals.append(total)
            restores.append(bt[-1])
            firsts.append(bt[0])
            busy.append(computing)
            stalls.append(total - computing)  # compute stream idle, waiting for a layer
    grp.close()
    return dict(total_ms=_median(totals), restore_ms=_median(restores),
                first_layer_ms=_median(firsts), compute_ms=compute_ms,
                compute_overlapped_ms=_median(busy), stall_ms=_median(stalls),
                compute_reps_per_layer=reps, layer_bytes=layer_bytes,
                restore_alone_ms=restore_alone_ms)


def run_concurrent(w, torch, steps, warmup, num_cta, streams_per_direction=32, verify=True):
    """c4: 32 D2H puts and 32 H2D gets issued at once from 64 threads.  Each
    direction has its own set of streams (one per request by default); the
    process has 4 hardware queues, so with more than 2 streams per direction
    puts and gets also share queues and partly serialize."""
    reqs = w.requests
    per_dir = max(1, min(streams_per_direction, len(reqs) // 2))
    pool = [[torch.cuda.Stream() for _ in range(per_dir)] for _ in range(2)]
    if per_dir == 1:
        # one put stream and one get stream: take a pair that does not share a hardware queue
        from flexkv_amd.c_ext import streams_run_concurrently
        spare = []
        while not streams_run_concurrently(pool[0][0], pool[1][0]) and len(spare) < 8:
            spare.append(pool[1][0])       # keep it alive so the next one is a different stream
            pool[1][0] = torch.cuda.Stream()
    streams = [pool[i % 2][(i // 2) % per_dir] for i in range(len(reqs))]
    lat = [[] for _ in reqs]
    walls = []
    w.transfer(w.gpu_ids, w.cpu_ids, False, transfer_num_cta=num_cta, sync=True)  # fill the host cache
    if verify:
        # make every request visible: engine blocks of the puts change sign (the host still
        # holds the old values), engine blocks of the gets are wiped (the host holds them)
        for i, (gi, _) in enumerate(reqs):
            idx = gi.to(w.device)
            for l in range(w.L):
                for kv in range(w.kv_dim):
                    rows = w.gpu_rows(l, kv)
                    if i % 2 == 0:
                        rows.index_copy_(0, idx, rows.index_select(0, idx) ^ 0x80)
                    else:
                        rows.index_fill_(0, idx, 0)
        torch.cuda.synchronize()

    def worker(i, barrier, record):
        gi, ci = reqs[i]
        with torch.cuda.stream(streams[i]):
            barrier.wait()
            t0 = time.perf_counter()
            w.transfer(gi, ci, h2d=(i % 2 == 1), transfer_num_cta=num_cta, sync=True)
            if record:
                lat[i].append((time.perf_counter() - t0) * 1e3)

    for it in range(warmup + steps):
        barrier = threading.Barrier(len(reqs) + 1)
        threads = [threading.Thread(target=worker, args=(i, barrier, it >= warmup))
                   for i in range(len(reqs))]
        for th in threads:
            th.start()
        torch.cuda.synchronize()
        barrier.wait()
        t0 = time.perf_counter()
        for th in threads:
            th.join()
        if it >= warmup:
            walls.append(time.perf_counter() - t0)
    all_lat = sorted(x for l in lat for x in l)
    p99 = all_lat[min(len(all_lat) - 1, int(0.99 * len(all_lat)))]
    total_bytes = sum(int(g.numel()) for g, _ in reqs) * w.L * w.kv_dim * w.chunk
    # after the requests the host image of every block equals its engine block, and no
    # block of a get is still wiped
    ok = None
    if verify:
        ok = w.verify_host_image(w.gpu_ids, w.cpu_ids) and all(
            bool(w.gpu_rows(l, 0).index_select(0, reqs[1][0].to(w.device)).any())
            for l in (0, w.L - 1))
    return dict(walls=walls, p99_ms=p99, p50_ms=_median(all_lat), total_bytes=total_bytes,
                blocks=[int(g.numel()) for g, _ in reqs], bit_exact=ok)


def _concurrent_pair(torch):
    """A put stream and a get stream that do not share a hardware queue."""
    from flexkv_amd.c_ext import streams_run_concurrently
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    spare = []
    while not streams_run_concurrently(a, b) and len(spare) < 8:
        spare.append(b)
        b = torch.cuda.Stream()
    return a, b, spare


def run_two_way(torch, device, num_cta):
    """Puts next to gets, the situations the link arbiter is there for (one
    process unless said otherwise; Llama-3-8B vLLM blocks of 2 MiB):
    request streams of several sizes, a large transfer that starts 1 ms after one
    of the other direction, a layerwise restore next to a put loop and one that
    puts interrupt, and a get loop next to the put loop of another process."""
    import subprocess
    import threading
    from flexkv_amd.c_ext import LayerwiseTransferGroup
    res = {}
    # every transfer stays on the stream it is issued on (read at the first transfer)
    os.environ.setdefault("FKV_LANE_STREAMS", "0")
    w = Workload("c4", torch, device)
    w.transfer(w.gpu_ids, w.cpu_ids, False, transfer_num_cta=num_cta, sync=True)
    sp, sg, _keep = _concurrent_pair(torch)
    block = w.L * w.kv_dim * w.chunk

    def streams_of(sizes_put, sizes_get):
        reqs, off = [], 0
        for a, b in zip(sizes_put, sizes_get):
            reqs.append((w.gpu_ids[off:off + a].contiguous(), w.cpu_ids[off:off + a].contiguous(), False))
            off += a
            reqs.append((w.gpu_ids[off:off + b].contiguous(), w.cpu_ids[off:off + b].contiguous(), True))
            off += b
        best = 1e9
        for _ in range(4):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for g, c, h2d in reqs:
                with torch.cuda.stream(sg if h2d else sp):
                    w.transfer(g, c, h2d=h2d, transfer_num_cta=num_cta, sync=False)
            torch.cuda.synchronize()
            best = min(best, time.perf_counter() - t0)
        return round(off * block / best / 1e9, 2)

    res["request_streams_GBps"] = {
        "1 x 1500 blocks per direction": streams_of([1500], [1500]),
        "4 x 375": streams_of([375] * 4, [375] * 4),
        "16 x 94": streams_of([94] * 16, [94] * 16),
        "125 x 12": streams_of([12] * 125, [12] * 125)}

    def second_starts_later(n, first_h2d):
        a = (w.gpu_ids[:n].contiguous(), w.cpu_ids[:n].contiguous())
        b = (w.gpu_ids[n:2 * n].contiguous(), w.cpu_ids[n:2 * n].contiguous())
        best = 1e9
        for _ in range(4):
            time.sleep(0.05)   # the first launch finds the link idle
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            with torch.cuda.stream(sg if first_h2d else sp):
                w.transfer(*a, h2d=first_h2d, transfer_num_cta=num_cta, sync=False)
            time.sleep(0.001)
            with torch.cuda.stream(sp if first_h2d else sg):
                w.transfer(*b, h2d=not first_h2d, transfer_num_cta=num_cta, sync=False)
            torch.cuda.synchronize()
            best = min(best, time.perf_counter() - t0)
        return round(2 * n * block / best / 1e9, 2)

    res["second_direction_starts_1ms_later_GBps"] = {
        "put first, 400 blocks each": second_starts_later(400, False),
        "get first, 400 blocks each": second_starts_later(400, True),
        "put first, 1500 blocks each": second_starts_later(1500, False),
        "get first, 1500 blocks each": second_starts_later(1500, True)}

    # a get loop next to the put loop of another process (94 blocks = 197 MB per request)
    n = 94
    g, c = w.gpu_ids[:n].contiguous(), w.cpu_ids[:n].contiguous()

    def loop(h2d, seconds):
        k, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            w.transfer(g, c, h2d=h2d, transfer_num_cta=num_cta, sync=True)
            k += 1
        return k * n * block / (time.perf_counter() - t0) / 1e9
    alone = loop(True, 1.0)
    child = subprocess.Popen([sys.executable, os.path.abspath(__file__), "--config", "twoway",
                              "--role", "putter"], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                             text=True)
    try:
        assert child.stdout.readline().strip() == "ready"
        child.stdin.write("\n")
        child.stdin.flush()
        time.sleep(0.3)
        gets = loop(True, 2.0)
        puts = float(child.stdout.readline())
    finally:
        child.wait(120)
    res["two_processes_GBps"] = {"gets_alone": round(alone, 2), "gets": round(gets, 2),
                                 "puts_of_the_other_process": round(puts, 2),
                                 "sum": round(gets + puts, 2)}
    del w
    torch.cuda.empty_cache()

    # a layerwise restore (MLA, 61 layers x 18 MiB for 256 blocks) next to puts
    w = Workload("c3", torch, device)
    w.transfer(w.gpu_ids, w.cpu_ids, False, transfer_num_cta=num_cta, sync=True)
    i64 = lambda v: torch.tensor([v], dtype=torch.int64)
    grp = LayerwiseTransferGroup(
        num_gpus=1, gpu_blocks=[w.tensors], cpu_blocks=w.host, ssd_files={}, num_layers=w.L,
        gpu_kv_strides_tensor=i64(w.gks), gpu_block_strides_tensor=i64(w.gbs),
        gpu_layer_strides_tensor=i64(w.gls), gpu_chunk_sizes_tensor=i64(w.chunk),
        iouring_entries=0, iouring_flags=0,
        layer_eventfds_tensor=torch.empty(0, dtype=torch.int32), tp_size=1, is_blockfirst=True)
    empty = torch.empty(0, dtype=torch.int64)
    half = w.num_blocks // 2
    gi, ci = w.gpu_ids[:half].contiguous(), w.cpu_ids[:half].contiguous()
    pg, pc = w.gpu_ids[half:half + 128].contiguous(), w.cpu_ids[half:half + 128].contiguous()
    rbytes = half * w.L * w.kv_dim * w.chunk

    def enqueue_restore():
        grp.layerwise_transfer(empty, empty, 0, 0, 0, 0, 0, gi, ci, w.cks, w.cls, w.cbs, w.chunk,
                               w.cks, w.cls, w.cbs, num_cta, False, w.L, 1, w.kv_dim, 1,
                               counter_id=0, kv_shared_across_ranks_mode="sharded",
                               notify_mode="polling")

    def restore():
        enqueue_restore()
        grp.synchronize()
    for _ in range(2):
        restore()
    t0 = time.perf_counter()
    restore()
    restore_alone = rbytes / (time.perf_counter() - t0) / 1e9
    go, stop, moved = threading.Event(), threading.Event(), [0, 0.0]

    def putter():
        with torch.cuda.stream(torch.cuda.Stream()):
            go.wait()
            t0 = time.perf_counter()
            while not stop.is_set():
                w.transfer(pg, pc, h2d=False, transfer_num_cta=num_cta, sync=True)
                moved[0] += 128 * w.L * w.kv_dim * w.chunk
            moved[1] = time.perf_counter() - t0
    th = threading.Thread(target=putter)
    th.start()
    go.set()
    time.sleep(0.05)
    t0 = time.perf_counter()
    for _ in range(5):
        restore()
    dt = time.perf_counter() - t0
    stop.set()
    th.join()
    res["restore_next_to_a_put_loop_GBps"] = {"restore_alone": round(restore_alone, 2),
                                              "restore": round(5 * rbytes / dt / 1e9, 2),
                                              "puts": round(moved[0] / moved[1] / 1e9, 2)}
    # The whole restore is enqueued on an idle link; the puts start 5 ms later.  Streams
    # that share a hardware queue with the restore's stream wait for it instead of
    # running next to it, so four put streams are tried: the longest restore is the one
    # that was interrupted.
    tries = []
    for _ in range(4):
        go.clear()
        stop.clear()
        th = threading.Thread(target=putter)
        th.start()
        time.sleep(0.1)
        t0 = time.perf_counter()
        enqueue_restore()
        time.sleep(0.005)
        go.set()
        grp.synchronize()
        tries.append(time.perf_counter() - t0)
        stop.set()
        th.join()
    dt = max(tries)
    res["puts_start_5ms_into_a_restore"] = {"restore_GBps": round(rbytes / dt / 1e9, 2),
                                            "restore_ms": round(dt * 1e3, 2),
                                            "restore_alone_ms": round(rbytes / restore_alone / 1e6, 2),
                                            "all_tries_ms": [round(t * 1e3, 2) for t in tries]}
    grp.close()
    return res


def run_neighbour(torch, device, num_cta, n=2048, count=150):
    """What a transfer costs a compute kernel that runs next to it: the time of
    one n^3 bf16 GEMM (150 in a row on a stream of their own) alone, next to a
    one-thread spin kernel, next to kernel transfers of either direction, and next
    to pinned copies of the copy engines."""
    w = Workload("c0", torch, device)
    w.transfer(w.gpu_ids, w.cpu_ids, False, transfer_num_cta=num_cta, sync=True)
    comp, other, _keep = _concurrent_pair(torch)
    a = torch.randn(n, n, device=device, dtype=torch.bfloat16)
    b = torch.randn(n, n, device=device, dtype=torch.bfloat16)
    c = torch.empty(n, n, device=device, dtype=torch.bfloat16)
    big_h = torch.empty(1 << 30, dtype=torch.uint8, pin_memory=True)
    big_d = torch.empty(1 << 30, dtype=torch.uint8, device=device)

    def case(background):
        torch.cuda.synchronize()
        if background:
            with torch.cuda.stream(other):
                background()
        time.sleep(0.002)
        with torch.cuda.stream(comp):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record(comp)
            for _ in range(count):
                torch.matmul(a, b, out=c)
            e.record(comp)
        e.synchronize()
        still_running = not other.query()
        torch.cuda.synchronize()
        return {"us_per_gemm": round(s.elapsed_time(e) / count * 1e3, 1),
                "background_outlasted_the_gemms": still_running}
    xfer = lambda h2d, cta, reps: (lambda: [w.transfer(w.gpu_ids, w.cpu_ids, h2d,
                                                       transfer_num_cta=cta, sync=False)
                                            for _ in range(reps)])
    for _ in range(2):
        case(None)
    return {
        "alone": case(None),
        "next to a one-thread spin kernel": case(lambda: torch.cuda._sleep(int(2.4e9 * 0.05))),
        "next to a host->GPU kernel transfer": case(xfer(True, num_cta, 3)),
        "next to a GPU->host kernel transfer": case(xfer(False, num_cta, 3)),
        "next to a host->GPU kernel transfer, transfer_num_cta=1": case(xfer(True, 1, 1)),
        "next to pinned hipMemcpyAsync host->GPU": case(
            lambda: [big_d.copy_(big_h, non_blocking=True) for _ in range(3)]),
        "next to pinned hipMemcpyAsync GPU->host": case(
            lambda: [big_h.copy_(big_d, non_blocking=True) for _ in range(3)])}


def run_groups(torch, device, num_cta, reps=30):
    """Whole-block ops of a model with layer groups of different chunk size (a latent
    group of 18 KiB chunks, a sliding-window group of 2.25 KiB, an indexer group of
    2 KiB): one transfer_kv_blocks call per group, as the reference's worker issues
    them, against one transfer_kv_blocks_multi call; then single groups of chunk
    sizes around 16 KiB, of which only some are a whole number of 8 KiB slices."""
    from flexkv_amd.c_ext import get_stats, reset_stats, transfer_kv_blocks, transfer_kv_blocks_multi
    pool = 1024

    class Group:
        def __init__(self, layers, chunk):
            self.layers, self.chunk = layers, chunk
            self.gpu = [torch.randint(0, 256, (pool, chunk), dtype=torch.uint8, device=device)
                        for _ in range(layers)]
            self.host = torch.zeros((pool, layers, chunk), dtype=torch.uint8).pin_memory()
            self.ptrs = torch.tensor([t.data_ptr() for t in self.gpu], dtype=torch.int64)

        def call(self, gids, cids, h2d, sync):
            c = self.chunk
            return ((gids, self.ptrs, pool * c, c, pool * c, cids, self.host, c, c, self.layers * c,
                     c, 0, self.layers),
                    dict(transfer_num_cta=num_cta, is_host_to_device=h2d, kv_dim=1, sync=sync))

        def check(self, gids, cids):
            for l in (0, self.layers - 1):
                if not torch.equal(self.host[cids, l], self.gpu[l][gids.to(device)].cpu()):
                    return False
            return True

    def timed(fn):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        reset_stats()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        dt = (time.perf_counter() - t0) / reps
        return dt, get_stats()["kernel_launches"] / reps

    res = {"one_op_of_three_groups": {}, "one_group_alone": {}}
    exact = True
    groups = [Group(30, 18432), Group(31, 2304), Group(30, 2048)]
    g = torch.Generator().manual_seed(3)
    for nblk in (64, 512):
        gids = torch.randperm(pool, generator=g)[:nblk].contiguous()
        cids = torch.randperm(pool, generator=g)[:nblk].contiguous()
        nbytes = sum(nblk * x.layers * x.chunk for x in groups)
        for h2d in (False, True):
            def per_group():
                for i, x in enumerate(groups):
                    a, k = x.call(gids, cids, h2d, i == len(groups) - 1)
                    transfer_kv_blocks(*a, **k)

            def together():
                transfer_kv_blocks_multi([x.call(gids, cids, h2d, True) for x in groups])
            for name, fn in (("one call per group", per_group), ("one call", together)):
                dt, launches = timed(fn)
                if not h2d:
                    exact = exact and all(x.check(gids, cids) for x in groups)
                res["one_op_of_three_groups"][
                    f"{nblk} blocks {'host->GPU' if h2d else 'GPU->host'}, {name}"] = {
                        "GBps": round(nbytes / dt / 1e9, 2), "us": round(dt * 1e6, 1),
                        "launches": launches}
    del groups
    gids = torch.randperm(pool, generator=g)[:512].contiguous()
    cids = torch.randperm(pool, generator=g)[:512].contiguous()
    for chunk in (16384, 18432, 20480, 9216, 12288):
        x = Group(30, chunk)
        for h2d in (False, True):
            a, k = x.call(gids, cids, h2d, True)
            dt, _ = timed(lambda: transfer_kv_blocks(*a, **k))
            if not h2d:
                exact = exact and x.check(gids, cids)
            res["one_group_alone"][f"30 layers x 512 blocks x {chunk} B "
                                   f"{'host->GPU' if h2d else 'GPU->host'}"] = \
                round(512 * 30 * chunk / dt / 1e9, 2)
        del x
    res["bit_exact"] = exact
    return res


def run_two_way_putter(torch, device, num_cta):
    """The other process of run_two_way: waits for a line on stdin, puts 94-block
    requests for 3 s and prints its rate."""
    w = Workload("c0", torch, device)
    n = 94
    g, c = w.gpu_ids[:n].contiguous(), w.cpu_ids[:n].contiguous()
    w.transfer(g, c, False, transfer_num_cta=num_cta, sync=True)
    print("ready", flush=True)
    sys.stdin.readline()
    k, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < 3.0:
        w.transfer(g, c, h2d=False, transfer_num_cta=num_cta, sync=True)
        k += 1
    print(f"{k * n * w.L * w.kv_dim * w.chunk / (time.perf_counter() - t0) / 1e9:.2f}", flush=True)


def run_notify_scales(torch, device, num_cta, iters=20, warmup=3):
    """Layerwise host->GPU restore end to end (call + device synchronize) at the
    three scales of the reference's notify-mode microbenchmark
    (benchmarks/microbenchmark_notify_mode.py:28-33, 87-147): MLA fp16, 16 tokens
    x 512 dims per block, layer_granularity 1, one GPU, no eventfd consumer."""
    from flexkv_amd.c_ext import LayerwiseTransferGroup
    scales = {"small": (8, 16), "medium": (32, 64), "large": (80, 256)}
    out = {}
    for name, (L, N) in scales.items():
        chunk = 16 * 512 * 2
        full = torch.zeros((L, 1, N, 16, 1, 512), dtype=torch.float16, device=device)
        gpu = [full[i] for i in range(L)]
        cpu = torch.zeros((N, L, 1, 16, 1, 512), dtype=torch.float16, pin_memory=True)
        i64 = lambda v: torch.tensor([v], dtype=torch.int64)
        ids = torch.arange(N, dtype=torch.int64)
        empty = torch.empty(0, dtype=torch.int64)
        row = {"bytes": L * N * chunk}
        for use_ce in (False, True):
            grp = LayerwiseTransferGroup(
                num_gpus=1, gpu_blocks=[gpu], cpu_blocks=cpu, ssd_files={}, num_layers=L,
                gpu_kv_strides_tensor=i64(N * chunk), gpu_block_strides_tensor=i64(chunk),
                gpu_layer_strides_tensor=i64(N * chunk), gpu_chunk_sizes_tensor=i64(chunk),
                iouring_entries=0, iouring_flags=0,
                layer_eventfds_tensor=torch.empty(0, dtype=torch.int32), tp_size=1,
                is_blockfirst=True)
            for notify in ("hostfunc", "polling"):
                ts = []
                for it in range(warmup + iters):
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    grp.layerwise_transfer(empty, empty, 0, 0, 0, 0, 0, ids, ids, chunk, chunk,
                                           L * chunk, chunk, chunk, chunk, L * chunk, num_cta,
                                           use_ce, L, 1, 1, 1, notify_mode=notify)
                    torch.cuda.synchronize()
                    if it >= warmup:
                        ts.append((time.perf_counter() - t0) * 1e3)
                key = ("ce_" if use_ce else "kernel_") + notify + "_p50_ms"
                row[key] = round(_median(ts), 4)
            grp.close()
        out[name] = row
    return out


# ---------------------------------------------------------------------------
# CPU baseline: the reference's CPU path (torch index-gather into the host
# cache layout), timed on this machine's host cores on a bounded sample.
# ---------------------------------------------------------------------------
def run_multi_group(torch, device, steps, warmup, num_cta, notify, use_ce, verify=True):
    """Layer groups of different shape restored layer by layer, one notification per
    original layer: members of every group attached to the layer, then its sidecar."""
    from flexkv_amd.c_ext import LayerwiseTransferGroup
    from flexkv_amd.layout import (KVCacheLayout, KVCacheLayoutType, LayerGroupSpec,
                                   MultiGroupBlockLayout, TransferStrides, multi_group_tables)
    t = torch
    L, page, n_gpu, n_cpu, nblk = 61, 256, 2048, 512, 512
    swa_tok, swa_width, swa_gpu, swa_cpu, nswa = 128, 1152, 256, 64, 64
    c4_layers = tuple(l for l in range(L) if l % 2 == 1)            # 30 layers, ratio 4
    c128_layers = tuple(l for l in range(L) if l % 2 == 0)          # 31 layers, ratio 128
    groups = [LayerGroupSpec(len(c4_layers), 1, 576, c4_layers, 2, 4),
              LayerGroupSpec(len(c128_layers), 1, 576, c128_layers, 2, 128),
              LayerGroupSpec(len(c4_layers), 1, 128, c4_layers, 1, 4)]  # indexer, one byte/elem
    cl = MultiGroupBlockLayout(n_cpu, page, tuple(groups), kv_dim=1)
    gls = [KVCacheLayout(KVCacheLayoutType.LAYERFIRST, g.num_layers, n_gpu,
                         page // g.compress_ratio, 1, g.head_size, kv_dim=1) for g in groups]
    tables = multi_group_tables(cl, L, [[x] for x in gls])
    gen = t.Generator(device=device).manual_seed(6)
    gpu = [[t.randint(0, 256, (n_gpu, page // g.compress_ratio, 1, g.head_size * g.itemsize),
                      device=device, dtype=t.uint8, generator=gen) for _ in range(g.num_layers)]
           for g in groups]
    host = t.randint(0, 256, (n_cpu, cl.get_block_stride()), dtype=t.uint8).pin_memory()
    scl = KVCacheLayout(KVCacheLayoutType.LAYERFIRST, L, swa_cpu, swa_tok, 1, swa_width, kv_dim=1)
    sgl = KVCacheLayout(KVCacheLayoutType.LAYERFIRST, L, swa_gpu, swa_tok, 1, swa_width, kv_dim=1)
    sc, sg = TransferStrides.from_layout(scl, 1), TransferStrides.from_layout(sgl, 1)
    swa_host = t.randint(0, 256, scl.kv_shape, dtype=t.uint8).pin_memory()
    swa_dev = [t.zeros((swa_gpu, swa_tok, 1, swa_width), device=device, dtype=t.uint8)
               for _ in range(L)]
    i64 = lambda v: t.tensor([v], dtype=t.int64)
    grp = LayerwiseTransferGroup(
        num_gpus=1, gpu_blocks_per_group=[[x] for x in gpu], cpu_blocks=host, ssd_files={},
        num_original_layers=L, layer_members=tables["layer_members"], iouring_entries=0,
        iouring_flags=0, layer_eventfds_tensor=t.empty(0, dtype=t.int32), tp_size=1,
        is_blockfirst=True, has_swa=True, swa_gpu_blocks=[swa_dev], swa_cpu_blocks=swa_host,
        swa_gpu_kv_strides_tensor=i64(sg.kv), swa_gpu_block_strides_tensor=i64(sg.block),
        swa_gpu_layer_strides_tensor=i64(sg.layer), swa_gpu_chunk_sizes_tensor=i64(sg.chunk),
        **{k: v for k, v in tables.items() if k.startswith("group_")})
    gg = t.Generator().manual_seed(6)
    gpu_ids = t.randperm(n_gpu, generator=gg)[:nblk].to(t.int64)
    cpu_ids = t.randperm(n_cpu, generator=gg)[:nblk].to(t.int64)
    swa_g = t.randperm(swa_gpu, generator=gg)[:nswa].to(t.int64)
    swa_c = t.randperm(swa_cpu, generator=gg)[:nswa].to(t.int64)
    empty = t.empty(0, dtype=t.int64)

    def restore():
        grp.layerwise_transfer_multi_group(
            empty, empty, 0, 1, 4, gpu_ids, cpu_ids, num_cta, use_ce, 1, 1, swa_h2d_src=swa_c,
            swa_h2d_dst=swa_g, swa_h2d_cpu_kv_stride_in_bytes=sc.kv,
            swa_h2d_cpu_layer_stride_in_bytes=sc.layer, swa_cpu_block_stride_in_bytes=sc.block,
            notify_mode=notify)
        grp.synchronize()

    for _ in range(warmup):
        restore()
    walls, last_layer = [], []
    for _ in range(steps):
        t.cuda.synchronize()
        t0 = time.perf_counter()
        restore()
        walls.append(time.perf_counter() - t0)
        last_layer.append(grp.batch_times_ms()[-1])
    main_bytes = sum(tables["group_chunk_sizes"][gi] * g.num_layers for gi, g in enumerate(groups)) \
        * nblk
    swa_bytes = L * nswa * sc.chunk
    ok = None
    if verify:
        ok = True
        st = cl.get_group_strides()
        gi_dev = gpu_ids.to(device)
        for gi, g in enumerate(groups):
            for l in range(g.num_layers):
                o = st[gi]["offset_bytes"] + l * st[gi]["layer_stride"]
                want = host[:, o:o + st[gi]["chunk_size"]].index_select(0, cpu_ids).to(device)
                got = gpu[gi][l].reshape(n_gpu, -1).index_select(0, gi_dev)
                ok = ok and bool(t.equal(want, got))
        for l in range(L):
            want = swa_host[l, 0].reshape(swa_cpu, -1).index_select(0, swa_c).to(device)
            ok = ok and bool(t.equal(want, swa_dev[l].reshape(swa_gpu, -1)
                                     .index_select(0, swa_g.to(device))))
    launches = sum(len(m) for m in tables["layer_members"]) + L
    grp.close()
    return {"wall_s": _median(walls), "device_ms": _median(last_layer), "bytes": main_bytes + swa_bytes,
            "main_bytes": main_bytes, "swa_bytes": swa_bytes, "bit_exact": ok,
            "copies_per_restore": launches, "layers": L,
            "desc": ("61 layers; groups: 30 x [2048,64,576] bf16 (ratio 4), 31 x [2048,2,576] bf16 "
                     "(ratio 128), 30 x [2048,64,128] u8 indexer; sidecar 61 x [256,128,1152] u8; "
                     "512 blocks + 64 sidecar slots, page 256")}


def run_worker_process(torch, device, steps, warmup, num_cta, use_ce, overlap=False):
    """c0-shaped put and get ops through a GPUCPUTransferWorker in its own process:
    what the pipe, the shared op pool and the completion queue add to a transfer.
    Then 8 puts and 8 gets of 64 blocks each, submitted together: one after the
    other, or gets next to puts when the worker overlaps the directions."""
    import numpy as np
    import torch.multiprocessing as mp
    from flexkv_amd.layout import KVCacheLayout, KVCacheLayoutType
    from flexkv_amd.transfer import trace
    from flexkv_amd.transfer.memory_handle import TensorSharedHandle
    from flexkv_amd.transfer.op_pool import SharedOpPool
    from flexkv_amd.transfer.ops import TransferOp, TransferType
    from flexkv_amd.transfer.worker import GPUCPUTransferWorker, PinnedPoolHandle
    os.environ["FLEXKV_TRANSFER_TRACE"] = "1"   # the worker reports its own timings
    trace.configure(True)
    t = torch
    # 1024 engine blocks: every shared allocation stays far below 2 GiB
    L, N, T, H, D, NH, n = 32, 1024, 16, 8, 128, 1024, 256
    gen = t.Generator(device=device).manual_seed(0)
    tensors = [t.randn(2, N, T, H, D, device=device, dtype=t.bfloat16, generator=gen)
               for _ in range(L)]
    gl = KVCacheLayout(KVCacheLayoutType.LAYERFIRST, L, N, T, H, D, kv_dim=2, num_kv_heads=H)
    cl = KVCacheLayout(KVCacheLayoutType.BLOCKFIRST, L, NH, T, H, D, kv_dim=2, num_kv_heads=H)
    ctx = mp.get_context("spawn")
    q = ctx.Queue()
    pool = SharedOpPool(64, 1024)
    h = GPUCPUTransferWorker.create_worker(
        ctx, q, pool.get_buffer(), [TensorSharedHandle(x) for x in tensors],
        PinnedPoolHandle(cl.kv_shape, t.bfloat16), gl, cl, t.bfloat16, 0,
        use_ce_transfer_h2d=use_ce, use_ce_transfer_d2h=use_ce, transfer_num_cta_h2d=num_cta,
        transfer_num_cta_d2h=num_cta, overlap_directions=overlap)
    h.wait_ready(300)
    gg = t.Generator().manual_seed(1)
    gpu_ids = t.randperm(N, generator=gg)[:n].numpy().astype(np.int64)
    cpu_ids = t.randperm(NH, generator=gg)[:n].numpy().astype(np.int64)
    nbytes = n * L * 2 * T * H * D * 2
    rec = {"D2H": [], "H2D": []}
    t_all = None
    for it in range(warmup + steps):
        if it == warmup:
            t_all = time.perf_counter()
        for kind, src, dst in ((TransferType.D2H, gpu_ids, cpu_ids),
                               (TransferType.H2D, cpu_ids, gpu_ids)):
            op = TransferOp(it, kind, src, dst)
            op.src_slot_id = pool.allocate_slot(src, 1 if kind == TransferType.D2H else 2)
            op.dst_slot_id = pool.allocate_slot(dst, 2 if kind == TransferType.D2H else 1)
            t0 = time.perf_counter()
            h.submit_transfer(op)
            op_id, ok, m = q.get(timeout=300)
            e2e = (time.perf_counter() - t0) * 1e3
            assert ok and op_id == op.op_id
            pool.free_slot(op.src_slot_id)
            pool.free_slot(op.dst_slot_id)
            if it >= warmup:
                rec[kind.value].append((e2e, m["xfer_ms"], m["ipc_ms"], m["wait_ms"]))
    wall = time.perf_counter() - t_all
    # mixed traffic: puts from engine blocks [0, 512) to host [0, 512), gets from host
    # [512, 1024) to engine blocks [512, 1024), 64 blocks per op, all submitted at once
    m_ops, m_blocks = 8, 64
    mixed_bytes = 2 * m_ops * m_blocks * L * 2 * T * H * D * 2
    mixed = []
    for it in range(warmup + steps):
        ops = []
        for k in range(m_ops):
            a = np.arange(k * m_blocks, (k + 1) * m_blocks, dtype=np.int64)
            for kind, src, dst in ((TransferType.D2H, a, a), (TransferType.H2D, a + 512, a + 512)):
                op = TransferOp(1000 + it, kind, src, dst)
                op.src_slot_id = pool.allocate_slot(src, 1 if kind == TransferType.D2H else 2)
                op.dst_slot_id = pool.allocate_slot(dst, 2 if kind == TransferType.D2H else 1)
                ops.append(op)
        t0 = time.perf_counter()
        for op in ops:
            h.submit_transfer(op)
        done = [q.get(timeout=300) for _ in ops]
        dt = time.perf_counter() - t0
        assert all(d[1] for d in done) and sorted(d[0] for d in done) == sorted(o.op_id for o in ops)
        for op in ops:
            pool.free_slot(op.src_slot_id)
            pool.free_slot(op.dst_slot_id)
        if it >= warmup:
            mixed.append(dt)
    h.shutdown()
    med = lambda xs: _median(list(xs))
    res = {"bytes_per_op": nbytes, "wall_s": wall, "exit_code": h.process.exitcode,
           "mixed": {"ops": 2 * m_ops, "blocks_per_op": m_blocks, "bytes": mixed_bytes,
                     "overlap_directions": bool(overlap),
                     "ms": round(med(mixed) * 1e3, 3),
                     "GBps": round(mixed_bytes / med(mixed) / 1e9, 3)}}
    for k, rows in rec.items():
        res[k] = {"e2e_ms": round(med(r[0] for r in rows), 3),
                  "worker_xfer_ms": round(med(r[1] for r in rows), 3),
                  "pipe_ms": round(med(r[2] for r in rows), 3),
                  "queue_wait_ms": round(med(r[3] for r in rows), 3),
                  "GBps_e2e": round(nbytes / (med(r[0] for r in rows) * 1e-3) / 1e9, 3),
                  "GBps_in_worker": round(nbytes / (med(r[1] for r in rows) * 1e-3) / 1e9, 3)}
    return res


def run_layout_transform(torch, device, steps, warmup, shape, verify=True):
    """Engine blocks <-> dense device buffer, both in HBM: the re-layout step of a
    direct-storage read or write (csrc/gds/layout_transform.cu), all blocks of a
    request in one call.  Times both directions with events on the current stream
    and a plain device copy of the same bytes as the yardstick."""
    import numpy as np
    from flexkv_amd.c_ext import layout_transform
    shapes = {  # name: (layers, kv_dim, pool blocks, blocks moved, chunk bytes, description)
        "c0": (32, 2, 4096, 2048, 32768, "32 x [2,4096,16,8,128] bf16, 2048 random blocks"),
        "c3": (61, 1, 2048, 1024, 73728, "61 x [1,2048,64,576] bf16 (MLA), 1024 random blocks"),
    }
    L_, K, N, nb, C, desc = shapes[shape]
    g = torch.Generator(device="cpu").manual_seed(5)
    tensors = [torch.randint(0, 256, (K, N, C), dtype=torch.uint8, device=device) for _ in range(L_)]
    ptrs = torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64)
    ids = torch.randperm(N, generator=g)[:nb]
    block = L_ * K * C
    buf = torch.zeros(nb * block, dtype=torch.uint8, device=device)
    B = nb * block
    args = (buf, K * C, C, block, C, ptrs, N * C, C, K * N * C, ids, L_, K)
    ev = lambda: torch.cuda.Event(enable_timing=True)
    res = {}
    for name, to_target in (("to_buffer", False), ("to_engine", True)):
        times = []
        for it in range(warmup + steps):
            a, b = ev(), ev()
            a.record()
            layout_transform(*args, to_target)
            b.record()
            b.synchronize()
            if it >= warmup:
                times.append(a.elapsed_time(b))
        res[name + "_ms"] = _median(times)
    other = torch.empty_like(buf)
    times = []
    for it in range(warmup + steps):
        a, b = ev(), ev()
        a.record()
        other.copy_(buf)
        b.record()
        b.synchronize()
        if it >= warmup:
            times.append(a.elapsed_time(b))
    res["plain_copy_ms"] = _median(times)
    ok = None
    if verify:
        layout_transform(*args, False)
        view = buf.view(nb, L_, K, C)
        di = ids.to(device)
        ok = all(torch.equal(view[:, l], tensors[l].index_select(1, di).transpose(0, 1))
                 for l in range(L_))
        back = torch.randperm(N, generator=g)[:nb]
        for t in tensors:
            t.index_fill_(1, back.to(device), 0)
        layout_transform(buf, K * C, C, block, C, ptrs, N * C, C, K * N * C, back, L_, K, True)
        ok = ok and all(torch.equal(tensors[l].index_select(1, back.to(device)).transpose(0, 1),
                                    view[:, l]) for l in range(L_))
    res.update(bytes=B, desc=desc, bit_exact=ok)
    return res


def run_ssd(torch, steps, warmup, ssd_dir, blocks, pinned):
    """Host pool <-> SSD files in the shape of the reference's SSD microbenchmark
    (benchmarks/microbenchmark_ssd_simulation.py): "small" MHA preset, both pool
    layouts, contiguous and scattered block ids, both directions, chunk-at-a-time
    requests (ssd_io_opt off) against coalesced ones, threads against io_uring."""
    import ctypes
    import mmap
    import shutil
    import tempfile
    import numpy as np
    from flexkv_amd import _lib
    from flexkv_amd.c_ext import SSDIOCTX, transfer_kv_blocks_ssd
    from flexkv_amd.layout import KVCacheLayout, KVCacheLayoutType, TransferStrides
    L_, H, D, T, KV, ES = 32, 8, 128, 16, 2, 2
    n_cpu, n_ssd, nfiles = blocks + blocks // 4, 2 * blocks, 4
    lib = _lib.load()
    work = tempfile.mkdtemp(prefix="fkv_ssd_bench_", dir=ssd_dir)
    rng = np.random.default_rng(1)
    out = {"cases": [], "dir": work}
    try:
        for kind in ("BLOCKFIRST", "LAYERFIRST"):
            cl = KVCacheLayout(KVCacheLayoutType[kind], L_, n_cpu, T, H, D, kv_dim=KV, num_kv_heads=H)
            fl = KVCacheLayout(KVCacheLayoutType[kind], L_, n_ssd, T, H, D, kv_dim=KV,
                               num_kv_heads=H).div_block(nfiles, padding=True)
            c, f = TransferStrides.from_layout(cl, ES), TransferStrides.from_layout(fl, ES)
            pool_bytes = cl.get_total_elements() * ES
            if pinned:
                pool_t = torch.empty(pool_bytes, dtype=torch.uint8, pin_memory=True)
                pool = pool_t.numpy()
            else:
                keep = mmap.mmap(-1, pool_bytes)
                pool = np.frombuffer(keep, dtype=np.uint8)
            pool[:] = rng.integers(0, 256, pool_bytes, dtype=np.uint8)
            paths = {0: [os.path.join(work, f"{kind}_{i}.bin") for i in range(nfiles)]}
            for p in paths[0]:
                with open(p, "wb") as fh:
                    fh.truncate(fl.get_total_elements() * ES)
            nbytes = blocks * L_ * KV * c.chunk
            for order in ("contiguous", "scattered"):
                if order == "contiguous":
                    ssd_ids, cpu_ids = np.arange(blocks), np.arange(blocks)
                else:
                    ssd_ids, cpu_ids = rng.permutation(n_ssd)[:blocks], rng.permutation(n_cpu)[:blocks]
                s_t, c_t = torch.from_numpy(ssd_ids.astype(np.int64)), torch.from_numpy(cpu_ids.astype(np.int64))
                for opt in (False, True):
                    rows = lib.fkv_ssd_plan(1, nfiles, 0, L_, s_t.data_ptr(), c_t.data_ptr(), blocks,
                                            c.layer, c.kv, f.layer, f.kv, c.chunk, c.block, 1, KV,
                                            int(opt), None, 0)
                    buf = np.zeros((rows, 5), dtype=np.int64)
                    lib.fkv_ssd_plan(1, nfiles, 0, L_, s_t.data_ptr(), c_t.data_ptr(), blocks,
                                     c.layer, c.kv, f.layer, f.kv, c.chunk, c.block, 1, KV,
                                     int(opt), buf.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), rows)
                    requests = int(buf[:, 0].max()) + 1
                    for entries in (0, 512):
                        ctx = SSDIOCTX(paths, 1, entries, 0)
                        rec = {"layout": kind, "order": order, "ssd_io_opt": opt,
                               "engine": "io_uring" if ctx.uses_iouring else "threads",
                               "requests": requests, "iovecs": int(rows)}
                        for name, is_read in (("write", False), ("read", True)):
                            times = []
                            for it in range(warmup + steps):
                                t0 = time.perf_counter()
                                transfer_kv_blocks_ssd(
                                    ctx, torch.arange(0, L_, dtype=torch.int32), pool.ctypes.data,
                                    s_t, c_t, c.layer, c.kv, f.layer, f.kv, c.chunk, c.block,
                                    is_read, n_ssd // nfiles, 1, 16, KV, opt)
                                if it >= warmup:
                                    times.append(time.perf_counter() - t0)
                            rec[name + "_GBps"] = round(nbytes / _median(times) / 1e9, 3)
                        rec["o_direct"] = ctx.last_transfer_was_direct
                        ctx.close()
                        out["cases"].append(rec)
            for p in paths[0]:
                os.unlink(p)
            del pool
        out["bytes_per_direction"] = nbytes
    finally:
        shutil.rmtree(work, ignore_errors=True)
    return out


def cpu_baseline(cfg, budget_s=20.0):
    import torch
    from oracle import fkv_oracle as O
    T, H, D = (64, 8, 128) if cfg == "c1" else (16, 8, 128)
    L, N, n, NH = 4, 4096, (1024 if cfg == "c1" else 256), 1024
    # vLLM-shaped [kv, N, T, H, D] tensors in host RAM; for the SGLang config a
    # page is the same 64x8x128 row block, K and V planes of a layer stacked.
    layers = [torch.empty(2, N, T, H, D, dtype=torch.bfloat16) for _ in range(L)]
    for i, x in enumerate(layers):
        x.view(torch.int16).copy_(
            (torch.arange(x.numel(), dtype=torch.int32) * (2 * i + 3)).to(torch.int16).view(x.shape))
    host = torch.zeros(NH, L, 2, T, H, D, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(7)
    gi = torch.randperm(N, generator=g)[:n]
    ci = torch.randperm(NH, generator=g)[:n]
    nbytes = 2 * n * L * 2 * T * H * D * 2  # gather + scatter
    O.torch_index_gather(layers, host, gi, ci)
    O.torch_index_scatter(layers, host, gi, ci)
    t_start, reps, best = time.perf_counter(), 0, float("inf")
    while True:
        t0 = time.perf_counter()
        O.torch_index_gather(layers, host, gi, ci)
        O.torch_index_scatter(layers, host, gi, ci)
        dt = time.perf_counter() - t0
        best = min(best, dt)
        reps += 1
        if time.perf_counter() - t_start > budget_s or reps >= 200:
            break
    elapsed = time.perf_counter() - t_start
    threads = torch.get_num_threads()
    torch.set_num_threads(1)
    t1, reps1 = time.perf_counter(), 0
    while time.perf_counter() - t1 < budget_s / 4 or reps1 < 1:
        O.torch_index_gather(layers, host, gi, ci)
        O.torch_index_scatter(layers, host, gi, ci)
        reps1 += 1
    one_thread = nbytes * reps1 / (time.perf_counter() - t1) / 1e9
    torch.set_num_threads(threads)
    return {"value": round(nbytes * reps / elapsed / 1e9, 3), "best": round(nbytes / best / 1e9, 3),
            "one_thread": round(one_thread, 3),
            "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": (f"{L} of 32 layers, {n} blocks of {T}x{H}x{D} bf16 K+V out of a {N}-block "
                       f"pool, torch index_select/index_copy_ gather into the block-first host "
                       f"cache then scatter back, {reps} repetitions ({elapsed:.1f} s), "
                       f"os.cpu_count()={os.cpu_count()}")}


# ---------------------------------------------------------------------------
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", default="c1", choices=["c0", "c1", "c2", "c3", "c4", "copycal", "notify", "mg", "worker", "ssd", "transform", "twoway", "neighbour", "groups"])
    ap.add_argument("--gemm-n", type=int, default=2048, help="neighbour: size of the GEMM")
    ap.add_argument("--role", default="", help=argparse.SUPPRESS)
    ap.add_argument("--shape", default="c0", choices=["c0", "c3"],
                    help="transform: which engine shape to re-lay out")
    ap.add_argument("--streams-per-direction", type=int, default=32,
                    help="c4: streams the 32 puts (and the 32 gets) are spread over")
    ap.add_argument("--ssd-dir", default=None,
                    help="ssd: directory for the cache files (default: the system temp dir)")
    ap.add_argument("--ssd-blocks", type=int, default=256,
                    help="ssd: 2 MiB blocks per transfer")
    ap.add_argument("--pageable-pool", action="store_true",
                    help="ssd: page-aligned ordinary memory for the host pool instead of pinned")
    ap.add_argument("--num-cta", type=int, default=4,
                    help="transfer_num_cta (reference default FLEXKV_TRANSFER_NUM_CTA_*=4)")
    ap.add_argument("--use-ce", action="store_true", help="copy-engine path instead of the kernel")
    ap.add_argument("--notify", default="polling", choices=["polling", "hostfunc"])
    ap.add_argument("--dummy", default="sdpa", choices=["sdpa", "gemm", "gemm4k", "elementwise"],
                    help="c3: the per-layer compute kernel the restore is overlapped with")
    ap.add_argument("--overlap-directions", action="store_true",
                    help="worker: the worker runs gets next to puts (second thread and stream)")
    ap.add_argument("--layer-spans", action="store_true",
                    help="c3: time every layer's compute with its own pair of events "
                         "(the events themselves slow the compute stream down)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the transfer path crosses one host "
              "link per GPU and has no cross-GPU step); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import flexkv_amd.c_ext as c_ext  # fails loudly if libfkv_hip.so is missing
    if args.config == "ssd":  # host pool <-> files: no GPU work in this one
        pinned = torch.cuda.is_available() and not args.pageable_pool
        r = run_ssd(torch, args.steps, args.warmup, args.ssd_dir, args.ssd_blocks, pinned)
        best = max(r["cases"], key=lambda x: x["read_GBps"])
        print(json.dumps({
            "metric": "host pool <-> SSD files GB/s (best read case)", "unit": "GB/s",
            "value": best["read_GBps"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8",
            "data": "synthetic",
            "config": {"workload": f"ssd: 32 layers x K+V x 32 KiB chunks (16 tok x 8 heads x 128 "
                                   f"bf16), {args.ssd_blocks} blocks of 2 MiB per transfer, 1 "
                                   f"device x 4 files, 16 threads or a 512-entry ring",
                       "host_pool": "pinned" if pinned else "pageable, page-aligned"},
            "bytes_per_direction": r["bytes_per_direction"], "cases": r["cases"]}))
        return
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    device = "cuda:0"
    torch.cuda.set_device(0)

    if args.config == "copycal":
        # Plain device-to-device copies of a known size: the yardstick the
        # FETCH_SIZE / WRITE_SIZE counters of the transfer kernel are scaled by.
        n = 1 << 30
        src = torch.randint(0, 256, (n,), device=device, dtype=torch.uint8)
        dst = torch.empty_like(src)
        for _ in range(max(1, args.steps)):
            dst.copy_(src)                         # runtime blit kernel
            torch.bitwise_or(src, 0, out=dst)      # elementwise kernel, reads n and writes n bytes
        torch.cuda.synchronize()
        print(json.dumps({"config": {"workload": "copycal"}, "copy_bytes": n,
                          "copies_of_each_kind": max(1, args.steps)}))
        return
    if args.config == "neighbour":
        res = run_neighbour(torch, device, args.num_cta, n=args.gemm_n)
        print(json.dumps({
            "metric": "time of a bf16 GEMM next to a transfer", "unit": "us",
            "value": res["next to a host->GPU kernel transfer"]["us_per_gemm"], "n_gpus": 1,
            "higher_is_better": False, "data": "synthetic", "vs_baseline": None,
            "config": {"workload": f"neighbour: {args.gemm_n}^3 bf16 GEMM x150 next to c0-shaped "
                                   "transfers of 512 MiB", "transfer_num_cta": args.num_cta},
            "results": res}))
        return
    if args.config == "groups":
        res = run_groups(torch, device, args.num_cta)
        print(json.dumps({
            "metric": "whole-block op of a multi-group model: GB/s host->GPU", "unit": "GB/s",
            "value": res["one_op_of_three_groups"]["512 blocks host->GPU, one call"]["GBps"],
            "n_gpus": 1, "higher_is_better": True, "dtype": "u8", "data": "synthetic",
            "vs_baseline": None, "bit_exact": res["bit_exact"],
            "config": {"workload": "groups: 30 layers x 18432 B + 31 x 2304 B + 30 x 2048 B per "
                                   "block, 64 and 512 blocks; single groups of 9-20 KiB chunks",
                       "transfer_num_cta": args.num_cta},
            "results": res}))
        return
    if args.config == "twoway":
        if args.role == "putter":
            run_two_way_putter(torch, device, args.num_cta)
            return
        bidir = measure_link_bidirectional(torch, device)
        res = run_two_way(torch, device, args.num_cta)
        print(json.dumps({
            "metric": "puts next to gets: GB/s in sum over the host link",
            "unit": "GB/s", "value": res["request_streams_GBps"]["16 x 94"], "n_gpus": 1,
            "higher_is_better": True, "dtype": "u8", "data": "synthetic", "vs_baseline": None,
            "config": {"workload": "twoway: Llama-3-8B vLLM blocks of 2 MiB (request streams, "
                                   "late second direction, two processes); MLA restore of 256 "
                                   "blocks x 61 layers next to puts",
                       "transfer_num_cta": args.num_cta},
            "bidir_link_peak_GBps": round(bidir, 3), "results": res}))
        return
    if args.config == "notify":
        res = run_notify_scales(torch, device, args.num_cta)
        print(json.dumps({
            "metric": "layerwise H2D end-to-end ms (p50) by notify mode and scale",
            "unit": "ms", "n_gpus": 1, "higher_is_better": False, "data": "synthetic",
            "config": {"workload": "notify: MLA fp16, 16 tok x 512 dim blocks; small 8 layers x 16 "
                                   "blocks, medium 32 x 64, large 80 x 256; layer_granularity 1"},
            "results": res,
            "reference_published_ms": {  # docs/flexkv_config_reference/README_en.md:119
                "hardware": "NVIDIA 8x GPU, kernel engine, 8 GPUs transferring at once",
                "small": {"hostfunc": 0.60, "polling": 0.40},
                "medium": {"hostfunc": 4.39, "polling": 1.87},
                "large": {"hostfunc": 16.79, "polling": 16.62}}}))
        return
    if args.config == "transform":
        r = run_layout_transform(torch, device, args.steps, args.warmup, args.shape,
                                 verify=not args.no_verify)
        avg_ms = (r["to_buffer_ms"] + r["to_engine_ms"]) / 2
        achieved = 2 * r["bytes"] / (avg_ms * 1e-3) / 1e9    # bytes read + bytes written
        plain = 2 * r["bytes"] / (r["plain_copy_ms"] * 1e-3) / 1e9
        print(json.dumps({
            "metric": "engine blocks <-> dense device buffer, GB/s of HBM traffic (read + write)",
            "unit": "GB/s", "value": round(achieved, 1), "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(avg_ms, 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": f"transform-{args.shape}: " + r["desc"]},
            "to_buffer_ms": round(r["to_buffer_ms"], 4), "to_engine_ms": round(r["to_engine_ms"], 4),
            "to_buffer_GBps": round(2 * r["bytes"] / (r["to_buffer_ms"] * 1e-3) / 1e9, 1),
            "to_engine_GBps": round(2 * r["bytes"] / (r["to_engine_ms"] * 1e-3) / 1e9, 1),
            "plain_device_copy_ms": round(r["plain_copy_ms"], 4),
            "plain_device_copy_GBps": round(plain, 1),
            "frac_of_plain_device_copy": round(achieved / plain, 4),
            "bytes_moved": r["bytes"], "bit_exact": r["bit_exact"],
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                         "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                         "traffic": MEASURED_TRAFFIC_BYTES.get(("transform-" + args.shape, "kernel")),
                         "kernel": "fkv_copy_chunks_kernel<16, true>",
                         "algorithmic_bytes_per_launch": 2 * r["bytes"],
                         "avg_launch_ms": round(avg_ms, 4)}}))
        return
    if args.config == "mg":
        link = measure_link()
        r = run_multi_group(torch, device, args.steps, args.warmup, args.num_cta, args.notify,
                            args.use_ce, verify=not args.no_verify)
        rate = r["bytes"] / (r["device_ms"] * 1e-3) / 1e9
        print(json.dumps({
            "metric": "multi-group layerwise restore GB/s (H2D) on 1 GPU", "unit": "GB/s",
            "value": round(rate, 3), "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(r["wall_s"] * 1e3, 3), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "mg: " + r["desc"], "notify": args.notify,
                       "path": "copy-engine" if args.use_ce else "kernel",
                       "transfer_num_cta": args.num_cta},
            "restore_device_ms": round(r["device_ms"], 3),
            "bytes": r["bytes"], "main_bytes": r["main_bytes"], "sidecar_bytes": r["swa_bytes"],
            "copies_per_restore": r["copies_per_restore"],
            "ms_per_original_layer": round(r["device_ms"] / r["layers"], 4),
            "h2d_frac_of_link": round(rate / link["h2d"], 4), "bit_exact": r["bit_exact"],
            "link_peak": {"h2d_GBps": round(link["h2d"], 3)}}))
        return
    if args.config == "worker":
        link = measure_link()
        r = run_worker_process(torch, device, args.steps, args.warmup, args.num_cta, args.use_ce,
                               overlap=args.overlap_directions)
        print(json.dumps({
            "metric": "put/get through a transfer worker process: GB/s seen by the submitter",
            "unit": "GB/s", "value": round(2 * r["bytes_per_op"] * args.steps / r["wall_s"] / 1e9, 3),
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(r["wall_s"] / args.steps * 1e3, 3), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "worker: c0 chunk shape (32 layers x [2,1024,16,8,128] bf16), "
                                   "256 random blocks per op, ids through the shared op pool, "
                                   "worker-owned pinned host pool",
                       "path": "copy-engine" if args.use_ce else "kernel",
                       "transfer_num_cta": args.num_cta},
            "put": r["D2H"], "get": r["H2D"], "bytes_per_op": r["bytes_per_op"],
            "puts_and_gets_submitted_together": r["mixed"],
            "worker_exit_code": r["exit_code"],
            "link_peak": {"d2h_GBps": round(link["d2h"], 3), "h2d_GBps": round(link["h2d"], 3)}}))
        return
    link = measure_link()
    w = Workload(args.config, torch, device)
    B = w.bytes_per_direction
    out = {"metric": METRIC, "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "u8", "data": "synthetic"}
    path_name = "copy-engine" if args.use_ce else "kernel"
    config = {"workload": f"{args.config}: {w.desc}", "path": path_name,
              "transfer_num_cta": args.num_cta, "blocks": w.num_blocks,
              "bytes_per_direction": B}

    if args.config in ("c0", "c1", "c2"):
        wall, d2h_ms, h2d_ms = run_gather_scatter(w, torch, args.steps, args.warmup, args.num_cta,
                                                  args.use_ce)
        taken = c_ext.last_transfer_path()
        d2h = B / (sum(d2h_ms) / len(d2h_ms) * 1e-3) / 1e9
        h2d = B / (sum(h2d_ms) / len(h2d_ms) * 1e-3) / 1e9
        out.update(value=round(2 * B * args.steps / wall / 1e9, 3),
                   ms_per_step=round(wall / args.steps * 1e3, 3),
                   d2h_GBps=round(d2h, 3), h2d_GBps=round(h2d, 3),
                   d2h_GiBps=round(d2h * 1e9 / 2**30, 3), h2d_GiBps=round(h2d * 1e9 / 2**30, 3),
                   d2h_frac_of_link=round(d2h / link["d2h"], 4),
                   h2d_frac_of_link=round(h2d / link["h2d"], 4))
        # dominant kernel: the gather/scatter kernel; one launch per direction moves B bytes
        avg_ms = (sum(d2h_ms) + sum(h2d_ms)) / (len(d2h_ms) + len(h2d_ms))
        achieved = B / (avg_ms * 1e-3) / 1e9
        kernel = "fkv_copy_chunks_kernel<16, false|true>" if not args.use_ce else taken
        out["roofline"] = {"bound": "hbm", "achieved": round(achieved, 3), "peak": HBM_PEAK_GBPS,
                           "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 5),
                           "traffic": MEASURED_TRAFFIC_BYTES.get((args.config, path_name)),
                           "kernel": kernel, "algorithmic_bytes_per_launch": B,
                           "avg_launch_ms": round(avg_ms, 4),
                           "limited_by": "host link (PCIe), not HBM",
                           "link_peak_GBps": round((link["d2h"] + link["h2d"]) / 2, 3),
                           "frac_of_link_peak": round(
                               achieved / ((link["d2h"] + link["h2d"]) / 2), 4)}
        config["path_taken"] = taken
        if not args.no_verify:
            out["bit_exact"] = verify_round_trip(w, torch, args.num_cta)
    elif args.config == "c3":
        # fill the host cache with the blocks to restore, then erase them on the GPU
        w.transfer(w.gpu_ids, w.cpu_ids, False, transfer_num_cta=args.num_cta, sync=True)
        gi = w.gpu_ids.to(device)
        saved = [w.gpu_rows(l, 0).index_select(0, gi) for l in range(w.L)]
        for l in range(w.L):
            w.gpu_rows(l, 0).index_fill_(0, gi, 0)
        r = run_layerwise(w, torch, args.steps, args.warmup, args.num_cta, args.notify, args.dummy,
                          layer_spans=args.layer_spans)
        restore = B / (r["restore_ms"] * 1e-3) / 1e9
        stall_beyond_first = max(0.0, r["stall_ms"] - r["first_layer_ms"])
        out.update(value=round(restore, 3), ms_per_step=round(r["total_ms"], 3),
                   h2d_GBps=round(restore, 3), h2d_frac_of_link=round(restore / link["h2d"], 4),
                   layerwise={"notify": args.notify, "dummy_compute": args.dummy,
                              "compute_units_per_layer": r["compute_reps_per_layer"],
                              "restore_alone_ms": round(r["restore_alone_ms"], 3),
                              "restore_alone_GBps": round(
                                  B / (r["restore_alone_ms"] * 1e-3) / 1e9, 3),
                              "restore_ms": round(r["restore_ms"], 3),
                              "first_layer_ms": round(r["first_layer_ms"], 3),
                              "compute_alone_ms": round(r["compute_ms"], 3),
                              "restore_plus_compute_ms": round(r["total_ms"], 3),
                              # the compute stream cannot finish before the last layer
                              # has landed and been computed on
                              "compute_tail_after_restore_ms": round(
                                  r["total_ms"] - r["restore_ms"], 3),
                              "compute_per_layer_ms": round(r["compute_ms"] / w.L, 3),
                              "layer_spans": bool(args.layer_spans),
                              "compute_stream_stall_ms": round(r["stall_ms"], 3),
                              "stall_beyond_first_layer_ms": round(stall_beyond_first, 3),
                              "overlap_frac_beyond_first_layer": round(
                                  1.0 - stall_beyond_first /
                                  max(1e-9, r["restore_ms"] - r["first_layer_ms"]), 4)})
        if args.layer_spans:
            out["layerwise"].update(
                compute_while_restoring_ms=round(r["compute_overlapped_ms"], 3),
                compute_slowdown=round(r["compute_overlapped_ms"] / r["compute_ms"], 3))
        if not args.no_verify:
            out["bit_exact"] = all(
                torch.equal(w.gpu_rows(l, 0).index_select(0, gi), saved[l]) for l in range(w.L))
        achieved = restore
        out["roofline"] = {"bound": "hbm", "achieved": round(achieved, 3), "peak": HBM_PEAK_GBPS,
                           "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 5),
                           "traffic": None, "kernel": "fkv_copy_chunks_kernel<16, true>",
                           "algorithmic_bytes_per_launch": r["layer_bytes"],
                           "limited_by": "host link (PCIe), not HBM",
                           "link_peak_GBps": round(link["h2d"], 3),
                           "frac_of_link_peak": round(achieved / link["h2d"], 4)}
    else:  # c4
        r = run_concurrent(w, torch, args.steps, args.warmup, args.num_cta,
                           args.streams_per_direction, verify=not args.no_verify)
        if r["bit_exact"] is not None:
            out["bit_exact"] = r["bit_exact"]
        bidir = measure_link_bidirectional(torch, device)
        agg = r["total_bytes"] / _median(r["walls"]) / 1e9
        out.update(value=round(agg, 3), ms_per_step=round(_median(r["walls"]) * 1e3, 3),
                   concurrent={"requests": 64, "streams_per_direction": args.streams_per_direction,
                               "total_blocks": sum(r["blocks"]),
                               "aggregate_bytes": r["total_bytes"],
                               "p50_latency_ms": round(r["p50_ms"], 3),
                               "p99_latency_ms": round(r["p99_ms"], 3),
                               "bidir_link_peak_GBps": round(bidir, 3),
                               "frac_of_bidir_link": round(agg / bidir, 4),
                               "frac_of_sum_of_one_way_peaks": round(
                                   agg / (link["d2h"] + link["h2d"]), 4)})
        out["roofline"] = {"bound": "hbm", "achieved": round(agg, 3), "peak": HBM_PEAK_GBPS,
                           "unit": "GB/s", "frac": round(agg / HBM_PEAK_GBPS, 5), "traffic": None,
                           "kernel": "fkv_copy_chunks_kernel<16, false|true>",
                           "limited_by": "host link (PCIe), both directions at once"}
    out["link_peak"] = {"d2h_GBps": round(link["d2h"], 3), "h2d_GBps": round(link["h2d"], 3),
                        "method": "1 GiB pinned hipMemcpyAsync x10, best, same run"}
    out["config"] = config
    if not args.no_cpu_baseline:
        del w
        torch.cuda.empty_cache()
        out["cpu_baseline"] = cpu_baseline(args.config)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
