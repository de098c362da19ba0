#!/usr/bin/env python3
"""Benchmark of the GPU<->CPU KV-block transfer path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config all|c0..c4|...]

A step is one pass of the hot path over one batch of block ids: a GPU->host
gather of the selected blocks into the host cache followed by the host->GPU
scatter of the same blocks (c0, c1, c2), one layer-by-layer restore (c3), or
one burst of 64 concurrent requests (c4).  Inputs are resident in HBM / pinned
host memory before the timed region starts.  One JSON line is printed.  Without
--config the line covers all five configurations: the headline fields (`value`, the
K timed steps) are c1's, and `configs` holds a record of each of c0..c4 with its own
GB/s, fraction of the link rate measured in the same run, bit-exactness and CPU
baseline on its own shape.

The five benchmark configurations:
  c0  Llama-3-8B, vLLM layout, bf16: 32 x [2,4096,16,8,128]; 256 random blocks
  c1  SGLang token-major, bf16, page 64: 64 x [262144,8,128]; 1024 pages
      (64 runs of 8 + 512 isolated)                      <- the headline of the default run
  c2  TRT-LLM layout, fp8 e4m3: [4096,80,2,8,32,128]; 2048 random blocks
  c3  DeepSeek-V3 MLA, bf16: 61 x [16384,64,576]; layerwise restore of 512 blocks
  c4  64 concurrent requests on the c0 shape with a 32768-block pool
Beyond those (the callers and formats either side of the path):
  mg      layerwise restore of heterogeneous layer groups + sliding-window sidecar
          (DeepSeek-V4-like: 61 layers, two compressed latent groups, an indexer group)
  worker  c0-shaped put/get ops through a transfer worker process (pipe + shared op pool)
  groups  whole-block ops of a model with three layer groups: one call per group against
          one call for all; chunk sizes that are no whole number of slices
Studies: --sequence CFG,CFG,... measures configurations of choice one behind the other in one
process (what one leaves behind for the next), --policy FIELD=VALUE sets a field of the
library's launch policy first, --hw-queues N the hardware queues of the process.
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
MEASURED_TRAFFIC_BYTES = {("c1", "kernel"): 8590410496, ("transform-c0", "kernel"): 8593325056}
TRAFFIC_SOURCE = {("c1", "kernel"): "profiles/fkv_copy_chunks_kernel_c1_pmc.md",
                  ("transform-c0", "kernel"): "profiles/fkv_copy_chunks_kernel_transform_c0.md"}


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
            self.backend, self.kv_dim, self.L, self.num_kv_heads = 0, 2, L, H
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
            self.backend, self.kv_dim, self.L, self.num_kv_heads = 2, 2, L, H
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
            self.backend, self.kv_dim, self.L, self.num_kv_heads = 1, 2, L, H
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
        elif name in ("c3", "c3f"):
            L, N, T, D = 61, 16384, 64, 576
            self.NH = 512 if name == "c3" else 4096
            self.desc = ("DeepSeek-V3 MLA latent KV bf16: 61 x [16384,64,576], layerwise restore of "
                         "512 blocks, host [%d,61,1,64,1,576]%s" % (
                             self.NH, "" if name == "c3" else
                             ", host block ids scattered over the pool (512 runs of one block)"))
            self.backend, self.kv_dim, self.L, self.num_kv_heads = 0, 1, L, 1
            self.chunk = T * D * 2
            gen = t.Generator(device=device).manual_seed(4)
            self.tensors = [(t.randn(N, T, D, device=device, dtype=t.bfloat16, generator=gen) * 0.5)
                            for _ in range(L)]
            self.num_gpu_blocks = N
            self.gks, self.gbs, self.gls = N * self.chunk, self.chunk, N * self.chunk
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

    def fragment_host_pool(self, pool_blocks=4096, seed=44):
        """c3 -> c3f in place: the same engine tensors and GPU blocks, a host pool of
        `pool_blocks` blocks and host block ids scattered over it."""
        t = self.torch
        self.name, self.NH = "c3f", pool_blocks
        self.desc = self.desc.replace("host [512,", "host [%d," % pool_blocks) + \
            ", host block ids scattered over the pool (512 runs of one block)"
        self.host = None
        release_cached_memory(t)
        self.host = t.empty(self.NH * self.cbs, dtype=t.uint8, pin_memory=True)
        gg = t.Generator().manual_seed(seed)
        self.cpu_ids = t.randperm(self.NH, generator=gg)[:self.num_blocks].to(t.int64)

    def transfer(self, gpu_ids, cpu_ids, h2d, **kw):
        from flexkv_amd.c_ext import transfer_kv_blocks
        kw.setdefault("sync", False)
        # the reference's workers pass the layout's head count (flexkv/transfer/worker.py:1020,
        # 1050); the copy-engine strategy tree reads it (csrc/ce_transfer.cu:71-104)
        kw.setdefault("num_kv_heads", self.num_kv_heads)
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


def release_cached_memory(torch):
    """Device memory and pinned host memory that torch keeps cached after a workload has
    gone: the next configuration (and a worker process that pins a pool of its own)
    needs the room."""
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    empty_host = getattr(torch._C, "_host_emptyCache", None)
    if empty_host is not None:
        empty_host()


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


def measure_hbm(device_index=0, nbytes=4 << 30, reps=10):
    """What HBM delivers to a streaming kernel on contiguous memory: read only, write
    only, copy (read + written bytes), GB/s, best of `reps`."""
    from flexkv_amd import _lib
    L = _lib.load()
    out = {}
    for name, mode in (("read_only", 0), ("write_only", 1), ("copy", 2)):
        best, med = ctypes.c_double(), ctypes.c_double()
        _lib.check(L.fkv_measure_hbm_rate(device_index, nbytes, reps, mode, ctypes.byref(best),
                                          ctypes.byref(med)))
        out[name + "_GBps"] = round(best.value, 1)
    r, w = out["read_only_GBps"], out["write_only_GBps"]
    # a copy moves half its bytes at the read rate and half at the write rate at best
    out["copy_bound_from_read_and_write_GBps"] = round(2.0 / (1.0 / r + 1.0 / w), 1)
    return out


def measure_link_bidirectional(torch, device, nbytes=1 << 30, reps=6):
    """Plain pinned copies in both directions at once (two streams), best of `reps`:
    the yardstick for puts running next to gets."""
    hd = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
    hu = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
    dd = torch.empty(nbytes, dtype=torch.uint8, device=device)
    du = torch.empty(nbytes, dtype=torch.uint8, device=device)
    # two streams that do not share a hardware queue (streams on one queue take turns)
    from flexkv_amd.c_ext import streams_run_concurrently
    s_up, s_down, spare = torch.cuda.Stream(), torch.cuda.Stream(), []
    while not streams_run_concurrently(s_up, s_down) and len(spare) < 8:
        spare.append(s_down)           # kept alive so that the next one is another stream
        s_down = torch.cuda.Stream()
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
        for k in range(steps):
            a, b, c = ev(), ev(), ev()
            a.record(st)
            w.transfer(w.gpu_ids, w.cpu_ids, False, **kw)
            b.record(st)
            w.transfer(reload_ids, w.cpu_ids, True, **kw)
            c.record(st)
            marks.append((a, b, c))
            # Copy-engine strategies queue hundreds of copy commands per step, and with some
            # 14 000 of them queued ahead (c0: 28 steps of 2 x 256 copies) the runtime runs the
            # GPU->host ones at half rate until the queue has drained.  No caller of the path
            # gets there (the workers wait for every op), so the benchmark does not either.
            if use_ce and k % 4 == 3:
                st.synchronize()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    for a, b, c in marks:
        d2h_ms.append(a.elapsed_time(b))
        h2d_ms.append(b.elapsed_time(c))
    # what a worker sees: host wall clock around one call with sync=True, per direction
    # (the reference's own method, benchmarks/benchmark_workers.py:524-556)
    sync_ms = {"d2h": [], "h2d": []}
    with torch.cuda.stream(st):
        for _ in range(min(steps, 5)):
            for name, ids, h2d in (("d2h", w.gpu_ids, False), ("h2d", reload_ids, True)):
                t1 = time.perf_counter()
                w.transfer(ids, w.cpu_ids, h2d, **dict(kw, sync=True))
                sync_ms[name].append((time.perf_counter() - t1) * 1e3)
    return wall, d2h_ms, h2d_ms, sync_ms


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
    # c2 reloads into another permutation of block ids; the others into the same blocks
    reload_ids = getattr(w, "gpu_ids_reload", w.gpu_ids)
    w.transfer(reload_ids, w.cpu_ids, True, transfer_num_cta=num_cta, sync=True)
    ri = reload_ids.to(w.device)
    for l in range(w.L):
        for kv in range(w.kv_dim):
            ok = ok and torch.equal(w.gpu_rows(l, kv).index_select(0, ri), saved[l][kv])
    return bool(ok)


def run_layerwise(w, torch, steps, warmup, num_cta, notify, dummy, layer_spans=False, use_ce=False,
                  name_compute_stream=True):
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
            w.cks, w.cls, w.cbs, num_cta, use_ce, w.L, 1, w.kv_dim, 1, counter_id=0,
            kv_shared_across_ranks_mode="sharded", notify_mode=notify)

    layer_bytes = w.num_blocks * w.kv_dim * w.chunk
    # Dummy per-layer compute on a second stream, sized to about one layer's copy
    # time: fused attention (default; what a restored layer feeds), a 2048^3 GEMM
    # chain, or a streaming elementwise kernel.
    comp = torch.cuda.Stream()
    # the engine names its forward stream: the group's own streams keep off its hardware queue
    t_name = time.perf_counter()
    sharing = grp.set_compute_stream(comp) if name_compute_stream else None
    naming_ms = (time.perf_counter() - t_name) * 1e3
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

    from flexkv_amd.c_ext import get_stats
    st0 = get_stats()
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
    st1 = get_stats()
    per = lambda k: (st1[k] - st0[k]) / (warmup + steps)
    staged, gathered = int(per("staged_batches")), int(per("gathered_batches"))
    route = (("copy-engine strategies (use_ce_transfer)" if use_ce else "kernel") if staged == 0 else
             "host threads gather each layer into a pinned buffer, one copy-engine command per "
             "layer, scatter launch%s" % (" (first layer by kernel)" if staged < w.L else "")
             if gathered else "copy engines, one command per run of host blocks, scatter launch")
    if use_ce and staged:
        route += " (asked for with use_ce_transfer)"
    return dict(staged_batches_per_restore=staged, gathered_batches_per_restore=gathered,
                gather_busy_ms_per_restore=round(per("gather_busy_us") / 1e3, 3), route=route,
                total_ms=_median(totals), restore_ms=_median(restores),
                first_layer_ms=_median(firsts), compute_ms=compute_ms,
                compute_overlapped_ms=_median(busy), stall_ms=_median(stalls),
                compute_reps_per_layer=reps, layer_bytes=layer_bytes,
                restore_alone_ms=restore_alone_ms,
                restore_alone_runs_ms=[round(x, 3) for x in alone],
                group_streams_on_compute_queue=sharing, naming_ms=round(naming_ms, 1))


def run_concurrent(w, torch, steps, warmup, num_cta, streams_per_direction=32, verify=True):
    """c4: 32 D2H puts and 32 H2D gets issued at once from 64 threads.  Each
    direction has its own set of streams (one per request by default); the
    process has a few hardware queues (GPU_MAX_HW_QUEUES: 4 by HIP's default, see
    --hw-queues), so with more streams per direction than half of them puts and gets
    also share queues and partly serialize."""
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

    starts = []     # per timed burst: when each request thread got to its call, sorted
    cores = []      # per timed burst: CPU time of the process / wall time

    def worker(i, barrier, record, began):
        gi, ci = reqs[i]
        with torch.cuda.stream(streams[i]):
            barrier.wait()
            t0 = time.perf_counter()
            w.transfer(gi, ci, h2d=(i % 2 == 1), transfer_num_cta=num_cta, sync=True)
            if record:
                lat[i].append((time.perf_counter() - t0) * 1e3)
            began[i] = t0

    for it in range(warmup + steps):
        barrier = threading.Barrier(len(reqs) + 1)
        began = [0.0] * len(reqs)
        threads = [threading.Thread(target=worker, args=(i, barrier, it >= warmup, began))
                   for i in range(len(reqs))]
        for th in threads:
            th.start()
        torch.cuda.synchronize()
        barrier.wait()
        t0 = time.perf_counter()
        cpu0 = time.process_time()
        for th in threads:
            th.join()
        if it >= warmup:
            walls.append(time.perf_counter() - t0)
            cores.append((time.process_time() - cpu0) / walls[-1])
            starts.append(sorted((b - t0) * 1e3 for b in began))
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
    from flexkv_amd.c_ext import get_stats
    st = get_stats()
    return dict(walls=walls, p99_ms=p99, p50_ms=_median(all_lat), total_bytes=total_bytes,
                blocks=[int(g.numel()) for g, _ in reqs], bit_exact=ok,
                # slots of the library's plan pool after the bursts, and how often a request
                # had to wait for the oldest user of one since the counters were last reset
                plan_memory={k: st[k] for k in ("plan_slots", "plan_slots_in_use", "plan_slot_waits")},
                # the 64 threads do not get to their calls at once: the interpreter hands its
                # lock from thread to thread.  Milliseconds after the start of a burst at which
                # half, nine tenths and all of them had made their call (medians over bursts).
                host_cores_busy=round(_median(cores), 2),   # of the whole process, during a burst
                call_starts_ms={"half": round(_median([s[len(s) // 2] for s in starts]), 2),
                                "nine_tenths": round(_median([s[len(s) * 9 // 10] for s in starts]), 2),
                                "all": round(_median([s[-1] for s in starts]), 2)})


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


def run_notify_scales(torch, device, num_cta, iters=20, warmup=3):
    """Layerwise host->GPU restore end to end (call + device synchronize) at the
    three scales of the reference's notify-mode microbenchmark
    (benchmarks/microbenchmark_notify_mode.py:28-33, 87-147): MLA fp16, 16 tokens
    x 512 dims per block, layer_granularity 1, one GPU, no eventfd consumer."""
    import flexkv_amd.c_ext as c_ext
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
                c_ext.reset_stats()
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
                st = c_ext.get_stats()
                if not use_ce and notify == "polling":   # which way the batches went
                    row["batches_through_copy_engines"] = st["staged_batches"] // (warmup + iters)
                    row["batches_on_second_stream"] = st["second_stream_batches"] // (warmup + iters)
            grp.close()
        out[name] = row
    return out


# ---------------------------------------------------------------------------
# CPU baseline: the reference's CPU path (torch index-gather into the host
# cache layout), timed on this machine's host cores on a bounded sample.
# ---------------------------------------------------------------------------
def run_multi_group(torch, device, steps, warmup, num_cta, notify, use_ce, verify=True,
                    fragmented=False):
    """Layer groups of different shape restored layer by layer, one notification per
    original layer: members of every group attached to the layer, then its sidecar."""
    from flexkv_amd.c_ext import LayerwiseTransferGroup
    from flexkv_amd.layout import (KVCacheLayout, KVCacheLayoutType, LayerGroupSpec,
                                   MultiGroupBlockLayout, TransferStrides, multi_group_tables)
    t = torch
    L, page, n_gpu, n_cpu, nblk = 61, 256, 2048, 512, 512
    swa_tok, swa_width, swa_gpu, swa_cpu, nswa = 128, 1152, 256, 64, 64
    if fragmented:   # host pools after churn: the blocks to restore are scattered over them
        n_cpu, swa_cpu = 4096, 512
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


def run_worker_process(torch, device, steps, warmup, num_cta, use_ce, overlap=False,
                       sweep_blocks=None, shuffle_ids=True):
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
    # one op at a time for a list of block counts, with the worker and its pool kept
    # (benchmarks/benchmark_workers.py --sweep-blocks / --shuffle-ids, :441-470)
    sweep = []
    for count in sweep_blocks or ():
        count = max(1, min(int(count), N))
        if shuffle_ids:
            g_ids = t.randperm(N, generator=gg)[:count].numpy().astype(np.int64)
            c_ids = t.randperm(NH, generator=gg)[:count].numpy().astype(np.int64)
        else:
            g_ids = c_ids = np.arange(count, dtype=np.int64)
        row = {"blocks": count, "bytes": count * L * 2 * T * H * D * 2, "shuffled_ids": bool(shuffle_ids)}
        for kind, src, dst, name in ((TransferType.D2H, g_ids, c_ids, "put"),
                                     (TransferType.H2D, c_ids, g_ids, "get")):
            e2e, inside = [], []
            for it in range(warmup + steps):
                op = TransferOp(2000 + it, kind, src, dst)
                op.src_slot_id = pool.allocate_slot(src, 1 if kind == TransferType.D2H else 2)
                op.dst_slot_id = pool.allocate_slot(dst, 2 if kind == TransferType.D2H else 1)
                t0 = time.perf_counter()
                h.submit_transfer(op)
                op_id, ok, m = q.get(timeout=300)
                dt = (time.perf_counter() - t0) * 1e3
                assert ok and op_id == op.op_id
                pool.free_slot(op.src_slot_id)
                pool.free_slot(op.dst_slot_id)
                if it >= warmup:
                    e2e.append(dt)
                    inside.append(m["xfer_ms"])
            row[name + "_e2e_ms"] = round(_median(e2e), 4)
            row[name + "_worker_xfer_ms"] = round(_median(inside), 4)
            row[name + "_GBps_e2e"] = round(row["bytes"] / (_median(e2e) * 1e-3) / 1e9, 3)
        sweep.append(row)
    h.shutdown()
    med = lambda xs: _median(list(xs))
    res = {"bytes_per_op": nbytes, "wall_s": wall, "exit_code": h.process.exitcode, "sweep": sweep,
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


def run_staging(torch, device, steps, warmup, num_cta):
    """Variable-size payloads between a dense device staging buffer and the host cache
    with a host-side size table (the device half of a compressed transfer around the
    codec): c0-shaped slots (32 layers x K+V x 32 KiB, 256 blocks = 16384 chunks), payload
    sizes uniform in 50-90 % of a slot.  GB/s of payload bytes, both directions."""
    import numpy as np
    from flexkv_amd.c_ext import staging_transfer
    L, K, NB, N, cap = 32, 2, 256, 1024, 32768
    total = L * K * NB
    g = torch.Generator().manual_seed(11)
    sizes_h = torch.randint(cap // 2, cap * 9 // 10, (total,), generator=g, dtype=torch.int64)
    sizes = sizes_h.to(device)
    staging = torch.randint(0, 256, (total * cap,), dtype=torch.uint8, device=device)
    host = torch.zeros(N * L * K * cap, dtype=torch.uint8, pin_memory=True)
    table = torch.zeros(N * L * K, dtype=torch.int32, pin_memory=True)
    ids = torch.randperm(N, generator=g)[:NB].to(torch.int64)
    overflow = torch.zeros(1, dtype=torch.int32, device=device)
    payload = int(sizes_h.sum())
    ev = lambda: torch.cuda.Event(enable_timing=True)

    def timed(write, sz):
        ms = []
        for it in range(warmup + steps):
            a, b = ev(), ev()
            a.record()
            staging_transfer(staging, cap, sz, host, cap, overflow, cap, K * cap, L * K * cap, ids,
                             table, L * K, K, 0, K, 0, total, write, transfer_num_cta=num_cta)
            b.record()
            b.synchronize()
            if it >= warmup:
                ms.append(a.elapsed_time(b))
        return _median(ms)
    write_ms = timed(True, sizes)
    want = staging.clone()
    staging.zero_()
    got_sizes = torch.zeros_like(sizes)
    read_ms = timed(False, got_sizes)
    # every payload came back, sizes restored from the table, nothing beyond a payload written
    idx = torch.arange(cap, device=device).unsqueeze(0) < sizes.unsqueeze(1)
    ok = bool(torch.equal(got_sizes, sizes)) and int(overflow.item()) == 0 and bool(
        torch.equal(staging.view(total, cap)[idx], want.view(total, cap)[idx])) and not bool(
        staging.view(total, cap)[~idx].any())
    return dict(write_ms=write_ms, read_ms=read_ms, payload_bytes=payload, chunks=total,
                bit_exact=ok)


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


def cpu_baseline(cfg, budget_s=5.0):
    """The reference's CPU path (torch index-gather into the block-first host cache
    and index-scatter back, oracle/fkv_oracle.py) on a bounded sample of the
    configuration's own shape, all host cores, then one thread."""
    import torch
    from oracle import fkv_oracle as O
    g = torch.Generator().manual_seed(7)

    def filled(*shape, dtype=torch.bfloat16):
        x = torch.empty(*shape, dtype=dtype)
        flat = x.view(torch.uint8).view(-1)
        pat = torch.randint(0, 255, (1 << 20,), dtype=torch.uint8, generator=g)  # finite fp8/bf16 bytes aside
        whole = flat.numel() // pat.numel() * pat.numel()
        flat[:whole].view(-1, pat.numel()).copy_(pat)
        flat[whole:].copy_(pat[:flat.numel() - whole])
        return x

    if cfg in ("c0", "c4"):
        L, N, T, H, D, NH = 4, 4096, 16, 8, 128, 1024
        layers = [filled(2, N, T, H, D) for _ in range(L)]
        host = torch.zeros(NH, L, 2, T, H, D, dtype=torch.bfloat16)
        if cfg == "c0":
            reqs = [(torch.randperm(N, generator=g)[:256], torch.randperm(NH, generator=g)[:256])]
            what = "256 blocks"
        else:
            sizes = torch.empty(64).geometric_(1.0 / 48, generator=g).clamp(1, 512).to(torch.int64)
            sizes = sizes[torch.cumsum(sizes, 0) <= NH]
            pg, pc = torch.randperm(N, generator=g), torch.randperm(NH, generator=g)
            offs = [0] + torch.cumsum(sizes, 0).tolist()
            reqs = [(pg[offs[i]:offs[i + 1]], pc[offs[i]:offs[i + 1]]) for i in range(len(sizes))]
            what = f"{len(reqs)} requests of {int(sizes.sum())} blocks in all, one after the other"
        n_blocks = sum(int(a.numel()) for a, _ in reqs)
        nbytes = 2 * n_blocks * L * 2 * T * H * D * 2

        def step():
            for i, (gi, ci) in enumerate(reqs):
                if cfg == "c0" or i % 2 == 0:
                    O.torch_index_gather(layers, host, gi, ci)
                if cfg == "c0" or i % 2 == 1:
                    O.torch_index_scatter(layers, host, gi, ci)
        if cfg == "c4":
            nbytes //= 2  # every request moves one way
        sample = (f"{L} of 32 layers, {what} of 16x8x128 bf16 K+V out of a {N}-block pool "
                  f"([2,N,16,8,128] per layer), gather into [NH,L,2,16,8,128] and scatter back")
    elif cfg == "c1":
        L, tokens, H, D, page, n = 4, 262144, 8, 128, 64, 1024
        N = tokens // page
        planes = [[filled(tokens, H, D).view(N, page, H, D) for _ in range(2)] for _ in range(L)]
        host = torch.zeros(n, L, 2, page, H, D, dtype=torch.bfloat16)
        gi = sglang_page_ids(torch, N, seed=2)
        ci = torch.arange(n)
        nbytes = 2 * n * L * 2 * page * H * D * 2

        def step():
            O.torch_index_gather_planes(planes, host, gi, ci)
            O.torch_index_scatter_planes(planes, host, gi, ci)
        sample = (f"{L} of 32 layers, 1024 pages (64 runs of 8 + 512 isolated) of 64x8x128 bf16 "
                  f"out of separate K and V tensors [262144,8,128], gather into "
                  f"[1024,L,2,64,8,128] and scatter back")
    elif cfg == "c2":
        N, L, H, T, D, n = 512, 80, 8, 32, 128, 256
        big = filled(N, L, 2, H, T, D, dtype=torch.uint8)
        host = torch.zeros(n, L, 2, H, T, D, dtype=torch.uint8)
        gi = torch.randperm(N, generator=g)[:n]
        gi2 = torch.randperm(N, generator=g)[:n]
        ci = torch.arange(n)
        nbytes = 2 * n * L * 2 * H * T * D

        def step():
            host.index_copy_(0, ci, big.index_select(0, gi))       # whole 5 MiB blocks
            big.index_copy_(0, gi2, host.index_select(0, ci))      # reload into another permutation
        sample = (f"{n} of 2048 blocks of [80,2,8,32,128] fp8 bytes out of a {N}-block pool, "
                  f"whole-block index_select into the host cache and index_copy_ back into another "
                  f"permutation")
    elif cfg in ("c3", "c3f"):
        L, N, T, D, n = 8, 2048, 64, 576, 512
        pool = n if cfg == "c3" else 4 * n   # c3f: host blocks scattered over a larger pool
        planes = [[filled(N, T, D)] for _ in range(L)]
        host = filled(pool, L, 1, T, D)
        gi = torch.randperm(N, generator=g)[:n]
        ci = torch.randperm(pool, generator=g)[:n]
        nbytes = n * L * T * D * 2

        def step():
            O.torch_index_scatter_planes(planes, host, gi, ci)     # the restore direction only
        sample = (f"{L} of 61 layers, 512 blocks of 64x576 bf16 (kv_dim 1) into a {N}-block pool "
                  f"per layer, index_select from the host cache [{pool},L,1,64,576] + index_copy_")
    else:
        raise ValueError(cfg)
    step()
    t_start, reps, best = time.perf_counter(), 0, float("inf")
    while True:
        t0 = time.perf_counter()
        step()
        best = min(best, time.perf_counter() - t0)
        reps += 1
        if time.perf_counter() - t_start > budget_s or reps >= 200:
            break
    elapsed = time.perf_counter() - t_start
    threads = torch.get_num_threads()
    torch.set_num_threads(1)
    t1, reps1 = time.perf_counter(), 0
    while time.perf_counter() - t1 < budget_s / 4 or reps1 < 1:
        step()
        reps1 += 1
    one_thread = nbytes * reps1 / (time.perf_counter() - t1) / 1e9
    torch.set_num_threads(threads)
    return {"value": round(nbytes * reps / elapsed / 1e9, 3), "best": round(nbytes / best / 1e9, 3),
            "one_thread": round(one_thread, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{sample}; {reps} repetitions ({elapsed:.1f} s), os.cpu_count()={os.cpu_count()}"}


def overlap_record(r, B, link):
    """The one definition of overlap used for the layerwise restore: `exposed_ms` is
    what restore and compute together take beyond the longer of the two alone;
    beyond the first layer (which nothing can hide: the compute has no input yet)
    it should be zero.  overlap_frac = 1 - exposed / the shorter of the two."""
    longer = max(r["restore_alone_ms"], r["compute_ms"])
    shorter = min(r["restore_alone_ms"], r["compute_ms"])
    exposed = max(0.0, r["total_ms"] - longer)
    beyond_first = max(0.0, exposed - r["first_layer_ms"])
    return {"restore_alone_ms": round(r["restore_alone_ms"], 3),
            "restore_alone_GBps": round(B / (r["restore_alone_ms"] * 1e-3) / 1e9, 3),
            "compute_alone_ms": round(r["compute_ms"], 3),
            "restore_plus_compute_ms": round(r["total_ms"], 3),
            "restore_next_to_compute_ms": round(r["restore_ms"], 3),
            "first_layer_ms": round(r["first_layer_ms"], 3),
            "restore_alone_runs_ms": r.get("restore_alone_runs_ms"),
            # after fkv_layerwise_set_compute_stream; None: the compute stream was not named
            "group_streams_on_compute_queue": r.get("group_streams_on_compute_queue"),
            "set_compute_stream_ms": r.get("naming_ms"),   # once, at set-up: the probes
            "compute_per_layer_ms": round(r["compute_ms"] / r["layers"], 3),
            "compute_units_per_layer": r["compute_reps_per_layer"],
            "exposed_ms": round(exposed, 3),
            "exposed_beyond_first_layer_ms": round(beyond_first, 3),
            "overlap_frac": round(1.0 - exposed / max(1e-9, shorter), 4),
            "overlap_frac_beyond_first_layer": round(1.0 - beyond_first / max(1e-9, shorter), 4),
            "fully_overlapped_beyond_first_layer": bool(
                r["total_ms"] <= 1.1 * longer + r["first_layer_ms"]),
            "staged_batches_per_restore": r.get("staged_batches_per_restore"),
            "gathered_batches_per_restore": r.get("gathered_batches_per_restore"),
            "host_gather_thread_ms_per_restore": r.get("gather_busy_ms_per_restore"),
            "route": r.get("route")}


def measure_config(name, args, torch, device, link, steps, warmup):
    """One of c0..c4 on the kernel path (or --use-ce): the fields of its record."""
    import flexkv_amd.c_ext as c_ext
    w = Workload(name, torch, device)
    B = w.bytes_per_direction
    path_name = "copy-engine" if args.use_ce else "kernel"
    out = {"workload": f"{name}: {w.desc}", "path": path_name, "transfer_num_cta": args.num_cta,
           "blocks": w.num_blocks, "bytes_per_direction": B, "steps": steps, "warmup": warmup}
    if name in ("c0", "c1", "c2"):
        wall, d2h_ms, h2d_ms, sync_ms = run_gather_scatter(w, torch, steps, warmup, args.num_cta,
                                                           args.use_ce)
        taken = c_ext.last_transfer_path()
        d2h = B / (sum(d2h_ms) / len(d2h_ms) * 1e-3) / 1e9
        h2d = B / (sum(h2d_ms) / len(h2d_ms) * 1e-3) / 1e9
        avg_ms = (sum(d2h_ms) + sum(h2d_ms)) / (len(d2h_ms) + len(h2d_ms))
        out.update(value=round(2 * B * steps / wall / 1e9, 3),
                   ms_per_step=round(wall / steps * 1e3, 3),
                   d2h_GBps=round(d2h, 3), h2d_GBps=round(h2d, 3),
                   d2h_GiBps=round(d2h * 1e9 / 2**30, 3), h2d_GiBps=round(h2d * 1e9 / 2**30, 3),
                   d2h_frac_of_link=round(d2h / link["d2h"], 4),
                   h2d_frac_of_link=round(h2d / link["h2d"], 4),
                   d2h_ms_median=round(_median(d2h_ms), 4), d2h_ms_min=round(min(d2h_ms), 4),
                   h2d_ms_median=round(_median(h2d_ms), 4), h2d_ms_min=round(min(h2d_ms), 4),
                   avg_launch_ms=round(avg_ms, 4), path_taken=taken,
                   d2h_ms_steps=[round(x, 3) for x in d2h_ms],
                   h2d_ms_steps=[round(x, 3) for x in h2d_ms],
                   sync_call_wall={
                       "what": "host wall clock around one call with sync=True, %d calls per "
                               "direction" % len(sync_ms["d2h"]),
                       "d2h_ms_median": round(_median(sync_ms["d2h"]), 4),
                       "d2h_ms_min": round(min(sync_ms["d2h"]), 4),
                       "h2d_ms_median": round(_median(sync_ms["h2d"]), 4),
                       "h2d_ms_min": round(min(sync_ms["h2d"]), 4),
                       "d2h_GBps": round(B / (_median(sync_ms["d2h"]) * 1e-3) / 1e9, 3),
                       "h2d_GBps": round(B / (_median(sync_ms["h2d"]) * 1e-3) / 1e9, 3)})
        if not args.no_verify:
            out["bit_exact"] = verify_round_trip(w, torch, args.num_cta)
    elif name in ("c3", "c3f"):
        out.update(measure_layerwise(w, args, torch, device, link, steps, warmup))
        if name == "c3" and getattr(args, "with_fragmented", False):
            # the same restore out of a host pool after churn: 4096 host blocks, ids scattered
            w.fragment_host_pool()
            frag = {"workload": f"c3f: {w.desc}", "transfer_num_cta": args.num_cta,
                    "blocks": w.num_blocks, "bytes_per_direction": B, "steps": steps,
                    "warmup": warmup}
            frag.update(measure_layerwise(w, args, torch, device, link, steps, warmup))
            # the same restore asked for on the copy engine, and out of a host pool the device
            # cannot read (ordinary pageable memory): both go through gathered rows as well
            variants = {}
            short = max(2, min(steps, 5))
            ce_args = argparse.Namespace(**{**vars(args), "use_ce": True})
            variants["with_use_ce_transfer"] = measure_layerwise(w, ce_args, torch, device, link,
                                                                 short, 2)
            pinned = w.host
            try:
                w.host = torch.empty(pinned.numel(), dtype=pinned.dtype)   # pageable
                w.host.copy_(pinned)
                variants["pageable_host_pool"] = measure_layerwise(w, ce_args, torch, device, link,
                                                                   short, 2, fill_host=False)
            finally:
                w.host = pinned
            frag["variants"] = {
                k: {"route": v["path"], "restore_alone_ms": v["layerwise"]["restore_alone_ms"],
                    "restore_alone_GBps": v["layerwise"]["restore_alone_GBps"],
                    "restore_plus_compute_ms": v["layerwise"]["restore_plus_compute_ms"],
                    "compute_alone_ms": v["layerwise"]["compute_alone_ms"],
                    "first_layer_ms": v["layerwise"]["first_layer_ms"],
                    "restore_alone_runs_ms": v["layerwise"].get("restore_alone_runs_ms"),
                    "host_gather_thread_ms_per_restore":
                        v["layerwise"].get("host_gather_thread_ms_per_restore"),
                    "bit_exact": v.get("bit_exact"), "steps": short}
                for k, v in variants.items()}
            out["fragmented_record"] = frag
    else:  # c4
        r = run_concurrent(w, torch, steps, warmup, args.num_cta, args.streams_per_direction,
                           verify=not args.no_verify)
        if r["bit_exact"] is not None:
            out["bit_exact"] = r["bit_exact"]
        bidir = link.get("bidir") or measure_link_bidirectional(torch, device)
        agg = r["total_bytes"] / _median(r["walls"]) / 1e9
        out.update(value=round(agg, 3), ms_per_step=round(_median(r["walls"]) * 1e3, 3),
                   aggregate_GBps=round(agg, 3), requests=64,
                   streams_per_direction=args.streams_per_direction,
                   hardware_queues=int(os.environ.get("GPU_MAX_HW_QUEUES", "4")),
                   total_blocks=sum(r["blocks"]), aggregate_bytes=r["total_bytes"],
                   p50_latency_ms=round(r["p50_ms"], 3), p99_latency_ms=round(r["p99_ms"], 3),
                   burst_ms=[round(x * 1e3, 2) for x in r["walls"]],   # every timed burst
                   plan_memory=r["plan_memory"], call_starts_ms=r["call_starts_ms"],
                   host_cores_busy=r["host_cores_busy"],
                   bidir_link_peak_GBps=round(bidir, 3), frac_of_bidir_link=round(agg / bidir, 4),
                   frac_of_sum_of_one_way_peaks=round(agg / (link["d2h"] + link["h2d"]), 4))
    del w
    release_cached_memory(torch)
    return out


def measure_layerwise(w, args, torch, device, link, steps, warmup, fill_host=True):
    """c3 / c3f: the fields of a layerwise-restore record.  `fill_host=False`: the host pool
    already holds the engine's blocks (a pageable copy of a pool filled before, which the
    kernel path could not write)."""
    import flexkv_amd.c_ext as c_ext
    B = w.bytes_per_direction
    # fill the host cache with the blocks to restore, then erase them on the GPU
    gi = w.gpu_ids.to(device)
    if fill_host:
        w.transfer(w.gpu_ids, w.cpu_ids, False, transfer_num_cta=args.num_cta, sync=True)
        saved = [w.gpu_rows(l, 0).index_select(0, gi) for l in range(w.L)]
    else:   # the engine's blocks are what an earlier restore out of the same bytes left
        saved = [w.gpu_rows(l, 0).index_select(0, gi) for l in range(w.L)]
    for l in range(w.L):
        w.gpu_rows(l, 0).index_fill_(0, gi, 0)
    c_ext.reset_stats()
    r = run_layerwise(w, torch, steps, warmup, args.num_cta, args.notify, args.dummy,
                      layer_spans=args.layer_spans, use_ce=args.use_ce)
    r["layers"] = w.L
    restore = B / (r["restore_ms"] * 1e-3) / 1e9
    pol = c_ext.get_launch_policy()
    out = dict(value=round(restore, 3), ms_per_step=round(r["total_ms"], 3),
               h2d_GBps=round(restore, 3), h2d_frac_of_link=round(restore / link["h2d"], 4),
               notify=args.notify, dummy_compute=args.dummy, layer_bytes=r["layer_bytes"],
               path=r["route"], layerwise=overlap_record(r, B, link))
    if r["gathered_batches_per_restore"]:
        out["layerwise"]["host_gather_threads"] = pol["gather_threads"]
    if args.layer_spans:
        out["layerwise"].update(
            compute_while_restoring_ms=round(r["compute_overlapped_ms"], 3),
            compute_slowdown=round(r["compute_overlapped_ms"] / r["compute_ms"], 3))
    if not args.no_verify:
        out["bit_exact"] = all(
            torch.equal(w.gpu_rows(l, 0).index_select(0, gi), saved[l]) for l in range(w.L))
    return out


def link_roofline(rec, link, traffic=None, traffic_source=None):
    """The contract's roofline object for the dominant kernel of a c0/c1/c2 record: the
    gather/scatter kernel against the published HBM peak, and against the roof that
    actually bounds it, the host link measured in the same run."""
    B = rec["bytes_per_direction"]
    achieved = B / (rec["avg_launch_ms"] * 1e-3) / 1e9
    peak_link = (link["d2h"] + link["h2d"]) / 2
    return {"bound": "hbm", "achieved": round(achieved, 3), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 5), "traffic": traffic,
            "traffic_source": (traffic_source + " (rocprofv3 --pmc runs of this script, not a "
                               "quantity of this run)") if traffic_source else None,
            "kernel": "fkv_copy_chunks_kernel<16, false, 8, true> (GPU->host), <16, true, 8, false> (host->GPU)",
            "algorithmic_bytes_per_launch": B, "avg_launch_ms": rec["avg_launch_ms"],
            "limited_by": "host link (PCIe), not HBM: one side of every copy is host memory",
            "link_peak_GBps": round(peak_link, 3),
            "frac_of_link_peak": round(achieved / peak_link, 4)}


# ---------------------------------------------------------------------------
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", default="all",
                    choices=["all", "c0", "c1", "c2", "c3", "c3f", "c4", "copycal", "notify", "mg", "worker",
                             "ssd", "transform", "groups", "staging"])
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
    ap.add_argument("--staged-restore", type=int, default=None, choices=[0, 1, 2],
                    help="c3: 0 keeps the restore on the kernel path, 1 lets the library choose "
                         "(default), 2 sends it through the copy engines whenever the layout allows")
    ap.add_argument("--staged-gather", type=int, default=None, choices=[0, 1, 2],
                    help="c3 / c3f: 0 never lets host threads gather the rows of a layer, 1 lets "
                         "the library choose (default), 2 whenever the run-by-run route is not taken")
    ap.add_argument("--gather-threads", type=int, default=None,
                    help="c3 / c3f: host threads that gather (default 6)")
    ap.add_argument("--gather-first-by-kernel", type=int, default=None, choices=[0, 1])
    ap.add_argument("--policy", action="append", default=[], metavar="FIELD=VALUE",
                    help="set a field of the launch policy (fkv_launch_policy) before the run; "
                         "may be given several times")
    ap.add_argument("--fragmented", action="store_true",
                    help="mg: host pools of 4096 / 512 blocks with the blocks to restore scattered "
                         "over them (default: pools of 512 / 64 blocks, all of them restored)")
    ap.add_argument("--sweep-blocks", default=None, metavar="N,N,...",
                    help="--config worker: also one put and one get at a time for each of these "
                         "block counts (at most 1024), worker and pool kept")
    ap.add_argument("--sequential-ids", action="store_true",
                    help="--sweep-blocks with block ids 0..n-1 on both sides instead of shuffled ones")
    ap.add_argument("--overlap-directions", action="store_true",
                    help="worker: the worker runs gets next to puts (second thread and stream)")
    ap.add_argument("--layer-spans", action="store_true",
                    help="c3: time every layer's compute with its own pair of events "
                         "(the events themselves slow the compute stream down)")
    ap.add_argument("--other-steps", type=int, default=10,
                    help="all: timed steps of the configurations next to the headline one "
                         "(3 warm-up steps each)")
    ap.add_argument("--hw-queues", type=int, default=0, choices=range(0, 33), metavar="0..32",
                    help="GPU_MAX_HW_QUEUES of this process (HIP's default is 4; 0, the default "
                         "here, leaves the environment as it is)")
    ap.add_argument("--sequence", default=None, metavar="CFG,CFG,...",
                    help="all: after the headline configuration measure only these, in this "
                         "order (NAME+ce: through the copy-engine strategies), without the "
                         "worker sub-record, and print them")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true")
    args = ap.parse_args()
    if args.sequence:
        known = {"c0", "c1", "c2", "c3", "c4"}
        bad = [n for n in args.sequence.split(",")
               if (n[:-3] if n.endswith("+ce") else n) not in known
               or (n.endswith("+ce") and n[:-3] not in ("c0", "c1", "c2"))]
        if bad:
            ap.error("--sequence: unknown configuration(s) %s (c0..c4, and c0+ce, c1+ce, c2+ce)"
                     % ", ".join(bad))
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the transfer path crosses one host "
              "link per GPU and has no cross-GPU step); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    # Hardware queues of the process: the runtime reads this when it starts.  HIP's default is
    # 4, the reference's platform gives a process 8 (CUDA_DEVICE_MAX_CONNECTIONS).  c4 reaches
    # the same 93 GB/s with 2, 4, 8 and 16, c3 its 42 ms with 4 and 8 once the group knows the
    # compute stream.  Left as the environment has it unless asked for.
    if args.hw_queues > 0:
        os.environ["GPU_MAX_HW_QUEUES"] = str(args.hw_queues)
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
    for item in args.policy:
        field, _, value = item.partition("=")
        c_ext.set_launch_policy(**{field.strip(): int(value, 0)})
    if args.staged_restore is not None:
        c_ext.set_launch_policy(staged_restore=args.staged_restore)
    if args.staged_gather is not None:
        c_ext.set_launch_policy(staged_gather=args.staged_gather)
    if args.gather_threads is not None:
        c_ext.set_launch_policy(gather_threads=args.gather_threads)
    if args.gather_first_by_kernel is not None:
        c_ext.set_launch_policy(gather_first_by_kernel=args.gather_first_by_kernel)

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
        print(json.dumps(transform_record(torch, device, args, args.steps, args.warmup)))
        return
    if args.config == "staging":
        link = measure_link()
        r = run_staging(torch, device, args.steps, args.warmup, args.num_cta)
        wr = r["payload_bytes"] / (r["write_ms"] * 1e-3) / 1e9
        rd = r["payload_bytes"] / (r["read_ms"] * 1e-3) / 1e9
        print(json.dumps({
            "metric": "compressed-staging payloads <-> host cache, GB/s of payload (to host, from host)",
            "unit": "GB/s", "value": round((wr + rd) / 2, 3), "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(r["write_ms"] + r["read_ms"], 3),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8",
            "data": "synthetic",
            "config": {"workload": "staging: 16384 slots of 32 KiB (32 layers x K+V x 256 blocks), "
                                   "payloads uniform in 16-29 KiB, block-first host cache, uint32 "
                                   "size table", "transfer_num_cta": args.num_cta},
            "to_host_GBps": round(wr, 3), "from_host_GBps": round(rd, 3),
            "to_host_frac_of_link": round(wr / link["d2h"], 4),
            "from_host_frac_of_link": round(rd / link["h2d"], 4),
            "payload_bytes": r["payload_bytes"], "chunks": r["chunks"], "bit_exact": r["bit_exact"],
            "link_peak": {"d2h_GBps": round(link["d2h"], 3), "h2d_GBps": round(link["h2d"], 3)}}))
        return
    if args.config == "mg":
        link = measure_link()
        c_ext.reset_stats()
        r = run_multi_group(torch, device, args.steps, args.warmup, args.num_cta, args.notify,
                            args.use_ce, verify=not args.no_verify, fragmented=args.fragmented)
        st = c_ext.get_stats()
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
            "host_blocks": "scattered over pools of 4096 / 512 blocks" if args.fragmented
                           else "all blocks of pools of 512 / 64 blocks (one run each)",
            "batches_through_copy_engines": st["staged_batches"],
            "batches_gathered_by_host_threads": st["gathered_batches"],
            "host_gather_thread_ms": round(st["gather_busy_us"] / 1e3, 3),
            "ms_per_original_layer": round(r["device_ms"] / r["layers"], 4),
            "h2d_frac_of_link": round(rate / link["h2d"], 4), "bit_exact": r["bit_exact"],
            "link_peak": {"h2d_GBps": round(link["h2d"], 3)}}))
        return
    if args.config == "worker":
        link = measure_link()
        counts = [int(x) for x in args.sweep_blocks.split(",")] if args.sweep_blocks else None
        r = run_worker_process(torch, device, args.steps, args.warmup, args.num_cta, args.use_ce,
                               overlap=args.overlap_directions, sweep_blocks=counts,
                               shuffle_ids=not args.sequential_ids)
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
            "sweep_blocks": r["sweep"],
            "worker_exit_code": r["exit_code"],
            "link_peak": {"d2h_GBps": round(link["d2h"], 3), "h2d_GBps": round(link["h2d"], 3)}}))
        return

    link = measure_link()
    if args.config in ("all", "c4"):
        # both directions at once, measured before anything else has created streams
        link["bidir"] = measure_link_bidirectional(torch, device)
    out = {"metric": METRIC, "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "u8", "data": "synthetic"}
    link_rec = {"d2h_GBps": round(link["d2h"], 3), "h2d_GBps": round(link["h2d"], 3),
                "method": "1 GiB pinned hipMemcpyAsync x10, best, same run"}
    if "bidir" in link:
        link_rec["both_directions_at_once_GBps"] = round(link["bidir"], 3)
    if args.config != "all":
        rec = measure_config(args.config, args, torch, device, link, args.steps, args.warmup)
        out.update(value=rec["value"], ms_per_step=rec["ms_per_step"])
        out.update({k: v for k, v in rec.items() if k not in ("workload", "path", "transfer_num_cta",
                                                              "blocks", "bytes_per_direction")})
        if "avg_launch_ms" in rec:
            key = (args.config, rec["path"])
            out["roofline"] = link_roofline(rec, link, MEASURED_TRAFFIC_BYTES.get(key),
                                            TRAFFIC_SOURCE.get(key))
        out["link_peak"] = link_rec
        out["config"] = {k: rec[k] for k in ("workload", "path", "transfer_num_cta", "blocks",
                                             "bytes_per_direction")}
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_baseline(args.config, budget_s=20.0)
        print(json.dumps(out))
        return

    # All five configurations in one line.  The headline (`value`, `ms_per_step`, the
    # K timed steps) is c1, the SGLang page-64 case: the first of the configurations
    # beyond the reference's own CPU-runnable one (c0), and the one that moves the
    # most bytes per step through the plain gather/scatter call (8 GiB each way).
    # c0, c2, c3 and c4 follow with `--other-steps` timed steps each.
    head = "c1"
    records = {}
    if not args.sequence:
        # c4 first (it used to be the one figure that moved with its place in the run: 64
        # waiting threads kept 13 of the box's 16 cores busy inside the runtime's waits, the
        # threads that still had to submit their request got to it up to 50 ms late, and how
        # late depended on what the process had done before; the library now lets only two
        # waiters wait that way).  `--sequence ...,c4` measures it behind configurations of
        # choice.
        records["c4"] = measure_config("c4", args, torch, device, link, 20, 1)
        records["c4"]["position_in_run"] = "first"
    records[head] = measure_config(head, args, torch, device, link, args.steps, args.warmup)

    def copy_engine_record(name, steps):
        # the same blocks through the copy-engine strategies (the library's choice among them)
        ce_args = argparse.Namespace(**{**vars(args), "use_ce": True, "no_verify": True})
        ce = measure_config(name, ce_args, torch, device, link, steps, 2)  # staging buffers are allocated in the first calls
        return {k: ce[k] for k in ("d2h_GBps", "h2d_GBps", "d2h_frac_of_link", "h2d_frac_of_link",
                                   "d2h_ms_median", "d2h_ms_min", "h2d_ms_median", "h2d_ms_min",
                                   "d2h_ms_steps", "h2d_ms_steps", "path_taken", "steps")}
    if not args.use_ce and not args.sequence:
        records[head]["copy_engine"] = copy_engine_record(head, min(3, args.steps))
    args.with_fragmented = True
    if args.sequence:   # a study of what one configuration leaves behind for the next
        for name in args.sequence.split(","):
            if name.endswith("+ce"):   # the same blocks through the copy-engine strategies
                records[name + "_in_sequence"] = copy_engine_record(name[:-3], min(5, args.other_steps))
                continue
            records[name + "_in_sequence"] = measure_config(
                name, args, torch, device, link, 20 if name == "c4" else args.other_steps,
                1 if name == "c4" else 3)
            records[name + "_in_sequence"].pop("fragmented_record", None)
        print(json.dumps({"sequence": args.sequence, "configs": records}))
        return
    for name in ("c0", "c2", "c3"):
        records[name] = measure_config(name, args, torch, device, link, args.other_steps, 3)
        if name in ("c0", "c2") and not args.use_ce:
            records[name]["copy_engine"] = copy_engine_record(name, min(5, args.other_steps))
    records["c3_fragmented"] = records["c3"].pop("fragmented_record")
    # one c0-shaped op at a time through a spawned transfer worker: submit -> completion on
    # the submitter's wall clock, 1 warm-up + 10 rounds (benchmarks/benchmark_workers.py:524-556)
    wk = run_worker_process(torch, device, 10, 1, args.num_cta, args.use_ce)
    records["c0"]["through_worker"] = {
        "what": "256-block put and get ops (536870912 B each) submitted one at a time to a "
                "GPUCPUTransferWorker process with a 1024-block engine pool; wall clock from "
                "submit to completion, median of 10",
        "put": wk["D2H"], "get": wk["H2D"], "worker_exit_code": wk["exit_code"]}
    rec = records[head]
    out.update(value=rec["value"], ms_per_step=rec["ms_per_step"],
               d2h_GBps=rec["d2h_GBps"], h2d_GBps=rec["h2d_GBps"],
               d2h_frac_of_link=rec["d2h_frac_of_link"], h2d_frac_of_link=rec["h2d_frac_of_link"],
               bit_exact=all(r.get("bit_exact", True) for r in records.values()))
    out["roofline"] = link_roofline(rec, link, MEASURED_TRAFFIC_BYTES.get((head, rec["path"])),
                                    TRAFFIC_SOURCE.get((head, rec["path"])))
    out["config"] = {"workload": rec["workload"], "path": rec["path"],
                     "transfer_num_cta": args.num_cta, "blocks": rec["blocks"],
                     "bytes_per_direction": rec["bytes_per_direction"],
                     "headline": "c1 = configs[1] of BASELINE.json, the first configuration beyond "
                                 "the reference's own CPU-runnable case (c0) and the one that is "
                                 "asked for on both engines; BASELINE.json's metric names no "
                                 "configuration.  c0, c2 (the most bytes: 10 GiB a direction), c3, "
                                 "c3_fragmented and c4 are under `configs`, each with its own "
                                 "steps / warmup"}
    out["link_peak"] = link_rec
    out["hardware_queues"] = int(os.environ.get("GPU_MAX_HW_QUEUES", "4"))   # of this process
    pol = c_ext.get_launch_policy()
    out["launch_policy"] = {k: pol[k] for k in (
        "model_seeded", "model_link_mbps", "model_kernel_d2h_mbps", "model_kernel_h2d_mbps",
        "link_gbps_estimate", "staged_copy_overhead_us", "staged_restore", "staged_gather",
        "gather_threads", "xcd_count")}
    # the one launch on this path that HBM bounds: engine blocks <-> dense device buffer
    out["device_staging"] = transform_record(torch, device, args, 5, 2)["roofline"]
    if not args.no_cpu_baseline:
        torch.cuda.empty_cache()
        for name, r in records.items():
            r["cpu_baseline"] = cpu_baseline("c3f" if name == "c3_fragmented" else name, budget_s=5.0)
        out["cpu_baseline"] = records[head]["cpu_baseline"]
    out["configs"] = records
    print(json.dumps(out))


def transform_record(torch, device, args, steps, warmup):
    r = run_layout_transform(torch, device, steps, warmup, args.shape, verify=not args.no_verify)
    avg_ms = (r["to_buffer_ms"] + r["to_engine_ms"]) / 2
    achieved = 2 * r["bytes"] / (avg_ms * 1e-3) / 1e9    # bytes read + bytes written
    plain = 2 * r["bytes"] / (r["plain_copy_ms"] * 1e-3) / 1e9
    hbm = measure_hbm()
    return {
        "hbm_yardsticks": hbm,
        "frac_of_contiguous_copy_yardstick": round(achieved / hbm["copy_GBps"], 4),
        "metric": "engine blocks <-> dense device buffer, GB/s of HBM traffic (read + write)",
        "unit": "GB/s", "value": round(achieved, 1), "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(avg_ms, 4), "higher_is_better": True,
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
                     "traffic_source": TRAFFIC_SOURCE.get(("transform-" + args.shape, "kernel")),
                     "kernel": "fkv_copy_chunks_kernel<16, true, 16, false>",
                     "workload": f"transform-{args.shape}: " + r["desc"],
                     "algorithmic_bytes_per_launch": 2 * r["bytes"],
                     "avg_launch_ms": round(avg_ms, 4), "bit_exact": r["bit_exact"],
                     "hbm_yardsticks": hbm,
                     "frac_of_contiguous_copy_yardstick": round(achieved / hbm["copy_GBps"], 4)}}


if __name__ == "__main__":
    main()
