"""Writes the golden vectors of tests/golden/ from the closed-form fixtures the
reference's own tests define.  Plain numpy; nothing of the library, of the oracle
or of the reference tree is imported, so the files are an independent statement
of the expected bytes.

    python tests/golden/make_vectors.py

1. ``tp1_fill_pattern.npz`` -- tests/test_kv_transfer_correctness.py:262-278
   (``fill_gpu`` / ``expected_val``): element (kv, block, token, head, d) of layer
   ``l`` on GPU ``g`` is ((g*100000 + kv*500000 + l*10000 + block*1000 + token*10 +
   d) % 997) / 997 as fp16, identical across heads.  Stored: the engine tensors of
   a small vLLM-shaped cache, the block ids of a put, and the block-first and
   layer-first host images that put must produce (untouched bytes zero).
2. ``multi_group_t6.npz`` -- tests/test_layerwise_multi_group_swa.py:24-37, 214-236
   (case T6: a main group on all four layers, an indexer group on layers 1-3, a
   uniform sliding-window sidecar).  Byte ``b`` of token ``tok`` of (original layer
   ``orig``, group ``gi``, local layer ``local``) is ((orig*100 + gi*10 + local*3 +
   tok) ^ b) & 0xFF; sidecar ((orig*31 + tok + 0xB2) ^ b) & 0xFF.  Stored: the host
   pool and sidecar pool images with those bytes at block CPU_SRC / SWA_CPU_SRC,
   and the device tensors a restore into block GPU_DST / SWA_GPU_DST must produce.
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def tp1_fill_pattern():
    L, KV, N, T, H, D, NH = 3, 2, 6, 4, 2, 8, 5
    gpu = np.zeros((L, KV, N, T, H, D), dtype=np.float16)
    for l in range(L):
        for kv in range(KV):
            for b in range(N):
                for t in range(T):
                    for d in range(D):
                        v = ((0 * 100000 + kv * 500000 + l * 10000 + b * 1000 + t * 10 + d) % 997) / 997.0
                        gpu[l, kv, b, t, :, d] = np.float16(np.float32(v))
    gpu_ids = np.array([4, 0, 5, 2], dtype=np.int64)
    cpu_ids = np.array([1, 3, 0, 4], dtype=np.int64)
    host_bf = np.zeros((NH, L, KV, T, H, D), dtype=np.float16)   # BLOCKFIRST
    host_lf = np.zeros((L, KV, NH, T, H, D), dtype=np.float16)   # LAYERFIRST
    for g, c in zip(gpu_ids, cpu_ids):
        for l in range(L):
            for kv in range(KV):
                host_bf[c, l, kv] = gpu[l, kv, g]
                host_lf[l, kv, c] = gpu[l, kv, g]
    np.savez_compressed(os.path.join(HERE, "tp1_fill_pattern.npz"), gpu=gpu.view(np.uint16),
                        gpu_ids=gpu_ids, cpu_ids=cpu_ids, host_blockfirst=host_bf.view(np.uint16),
                        host_layerfirst=host_lf.view(np.uint16),
                        shape=np.array([L, KV, N, T, H, D, NH], dtype=np.int64))


def multi_group_t6():
    NUM_BLOCKS, TPB, MAIN, INDEXER, SWA_W = 8, 16, 32, 16, 64
    CPU_SRC, GPU_DST, SWA_CPU_SRC, SWA_GPU_DST = 2, 5, 3, 6
    OL = 4
    groups = [(4, MAIN, (0, 1, 2, 3)), (3, INDEXER, (1, 2, 3))]   # (layers, bytes per token, original layers)
    block_stride = sum(n * TPB * w for n, w, _ in groups)
    offsets = [0, groups[0][0] * TPB * groups[0][1]]
    host = np.zeros(NUM_BLOCKS * block_stride, dtype=np.uint8)
    gpu = [np.zeros((n, NUM_BLOCKS, TPB, 1, w), dtype=np.uint8) for n, w, _ in groups]
    tok = np.arange(TPB)[:, None]
    for gi, (n, w, orig_layers) in enumerate(groups):
        b = np.arange(w)[None, :]
        for local, orig in enumerate(orig_layers):
            chunk = (((orig * 100 + gi * 10 + local * 3 + tok) ^ b) & 0xFF).astype(np.uint8)
            at = CPU_SRC * block_stride + offsets[gi] + local * TPB * w
            host[at:at + TPB * w] = chunk.reshape(-1)
            gpu[gi][local, GPU_DST, :, 0, :] = chunk
    swa_host = np.zeros((OL, 1, NUM_BLOCKS, TPB, 1, SWA_W), dtype=np.uint8)   # LAYERFIRST
    swa_gpu = np.zeros((OL, NUM_BLOCKS, TPB, 1, SWA_W), dtype=np.uint8)
    b = np.arange(SWA_W)[None, :]
    for orig in range(OL):
        chunk = (((orig * 31 + tok + 0xB2) ^ b) & 0xFF).astype(np.uint8)
        swa_host[orig, 0, SWA_CPU_SRC, :, 0, :] = chunk
        swa_gpu[orig, SWA_GPU_DST, :, 0, :] = chunk
    np.savez_compressed(os.path.join(HERE, "multi_group_t6.npz"), host=host, gpu_main=gpu[0],
                        gpu_indexer=gpu[1], swa_host=swa_host, swa_gpu=swa_gpu,
                        ids=np.array([CPU_SRC, GPU_DST, SWA_CPU_SRC, SWA_GPU_DST], dtype=np.int64),
                        block_stride=np.array([block_stride], dtype=np.int64))


if __name__ == "__main__":
    tp1_fill_pattern()
    multi_group_t6()
    for name in sorted(os.listdir(HERE)):
        if name.endswith(".npz"):
            print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")
