"""HIP gather/scatter kernel vs the CPU oracle, through the C ABI, bit-exact."""
import numpy as np
import pytest

from kvsetup import KVSetup, VLLM, TRTLLM, SGLANG, block_ids

pytestmark = pytest.mark.gpu

# (backend, L, kv_dim, N_gpu, N_cpu, chunk, cpu_layout, gpu_layout)
KERNEL_CASES = [
    pytest.param(VLLM, 4, 2, 64, 48, 16 * 8 * 128 * 2, "BLOCKFIRST", "LAYERFIRST", id="vllm-llama-bf"),
    pytest.param(VLLM, 4, 2, 64, 48, 16 * 8 * 128 * 2, "LAYERFIRST", "LAYERFIRST", id="vllm-llama-lf"),
    pytest.param(VLLM, 3, 2, 40, 40, 4096, "BLOCKFIRST", "LAYERBLOCK", id="vllm-layerblock"),
    pytest.param(VLLM, 5, 1, 32, 32, 64 * 576 * 2, "BLOCKFIRST", "LAYERFIRST", id="mla-packed"),
    pytest.param(TRTLLM, 6, 2, 32, 32, 8 * 32 * 128, "BLOCKFIRST", "LAYERFIRST", id="trtllm-fp8"),
    pytest.param(SGLANG, 4, 2, 64, 32, 64 * 8 * 128 * 2, "BLOCKFIRST", "LAYERFIRST", id="sglang-page64"),
    pytest.param(SGLANG, 4, 2, 64, 32, 1024, "LAYERFIRST", "LAYERFIRST", id="sglang-lf"),
]


@pytest.mark.parametrize("backend,L,K,N,NH,chunk,cpu_layout,gpu_layout", KERNEL_CASES)
@pytest.mark.parametrize("pattern", ["scattered", "contiguous", "few_seg"])
def test_kernel_d2h_then_h2d_matches_oracle(gpu_device, backend, L, K, N, NH, chunk, cpu_layout,
                                            gpu_layout, pattern):
    s = KVSetup(backend, L, K, N, NH, chunk, cpu_layout, gpu_layout, seed=11)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(5)
    n = 24
    gids, cids = block_ids(rng, N, n, pattern), block_ids(rng, NH, n, pattern)
    print(f"case backend={backend} L={L} kv={K} chunk={chunk} {cpu_layout} {pattern}", flush=True)
    # D2H gather
    dev.transfer(gids, cids, is_h2d=False)
    s.oracle_transfer(gids, cids, is_h2d=False)
    dev.assert_matches_reference("after D2H")
    # H2D scatter into different GPU blocks
    gids2 = block_ids(rng, N, n, "scattered")
    dev.transfer(gids2, cids, is_h2d=True)
    s.oracle_transfer(gids2, cids, is_h2d=True)
    dev.assert_matches_reference("after H2D")
