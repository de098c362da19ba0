"""Pins the multi-group / sliding-window restatement of the oracle against the
known answers of the reference's own tests, and checks the host-side layout
helpers the restore is configured with.  Runs without a GPU."""
import numpy as np
import pytest

from flexkv_amd.layout import (LayerGroupSpec, MultiGroupBlockLayout, build_layer_member_map)
from mgsetup import (CPU_SRC, GPU_DST, INDEXER_HEAD_SIZE, MAIN_HEAD_SIZE, SWA_CPU_SRC,
                     SWA_GPU_DST, MGCase, gpu_layout_of, main_seed, swa_seed)


def _t6_groups(num_layers=4):
    main = LayerGroupSpec(num_layers, 1, MAIN_HEAD_SIZE, tuple(range(num_layers)), itemsize=1)
    indexer = LayerGroupSpec(3, 1, INDEXER_HEAD_SIZE, (1, 2, 3), itemsize=1)
    return [main, indexer]


# ---- layout helpers ---------------------------------------------------------------

def test_member_map_examples_of_the_reference_docstring():
    # flexkv/common/config.py:76-86
    single = build_layer_member_map([LayerGroupSpec(3, 1, 8, (0, 1, 2))], 3)
    assert single.members == (((0, 0),), ((0, 1),), ((0, 2),))
    both = build_layer_member_map([LayerGroupSpec(2, 1, 8, (0, 1)),
                                   LayerGroupSpec(2, 1, 4, (0, 1))], 2)
    assert both.members == (((0, 0), (1, 0)), ((0, 1), (1, 1)))
    alt = build_layer_member_map([LayerGroupSpec(2, 1, 8, (0, 2)),
                                  LayerGroupSpec(2, 1, 4, (1, 3))], 4)
    assert alt.members == (((0, 0),), ((1, 0),), ((0, 1),), ((1, 1),))
    assert alt.num_original_layers == 4 and alt.members_of(2) == ((0, 1),)


def test_member_map_dsv4_shape():
    # tests/test_layerwise_dsv4_multi_group_swa_roundtrip.py:459-474
    c4, c128 = (0, 1, 2, 3), (4, 5, 6, 7)
    groups = [LayerGroupSpec(4, 1, 64, c4, 1, 4), LayerGroupSpec(4, 1, 32, c128, 1, 128),
              LayerGroupSpec(4, 1, 40, c4, 1, 4)]
    mm = build_layer_member_map(groups, 8)
    for orig in c4:
        assert {gi for gi, _ in mm.members_of(orig)} == {0, 2}
    for orig in c128:
        assert len(mm.members_of(orig)) == 1 and mm.members_of(orig)[0][0] == 1


def test_member_map_rejects_bad_indices():
    with pytest.raises(ValueError):
        build_layer_member_map([LayerGroupSpec(1, 1, 8, (5,))], 4)
    with pytest.raises(ValueError):
        LayerGroupSpec(2, 1, 8, (1, 1))
    with pytest.raises(ValueError):
        LayerGroupSpec(3, 1, 8, (0, 1))


def test_block_layout_bytes_and_group_offsets():
    # storage.py:120-127: sum over groups of L_g * kv_dim * (tpb / ratio) * heads * dim * itemsize
    groups = [LayerGroupSpec(4, 1, 64, (0, 1, 2, 3), 2, 4), LayerGroupSpec(4, 1, 32, (4, 5, 6, 7), 2, 128),
              LayerGroupSpec(4, 1, 40, (0, 1, 2, 3), 1, 4)]
    lay = MultiGroupBlockLayout(8, 128, tuple(groups), kv_dim=1, tp_size=1)
    per_group = [4 * 32 * 64 * 2, 4 * 1 * 32 * 2, 4 * 32 * 40]
    assert lay.get_block_stride() == sum(per_group)
    assert lay.kv_shape == (8, sum(per_group))
    st = lay.get_group_strides()
    assert [s["offset_bytes"] for s in st] == [0, per_group[0], per_group[0] + per_group[1]]
    assert [s["chunk_size"] for s in st] == [32 * 64 * 2, 32 * 2, 32 * 40]
    assert all(s["layer_stride"] == s["kv_stride"] for s in st)  # kv_dim == 1
    # every rank of a TP group has its own copy of the block
    assert MultiGroupBlockLayout(8, 128, tuple(groups), tp_size=4).get_block_stride() == \
        4 * sum(per_group)
    with pytest.raises(ValueError):
        MultiGroupBlockLayout(8, 100, tuple(groups))


def test_tables_match_the_reference_fixture_numbers():
    # T6 geometry of tests/test_layerwise_multi_group_swa.py: uint8, 16 tokens
    case = MGCase(_t6_groups(), 4)
    t = case.tables
    assert t["group_chunk_sizes"] == [16 * 32, 16 * 16]
    assert t["group_cpu_offset_bytes"] == [0, 4 * 512]
    assert t["cpu_block_stride"] == 4 * 512 + 3 * 256
    assert t["group_cpu_block_strides"] == [2816, 2816]
    assert t["group_cpu_tp_strides"] == [2816, 2816]
    assert t["group_h2d_cpu_layer_strides"] == [512, 256]
    # LAYERFIRST device pools: [layer, kv=1, block, token, head, dim]
    assert t["group_gpu_block_strides"] == [512, 256]
    assert t["group_gpu_kv_strides"] == [8 * 512, 8 * 256]
    assert t["group_gpu_layer_strides"] == [8 * 512, 8 * 256]
    assert t["layer_members"] == [[(0, 0)], [(0, 1), (1, 0)], [(0, 2), (1, 1)], [(0, 3), (1, 2)]]
    assert gpu_layout_of(case.layer_groups[1], 8, 16).kv_shape == (3, 1, 8, 16, 1, 16)


# ---- the oracle against the reference's known answers -------------------------------

def test_seed_formulas_spot_values():
    # hand-evaluated: ((orig*100 + gi*10 + local*3 + tok) ^ b) & 0xFF
    s = main_seed(3, 1, 2, 16, 1, 16)
    assert s[5, 0, 9] == ((300 + 10 + 6 + 5) ^ 9) & 0xFF == 72
    w = swa_seed(2, 16, 64)
    assert w[7, 0, 33] == ((62 + 7 + 0xB2) ^ 33) & 0xFF == 214


def _run_oracle(case, with_swa, cpu_ids=(CPU_SRC,), gpu_ids=(GPU_DST,)):
    from oracle import fkv_oracle as O
    swa = case.oracle_swa([SWA_CPU_SRC], [SWA_GPU_DST]) if with_swa else None
    return O.layerwise_multi_group(1, case.oracle_groups(), case.members, case.host,
                                   list(gpu_ids), list(cpu_ids), 1, 1, "sharded", swa)


def test_oracle_t6_main_indexer_and_swa():
    case = MGCase(_t6_groups(), 4)
    exp_main = case.seed_all_main()
    exp_swa = case.seed_all_swa()
    immediate, work = _run_oracle(case, True)
    assert immediate == [] and work == [0, 1, 2, 3]
    assert len(exp_main) == 7
    for (orig, gi, local), exp in exp_main.items():
        assert np.array_equal(case.gpu[gi][local][GPU_DST], exp), (orig, gi, local)
        others = np.delete(case.gpu[gi][local], GPU_DST, axis=0)
        assert not others.any()
    for orig, exp in exp_swa.items():
        assert np.array_equal(case.swa_gpu[orig][SWA_GPU_DST], exp)
        assert not np.delete(case.swa_gpu[orig], SWA_GPU_DST, axis=0).any()


def test_oracle_t4_empty_member_layer():
    main = LayerGroupSpec(3, 1, MAIN_HEAD_SIZE, (1, 2, 3), itemsize=1)
    case = MGCase([main], 4)
    assert tuple(case.members[0]) == ()
    exp_main = case.seed_all_main()
    exp_swa = case.seed_all_swa()
    immediate, work = _run_oracle(case, True)
    assert immediate == [] and work == [0, 1, 2, 3]  # layer 0 waits for its sidecar copy
    for (orig, gi, local), exp in exp_main.items():
        assert np.array_equal(case.gpu[gi][local][GPU_DST], exp)
    for orig, exp in exp_swa.items():
        assert np.array_equal(case.swa_gpu[orig][SWA_GPU_DST], exp)
    # without sidecar ids layer 0 is announced on entry
    # (tests/test_layerwise_eventfd_timing.py:396-427)
    case2 = MGCase([main], 4)
    immediate, work = _run_oracle(case2, False)
    assert immediate == [0] and work == [1, 2, 3]
    assert not any(a.any() for a in case2.swa_gpu)


def test_oracle_dsv4_round_trip():
    """tests/test_layerwise_dsv4_multi_group_swa_roundtrip.py:397-457 on host memory."""
    from oracle import fkv_oracle as O
    c4, c128 = (0, 1, 2, 3), (4, 5, 6, 7)
    groups = [LayerGroupSpec(4, 1, 64, c4, 1, 4), LayerGroupSpec(4, 1, 32, c128, 1, 128),
              LayerGroupSpec(4, 1, 40, c4, 1, 4)]
    case = MGCase(groups, 8, tpb=128, swa_width=128)
    gpu_src, cpu_dst, gpu_back, swa_cpu_dst, swa_gpu_back = 1, 2, 5, 3, 6
    golden = {}
    for orig in range(8):
        for gi, local in case.members[orig]:
            g = groups[gi]
            golden[(gi, local)] = main_seed(orig, gi, local, 128 // g.compress_ratio, 1,
                                            g.head_size, mul=(97, 13, 7))
            case.gpu[gi][local][gpu_src] = golden[(gi, local)]
    swa_golden = {orig: swa_seed(orig, 128, 128, salt=0xD4) for orig in range(8)}
    for orig, v in swa_golden.items():
        case.swa_gpu[orig][gpu_src] = v
    t = case.tables
    for gi, grp in enumerate(case.oracle_groups()):  # PUT: one D2H per group into its slice
        O.transfer_c(grp.backend, [a.ctypes.data for a in case.gpu[gi]], grp.num_layers,
                     grp.gpu_kv_strides[0], grp.gpu_block_strides[0], grp.gpu_layer_strides[0], 0,
                     case.host.ctypes.data + t["group_cpu_offset_bytes"][gi],
                     t["group_cpu_kv_strides"][gi], t["group_cpu_layer_strides"][gi],
                     t["group_cpu_block_strides"][gi], 0, t["group_chunk_sizes"][gi], 0,
                     grp.num_layers, 1, [gpu_src], [cpu_dst], False)
    s, c = case.swa_gpu_strides, case.swa_cpu_strides
    O.transfer_c(O.BACKEND_VLLM, [a.ctypes.data for a in case.swa_gpu], 8, s.kv, s.block, s.layer,
                 0, case.swa_host.ctypes.data, c.kv, c.layer, c.block, 0, c.chunk, 0, 8, 1,
                 [gpu_src], [swa_cpu_dst], False)
    for grp in case.gpu:
        for a in grp:
            a[:] = 0
    for a in case.swa_gpu:
        a[:] = 0
    swa = case.oracle_swa([swa_cpu_dst], [swa_gpu_back])
    O.layerwise_multi_group(1, case.oracle_groups(), case.members, case.host, [gpu_back],
                            [cpu_dst], 1, 1, "sharded", swa)
    for (gi, local), v in golden.items():
        assert np.array_equal(case.gpu[gi][local][gpu_back], v), (gi, local)
    for orig, v in swa_golden.items():
        assert np.array_equal(case.swa_gpu[orig][swa_gpu_back], v), orig
