"""The Python operators of flexkv_amd.c_ext against the reference's pybind argument
lists: names, positional order and defaults (tests/golden/c_ext_signatures.json, written
by tests/golden/make_signatures.py from csrc/bindings.cpp).  The reference's workers call
these operators positionally (flexkv/transfer/worker.py:1032-1059, 1218-1236, 1484-1499;
flexkv/transfer/layerwise.py:647-664, 953-1001), so a renamed or reordered argument is a
broken drop-in even when every keyword call still works.  No GPU involved.
"""
import inspect
import json
import os

import pytest
import torch

import flexkv_amd.c_ext as c_ext

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "c_ext_signatures.json"), encoding="utf-8") as f:
    REF = json.load(f)["operators"]


def same_default(ref, ours) -> bool:
    """A literal must be equal in value and type; an empty container of the reference
    may be None or an empty container of the same kind here."""
    if "value" in ref:
        return type(ours) is type(ref["value"]) and ours == ref["value"]
    kind = ref["empty"]
    if ours is None:
        return True
    if kind == "tensor":
        return isinstance(ours, torch.Tensor) and ours.numel() == 0
    if kind == "list":
        return isinstance(ours, (list, tuple)) and len(ours) == 0
    return isinstance(ours, dict) and len(ours) == 0


def compare(name, ref_args, our_params):
    """our_params: [(name, default or inspect.Parameter.empty)] in positional order."""
    assert [a for a, _ in ref_args] == [p for p, _ in our_params], name
    for (arg, ref), (_, ours) in zip(ref_args, our_params):
        if ref.get("required"):
            assert ours is inspect.Parameter.empty, f"{name}: {arg} must have no default"
        else:
            assert ours is not inspect.Parameter.empty, f"{name}: {arg} lost its default"
            assert same_default(ref, ours), f"{name}: default of {arg}: {ours!r} vs {ref}"


def params_of(fn, skip_self=False):
    ps = list(inspect.signature(fn).parameters.values())
    if skip_self:
        ps = ps[1:]
    for p in ps:
        assert p.kind is inspect.Parameter.POSITIONAL_OR_KEYWORD, (fn.__qualname__, p.name)
    return [(p.name, p.default) for p in ps]


@pytest.mark.parametrize("op,fn,skip_self", [
    ("transfer_kv_blocks", c_ext.transfer_kv_blocks, False),
    ("transfer_kv_blocks_ssd", c_ext.transfer_kv_blocks_ssd, False),
    ("TPTransferThreadGroup.__init__", c_ext.TPTransferThreadGroup.__init__, True),
    ("TPTransferThreadGroup.update_gpu_block_ptrs",
     c_ext.TPTransferThreadGroup.update_gpu_block_ptrs, True),
    ("TPTransferThreadGroup.tp_group_transfer", c_ext.TPTransferThreadGroup.tp_group_transfer, True),
    ("LayerwiseTransferGroup.init_swa_multi_group",
     c_ext.LayerwiseTransferGroup.init_swa_multi_group, True),
    ("LayerwiseTransferGroup.layerwise_transfer", c_ext.LayerwiseTransferGroup.layerwise_transfer,
     True),
    ("LayerwiseTransferGroup.layerwise_transfer_multi_group",
     c_ext.LayerwiseTransferGroup.layerwise_transfer_multi_group, True),
])
def test_operator_matches_the_reference_argument_list(op, fn, skip_self):
    (ref_args,) = REF[op]
    compare(op, ref_args, params_of(fn, skip_self))


def test_both_layerwise_constructors_match_the_reference_argument_lists():
    """The group takes *args / **kwargs and tells the two constructors apart the way
    pybind does; its name tables are what decides where a positional argument lands."""
    cls = c_ext.LayerwiseTransferGroup
    single, multi = sorted(REF["LayerwiseTransferGroup.__init__"], key=len)
    E = inspect.Parameter.empty
    common = list(cls._COMMON_DEFAULTS.items())
    compare("single-group constructor", single, [(n, E) for n in cls._SINGLE_NAMES] + common)
    compare("multi-group constructor", multi, [(n, E) for n in cls._MULTI_NAMES] + common)


# ---- the reference's own call shapes, positionally, with empty block lists ----------

class Recorder:
    """Stands in for the loaded library: records the descriptor of the call."""

    def __init__(self):
        self.calls = []

    def __getattr__(self, name):
        def call(*args):
            self.calls.append((name, args))
            return 0
        return call


def test_transfer_kv_blocks_called_as_the_reference_worker_calls_it(monkeypatch):
    """flexkv/transfer/worker.py:1032-1059: 25 positional arguments and one keyword."""
    rec = Recorder()
    monkeypatch.setattr(c_ext, "_L", rec)
    monkeypatch.setattr(c_ext, "_current_stream_handle", lambda: 0)
    ids = torch.empty(0, dtype=torch.int64)
    ptrs = torch.tensor([4096, 8192], dtype=torch.int64)
    host = torch.zeros(2 * 2 * 2 * 64, dtype=torch.uint8)
    c_ext.transfer_kv_blocks(
        ids, ptrs, 512, 64, 1024, ids, host, 64, 128, 256, 64,
        0,            # start_layer_id (whole-model)
        2,            # num_layers
        4,            # transfer_num_cta
        True,         # H2D
        False,        # use_ce_transfer
        2,            # kv_dim
        8,            # num_kv_heads
        0,            # gpu_block_type
        True,         # sync
        True,         # ce_path_opt
        8,            # ce_segment_threshold
        -1,           # ce_force_path
        False,        # ce_enable_memcpy2d
        True,         # cpu_is_blockfirst
        enable_transfer_trace=False)
    (name, (desc_ref, stream)), = rec.calls
    d = desc_ref._obj
    assert name == "fkv_transfer_kv_blocks"
    assert (d.gpu_kv_stride, d.gpu_block_stride, d.gpu_layer_stride) == (512, 64, 1024)
    assert (d.cpu_kv_stride, d.cpu_layer_stride, d.cpu_block_stride, d.chunk_size) == (64, 128, 256, 64)
    assert (d.start_layer_id, d.num_layers, d.transfer_num_cta, d.is_host_to_device) == (0, 2, 4, 1)
    assert (d.use_ce_transfer, d.kv_dim, d.backend, d.sync, d.num_blocks) == (0, 2, 0, 1, 0)
    assert (d.ce.path_opt_enabled, d.ce.segment_threshold, d.ce.force_path) == (1, 8, -1)
    assert (d.ce.enable_memcpy2d, d.ce.is_blockfirst, d.ce.num_kv_heads) == (0, 1, 8)


def test_tp_group_called_as_the_reference_worker_calls_it(monkeypatch):
    """flexkv/transfer/worker.py:1218-1236 passes (ce_segment_threshold, ce_path_opt,
    enable_ce_memcpy2d, cpu_is_blockfirst, num_kv_heads) right behind gpu_device_ids, where
    the binding has (enable_nvcomp, nvcomp_batch_size, nvcomp_data_type, ce_segment_threshold,
    ce_path_opt): the arguments land one group to the left, exactly as they do in the
    reference, whose default build ignores the nvcomp ones
    (csrc/tp_transfer_thread_group.cpp:132-136).  The call must be accepted all the same;
    worker.py:1484-1499 then calls tp_group_transfer with 14 positional arguments."""
    rec = Recorder()
    monkeypatch.setattr(c_ext, "_L", rec)
    grp = c_ext.TPTransferThreadGroup(
        1, [4096, 8192], 2, 1 << 20, 2, [512], [64], [1024], [64], [0],
        8,          # GLOBAL_CONFIG_FROM_ENV.ce_segment_threshold  -> enable_nvcomp
        True,       # ce_path_opt                                   -> nvcomp_batch_size
        True,       # enable_ce_memcpy2d                            -> nvcomp_data_type
        True,       # cpu_is_blockfirst                             -> ce_segment_threshold
        8,          # num_kv_heads                                  -> ce_path_opt
        ce_gather_threads=4, ce_gather_nt=True)
    name, (params_ref, _) = rec.calls[0]
    p = params_ref._obj
    assert name == "fkv_tp_group_create"
    assert (p.num_gpus, p.num_tensors_per_gpu, p.num_layers) == (1, 2, 2)
    assert (p.ce.segment_threshold, p.ce.path_opt_enabled) == (1, 1)
    assert (p.ce.force_path, p.ce.enable_memcpy2d, p.ce.is_blockfirst, p.ce.num_kv_heads) == \
        (-1, 0, 0, 1)
    ids = torch.empty(0, dtype=torch.int64)
    grp.tp_group_transfer(ids, ids, 64, 128, 256, 256, 4, True, False,
                          0,       # start layer (whole model)
                          2,       # layer_granularity = all layers
                          2, 8, "sharded")
    name, args = rec.calls[1]
    assert name == "fkv_tp_group_transfer"
    assert [int(getattr(a, "value", a)) if not isinstance(a, bytes) else a for a in args[3:]] == \
        [0, 64, 128, 256, 256, 4, 1, 0, 0, 2, 2, 8, b"sharded", 0]
    grp._h = None   # nothing was created: nothing to destroy
