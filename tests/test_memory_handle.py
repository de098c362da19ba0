"""TensorSharedHandle: what the owner constructs, what the pickle carries, what a
worker process gets back.  The shape of the reference's tests/test_memory_handle.py
(construction from a tensor with torch's IPC and with a direct IPC handle, from
raw handle bytes, dtype given as a string, bf16 / fp8 payloads, writes of the
child seen by the parent), plus a tensor that starts inside its allocation."""
import pickle

import pytest
import torch
import torch.multiprocessing as mp

from flexkv_amd.transfer.memory_handle import (IPC_HANDLE_BYTES, TensorSharedHandle, _as_dtype,
                                               _carrier_dtype)


# ---- construction rules: no GPU needed ------------------------------------------------------

def test_rejects_what_it_cannot_share():
    with pytest.raises(ValueError, match="Unsupported data type"):
        TensorSharedHandle([1, 2, 3])
    with pytest.raises(ValueError, match="Only support CUDA tensor sharing"):
        TensorSharedHandle(torch.zeros(4))
    raw = bytes(IPC_HANDLE_BYTES)
    with pytest.raises(ValueError, match="needs tensor_shape, tensor_dtype and device_id"):
        TensorSharedHandle(raw, device_id=0)
    with pytest.raises(ValueError, match="needs tensor_shape, tensor_dtype and device_id"):
        TensorSharedHandle(raw, tensor_shape=(2,), tensor_dtype=torch.float16)
    with pytest.raises(ValueError, match="64 bytes, got 10"):
        TensorSharedHandle(bytes(10), device_id=0, tensor_shape=(2,), tensor_dtype="float16")
    with pytest.raises(ValueError, match="not supported on this platform"):
        TensorSharedHandle(raw, device_id=0, tensor_shape=(2,), tensor_dtype="float16",
                           handle_type="vmm_fabric")
    with pytest.raises(ValueError, match="unknown dtype"):
        TensorSharedHandle(raw, device_id=0, tensor_shape=(2,), tensor_dtype="floatish")


def test_handle_from_bytes_keeps_what_it_was_given():
    raw = bytes(range(IPC_HANDLE_BYTES))
    h = TensorSharedHandle(raw, device_id=0, tensor_shape=(10, 20), tensor_dtype="float16",
                           offset=4096)
    assert h.use_direct_ipc and h.handle_type == "hip_ipc" and h.rebuild_func is None
    assert h.ipc_handle == raw and h.tensor_shape == (10, 20) and h.tensor_numel == 200
    assert h.tensor_dtype == torch.float16 and h.offset == 4096 and h.device.index == 0
    back = pickle.loads(pickle.dumps(h))
    assert back.ipc_handle == raw and back.tensor_shape == (10, 20) and back.offset == 4096
    assert back.tensor_dtype == torch.float16 and back._opened_base is None


@pytest.mark.parametrize("name,dtype", [("float32", torch.float32), ("torch.float16", torch.float16),
                                        ("bfloat16", torch.bfloat16), ("int8", torch.int8),
                                        ("uint8", torch.uint8), ("int64", torch.int64),
                                        ("float8_e4m3fn", torch.float8_e4m3fn)])
def test_dtype_names(name, dtype):
    assert _as_dtype(name) == dtype and _as_dtype(dtype) == dtype
    assert _carrier_dtype(dtype).itemsize == dtype.itemsize   # bytes travel unchanged


# ---- across processes, on the GPU -------------------------------------------------------------

def _child(conn, expect_direct):
    try:
        h, shape, dtype, want = conn.recv()
        assert isinstance(h, TensorSharedHandle) and h.use_direct_ipc == expect_direct
        t = h.get_tensor()
        assert t.is_cuda and tuple(t.shape) == tuple(shape) and t.dtype == dtype
        carrier = torch.int16 if dtype.itemsize == 2 else torch.uint8 if dtype.itemsize == 1 \
            else torch.int32
        assert torch.equal(t.view(carrier).cpu(), want), "bytes differ from the owner's"
        t.view(carrier).fill_(7)                           # the parent must see this
        torch.cuda.synchronize()
        h.release()
        conn.send(True)
    except Exception as e:  # noqa: BLE001
        conn.send(f"Error: {type(e).__name__}: {e}")


def _share(handle, tensor, carrier, direct):
    ctx = mp.get_context("spawn")
    parent, child = ctx.Pipe()
    p = ctx.Process(target=_child, args=(child, direct), daemon=True)
    p.start()
    parent.send((handle, tuple(tensor.shape), tensor.dtype, tensor.view(carrier).cpu()))
    assert parent.poll(180), "child did not answer"
    result = parent.recv()
    p.join(30)
    assert result is True, result
    torch.cuda.synchronize()
    assert bool((tensor.view(carrier) == 7).all()), "the child's writes did not reach the owner"


@pytest.mark.gpu
@pytest.mark.parametrize("direct", [False, True], ids=["torch_reduce", "hip_ipc"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float8_e4m3fn],
                         ids=["f32", "bf16", "fp8"])
def test_handle_from_tensor_across_processes(gpu_device, direct, dtype):
    carrier = torch.int16 if dtype.itemsize == 2 else torch.uint8 if dtype.itemsize == 1 \
        else torch.int32
    t = torch.arange(200, dtype=torch.float32, device=gpu_device).reshape(10, 20).to(dtype)
    h = TensorSharedHandle(t, device_id=0, force_direct_ipc=direct)
    assert h.use_direct_ipc == direct and h.device.index == 0
    if direct:
        assert len(h.ipc_handle) == IPC_HANDLE_BYTES and h.rebuild_func is None
        assert h.tensor_shape == (10, 20) and h.tensor_dtype == dtype and h.tensor_numel == 200
    else:
        assert h.rebuild_func is not None and h.rebuild_args is not None
    _share(h, t, carrier, direct)


@pytest.mark.gpu
def test_handle_from_bytes_with_an_offset_into_the_allocation(gpu_device):
    """An engine that exported the handle of its whole pool itself: the worker gets
    bytes + shape + dtype + offset and must land on the right sub-range."""
    pool = torch.zeros(3, 10, 20, dtype=torch.float16, device=gpu_device)
    pool[1] = torch.arange(200, dtype=torch.float16, device=gpu_device).reshape(10, 20)
    part = pool[1]
    owner = TensorSharedHandle(part, device_id=0, force_direct_ipc=True)
    assert owner.offset >= part.numel() * 2 or owner.offset == part.data_ptr() - pool.data_ptr()
    h = TensorSharedHandle(owner.ipc_handle, device_id=0, tensor_shape=owner.tensor_shape,
                           tensor_dtype="float16", offset=owner.offset)
    assert h.use_direct_ipc and h.ipc_handle == owner.ipc_handle
    _share(h, part, torch.int16, True)
    assert not pool[0].any() and not pool[2].any()         # neighbours untouched
