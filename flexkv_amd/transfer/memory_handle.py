"""Handles that carry an engine's KV tensors into a transfer-worker process.

``TensorSharedHandle`` keeps the constructor and ``get_tensor()`` contract of the
reference (``flexkv/common/memory_handle.py:466-545, 808-838``): built from a
device tensor by the owner, pickled across the pipe, turned back into a tensor
that aliases the same device memory by the worker.  Two export forms:

* ``torch_reduce`` — torch's own sharing of caching-allocator blocks
  (``torch.multiprocessing.reductions.reduce_tensor``), the default;
* ``hip_ipc`` — ``hipIpcGetMemHandle`` of the allocation the tensor lives in plus
  the tensor's byte offset inside it, for memory torch does not manage or when
  ``force_direct_ipc`` is set.  A handle built from raw bytes (an engine that
  exported the handle itself) also takes this form.

The driver-level virtual-memory export of the reference (fabric / POSIX-fd
handles for engines that allocate KV with cuMemCreate) has no use here: nothing
on this platform allocates KV memory that way, so those handle types are
rejected on construction.
"""
from __future__ import annotations

import ctypes
import logging
import weakref
from typing import Any, Callable, Optional, Tuple, Union

import torch
from torch.multiprocessing import reductions

from .. import _lib
from .._lib import check

logger = logging.getLogger("flexkv")

IPC_HANDLE_BYTES = 64

# names usable in __cuda_array_interface__; two-byte and one-byte floats travel as
# integers of the same width and are viewed back
_TYPESTR = {torch.float32: "<f4", torch.float64: "<f8", torch.float16: "<f2",
            torch.int32: "<i4", torch.int64: "<i8", torch.int16: "<i2", torch.uint8: "|u1",
            torch.int8: "|i1", torch.bool: "|b1"}
if hasattr(torch, "uint16"):
    _TYPESTR[torch.uint16] = "<u2"


def _carrier_dtype(dtype: torch.dtype) -> torch.dtype:
    if dtype in _TYPESTR:
        return dtype
    if dtype.itemsize == 2:
        return torch.int16
    if dtype.itemsize == 1:
        return torch.uint8
    raise ValueError(f"Unsupported dtype for a device pointer: {dtype}")


class _DevicePointer:
    def __init__(self, ptr: int, shape: Tuple[int, ...], typestr: str) -> None:
        self.__cuda_array_interface__ = {"data": (ptr, False), "shape": tuple(shape),
                                         "typestr": typestr, "version": 3, "strides": None}


def tensor_from_device_pointer(ptr: int, shape: Tuple[int, ...], dtype: torch.dtype,
                               device: torch.device) -> torch.Tensor:
    """Zero-copy tensor over device memory this process did not allocate through
    torch (memory_handle.py:1055-1141)."""
    carrier = _carrier_dtype(dtype)
    t = torch.as_tensor(_DevicePointer(ptr, shape, _TYPESTR[carrier]), device=device)
    return t if carrier == dtype else t.view(dtype)


def _as_dtype(dtype: Union[torch.dtype, str]) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        return dtype
    name = str(dtype).replace("torch.", "")
    got = getattr(torch, name, None)
    if not isinstance(got, torch.dtype):
        raise ValueError(f"unknown dtype {dtype!r}")
    return got


class TensorSharedHandle:
    def __init__(self, data: Union[torch.Tensor, bytes], device_id: int = -1,
                 force_direct_ipc: bool = False, *,
                 tensor_shape: Optional[Tuple[int, ...]] = None,
                 tensor_dtype: Optional[Union[torch.dtype, str]] = None,
                 offset: int = 0, handle_type: Optional[str] = None) -> None:
        self.rebuild_func: Optional[Callable] = None
        self.rebuild_args: Optional[Tuple[Any, ...]] = None
        self.use_direct_ipc = False
        self.ipc_handle: Optional[bytes] = None
        self.tensor_shape: Optional[Tuple[int, ...]] = None
        self.tensor_dtype: Optional[torch.dtype] = None
        self.tensor_numel: Optional[int] = None
        self.offset = 0
        self.handle_type = "torch_reduce"
        self._opened_base: Optional[int] = None
        if isinstance(data, torch.Tensor):
            self._from_tensor(data, device_id, force_direct_ipc)
        elif isinstance(data, (bytes, bytearray)):
            if handle_type not in (None, "cuda_ipc", "hip_ipc"):
                raise ValueError(f"handle_type {handle_type!r} is not supported on this platform")
            if tensor_shape is None or tensor_dtype is None or device_id < 0:
                raise ValueError("a raw IPC handle needs tensor_shape, tensor_dtype and device_id")
            if len(data) != IPC_HANDLE_BYTES:
                raise ValueError(f"an IPC handle is {IPC_HANDLE_BYTES} bytes, got {len(data)}")
            self._set_direct(bytes(data), tuple(tensor_shape), _as_dtype(tensor_dtype),
                             torch.device(f"cuda:{device_id}"), int(offset))
        else:
            raise ValueError(f"Unsupported data type {type(data)} for TensorSharedHandle, "
                             "expected torch.Tensor / bytes-like")

    # ---- owner side ------------------------------------------------------------------
    def _from_tensor(self, tensor: torch.Tensor, device_id: int, force_direct_ipc: bool) -> None:
        if not tensor.is_cuda:
            raise ValueError("Only support CUDA tensor sharing")
        device = tensor.device if device_id == -1 else torch.device(f"cuda:{device_id}")
        if not force_direct_ipc:
            try:
                self.rebuild_func, args = reductions.reduce_tensor(tensor)
                if device_id != -1:
                    args = list(args)
                    args[6] = device_id  # the device the worker rebuilds on
                self.rebuild_args = tuple(args)
                self.device = device
                return
            except RuntimeError as e:
                logger.warning("torch IPC export failed (%s); exporting the allocation directly", e)
        if not tensor.is_contiguous():
            raise ValueError("direct IPC export needs a contiguous tensor")
        handle = (ctypes.c_uint8 * IPC_HANDLE_BYTES)()
        off = ctypes.c_int64(0)
        size = ctypes.c_int64(0)
        with torch.cuda.device(tensor.device):
            check(_lib.load().fkv_ipc_export(tensor.data_ptr(), handle, ctypes.byref(off),
                                             ctypes.byref(size)))
        self._set_direct(bytes(handle), tuple(tensor.shape), tensor.dtype, device, off.value)

    def _set_direct(self, handle: bytes, shape, dtype, device, offset: int) -> None:
        self.ipc_handle = handle
        self.use_direct_ipc = True
        self.handle_type = "hip_ipc"
        self.tensor_shape = shape
        self.tensor_dtype = dtype
        numel = 1
        for e in shape:
            numel *= int(e)
        self.tensor_numel = numel
        self.offset = offset
        self.device = device

    # ---- worker side -----------------------------------------------------------------
    def get_tensor(self) -> torch.Tensor:
        if not self.use_direct_ipc:
            tensor = self.rebuild_func(*self.rebuild_args)
            if tensor.device != self.device:
                raise RuntimeError(f"shared tensor arrived on {tensor.device}, expected "
                                   f"{self.device}")
            return tensor
        dev = self.device.index if self.device.index is not None else 0
        torch.cuda.set_device(dev)
        torch.zeros(1, device=self.device)  # the runtime must be up before the open
        base = ctypes.c_void_p()
        buf = (ctypes.c_uint8 * IPC_HANDLE_BYTES).from_buffer_copy(self.ipc_handle)
        check(_lib.load().fkv_ipc_open(buf, dev, ctypes.byref(base)))
        self._opened_base = base.value
        return tensor_from_device_pointer(base.value + self.offset, self.tensor_shape,
                                          self.tensor_dtype, self.device)

    def release(self) -> None:
        """Drops the mapping ``get_tensor`` opened (direct form only).  Tensors made
        from it must not be used afterwards."""
        if self._opened_base is not None:
            check(_lib.load().fkv_ipc_close(ctypes.c_void_p(self._opened_base)))
            self._opened_base = None

    def __getstate__(self):
        state = dict(self.__dict__)
        state["_opened_base"] = None
        return state


def discard_tensor_handles(handles) -> None:
    """Let go of handles this process received and will not use (a rejected request).  The
    owner of a tensor shared through torch keeps its memory until every handle it sent has
    been opened and dropped by a receiver; a handle that is just forgotten holds that
    memory until the owner exits.  Accepts nested lists."""
    for h in handles or ():
        if isinstance(h, (list, tuple)):
            discard_tensor_handles(h)
        elif isinstance(h, TensorSharedHandle) and not h.use_direct_ipc:
            try:
                t = h.get_tensor()
                del t
            except Exception as e:  # noqa: BLE001 - nothing more can be done for it
                logger.warning("could not open a shared tensor to release it: %s", e)
    try:
        if torch.cuda.is_initialized():
            torch.cuda.ipc_collect()
    except Exception:  # noqa: BLE001
        pass


# handle object -> weak reference to the tensor this process made of it
_OPENED: "weakref.WeakKeyDictionary[TensorSharedHandle, weakref.ref]" = weakref.WeakKeyDictionary()


def _tensor_of(h: "TensorSharedHandle") -> torch.Tensor:
    """One tensor per handle object and process while that tensor is alive.  A worker for a
    model with layer groups is handed the first group's handles twice (as ``gpu_blocks`` and
    inside ``gpu_blocks_per_group``, ``flexkv/transfer/worker.py:850-870``); a handle made by
    torch's own sharing counts one receiver, and opening it twice leaves the owner's
    count off by one for good."""
    ref = _OPENED.get(h)
    t = ref() if ref is not None else None
    if t is None:
        t = h.get_tensor()
        _OPENED[h] = weakref.ref(t)
    return t


def import_tensor_handles(handles) -> list:
    """Tensors of a list of handles, after switching to their device
    (``flexkv/transfer/worker.py:70-76``)."""
    if handles:
        dev = handles[0].device
        if isinstance(dev, torch.device) and dev.type == "cuda":
            torch.cuda.set_device(0 if dev.index is None else dev.index)
    return [_tensor_of(h) if isinstance(h, TensorSharedHandle) else h for h in handles]
