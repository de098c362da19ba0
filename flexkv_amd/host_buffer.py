"""Host-pool memory for the transfer path.

Mirror of the functions of ``flexkv/transfer/host_buffer.py`` that the
GPU<->CPU workers use: chunked registration of an existing host tensor
(``cudaHostRegister`` / ``cudaHostUnregister``, host_buffer.py:66-118, names
kept so the reference's worker code reads unchanged) and allocation of a
mapped pinned tensor that device kernels can store into
(``alloc_mapped_host_tensor``, host_buffer.py:180-202).
"""
from __future__ import annotations

import ctypes
import os
import weakref

import numpy as np
import torch

from . import _lib
from ._lib import check

_L = _lib.load()


def _chunk_bytes() -> int:
    """FLEXKV_CUDAHOST_CHUNK_SIZE_GB -> bytes per registration call (0 = one call)."""
    return int(_L.fkv_host_chunk_bytes_from_gb(
        float(os.getenv("FLEXKV_CUDAHOST_CHUNK_SIZE_GB", "0"))))


def cudaHostRegister(tensor: torch.Tensor) -> None:
    """Pin + map an existing host tensor for device access, in chunks when
    FLEXKV_CUDAHOST_CHUNK_SIZE_GB is set; already-registered chunks are rolled
    back if a later one fails."""
    nbytes = tensor.numel() * tensor.element_size()
    check(_L.fkv_host_register(tensor.data_ptr(), nbytes, _chunk_bytes()))


def cudaHostUnregister(tensor: torch.Tensor) -> None:
    nbytes = tensor.numel() * tensor.element_size()
    check(_L.fkv_host_unregister(tensor.data_ptr(), nbytes, _chunk_bytes()))


hipHostRegister = cudaHostRegister
hipHostUnregister = cudaHostUnregister


def alloc_mapped_host_tensor(num_elements: int, dtype: torch.dtype) -> torch.Tensor:
    """Pinned, device-mapped host tensor (hipHostMalloc Portable|Mapped); freed
    when the last tensor that views the allocation is garbage collected."""
    nbytes = int(num_elements) * dtype.itemsize
    ptr = ctypes.c_void_p()
    check(_L.fkv_host_alloc(nbytes, ctypes.byref(ptr)))
    raw = (ctypes.c_uint8 * nbytes).from_address(ptr.value)
    arr = np.frombuffer(raw, dtype=np.uint8, count=nbytes)
    # The storage of every view keeps `arr`, and through it `raw`, alive: the
    # allocation goes when `raw` does, not when the first tensor object does.
    weakref.finalize(raw, _L.fkv_host_free, ctypes.c_void_p(ptr.value))
    return torch.from_numpy(arr).view(dtype)[:num_elements]
