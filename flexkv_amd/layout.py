"""KV-cache layouts and the byte strides the transfer path is driven with.

Host-side mirror of the part of FlexKV's ``flexkv/common/storage.py`` that the
GPU<->CPU transfer workers consume (``KVCacheLayout`` and its stride getters,
storage.py:87-247), of the stride probe the worker runs on a real engine
tensor (``flexkv/transfer/worker.py:262-306``) and of the rule that derives the
GPU addressing mode from the number of engine tensors (``worker.py:804-814``,
``csrc/tp_transfer_thread_group.cpp:71-80``).

All getters return ELEMENT counts like the reference; multiply by
``dtype.itemsize`` for bytes (``TransferStrides`` does that).
"""
from __future__ import annotations

import enum
from dataclasses import dataclass, replace
from typing import Optional, Sequence, Tuple


class KVCacheLayoutType(enum.Enum):
    LAYERFIRST = "LAYERFIRST"   # [layer, kv, block, token, head, dim]
    BLOCKFIRST = "BLOCKFIRST"   # [block, layer, kv, token, head, dim]
    LAYERBLOCK = "LAYERBLOCK"   # [layer, block, kv, token, head, dim]


# axis order of each layout, as names
_AXES = {
    KVCacheLayoutType.LAYERFIRST: ("layer", "kv", "block", "token", "head", "dim"),
    KVCacheLayoutType.BLOCKFIRST: ("block", "layer", "kv", "token", "head", "dim"),
    KVCacheLayoutType.LAYERBLOCK: ("layer", "block", "kv", "token", "head", "dim"),
}

GPU_BLOCK_TYPE_VLLM = 0
GPU_BLOCK_TYPE_TRTLLM = 1
GPU_BLOCK_TYPE_SGLANG = 2


@dataclass(frozen=True)
class KVCacheLayout:
    """Dense 6-D KV cache of one pool (storage.py:33-63).

    ``kv_dim`` is 2 when K and V are separate planes and 1 when they are packed
    (MLA latent cache, packed MHA).  ``num_kv_heads == 1`` marks KV that is
    identical on every tensor-parallel rank.
    """
    type: KVCacheLayoutType
    num_layer: int
    num_block: int
    tokens_per_block: int
    num_head: int
    head_size: int
    kv_dim: int = 2
    num_kv_heads: int = 1

    def _extent(self, axis: str) -> int:
        return {"layer": self.num_layer, "kv": self.kv_dim, "block": self.num_block,
                "token": self.tokens_per_block, "head": self.num_head,
                "dim": self.head_size}[axis]

    @property
    def kv_shape(self) -> Tuple[int, ...]:
        """storage.py:128-148."""
        return tuple(self._extent(a) for a in _AXES[self.type])

    def _stride_of(self, axis: str) -> int:
        axes = _AXES[self.type]
        n = 1
        for a in axes[axes.index(axis) + 1:]:
            n *= self._extent(a)
        return n

    def get_chunk_size(self) -> int:
        """Elements of one (layer, k-or-v, block): storage.py:203-207."""
        return self.tokens_per_block * self.num_head * self.head_size

    def get_layer_stride(self) -> int:
        """storage.py:209-220."""
        return self._stride_of("layer")

    def get_kv_stride(self) -> int:
        """storage.py:236-247."""
        return self._stride_of("kv")

    def get_block_stride(self) -> int:
        """storage.py:222-234."""
        return self._stride_of("block")

    def get_total_elements(self) -> int:
        n = 1
        for e in self.kv_shape:
            n *= e
        return n

    def div_head(self, num_chunks: int) -> "KVCacheLayout":
        """Per-rank view after a tensor-parallel head split (storage.py:188-201)."""
        if self.num_head % num_chunks:
            raise ValueError(f"num_head {self.num_head} must be divisible by {num_chunks}")
        return replace(self, num_head=self.num_head // num_chunks)

    def div_block(self, num_chunks: int, padding: bool = False) -> "KVCacheLayout":
        """storage.py:152-171."""
        if padding:
            nb = -(-self.num_block // num_chunks)
        else:
            if self.num_block % num_chunks:
                raise ValueError(
                    f"num_block {self.num_block} must be divisible by {num_chunks}")
            nb = self.num_block // num_chunks
        return replace(self, num_block=nb)

    def div_layer(self, num_chunks: int) -> "KVCacheLayout":
        """storage.py:173-186."""
        if self.num_layer % num_chunks:
            raise ValueError(f"num_layer {self.num_layer} must be divisible by {num_chunks}")
        return replace(self, num_layer=self.num_layer // num_chunks)


@dataclass(frozen=True)
class TransferStrides:
    """Byte strides of one side of a transfer."""
    kv: int
    block: int
    layer: int
    chunk: int

    @classmethod
    def from_layout(cls, layout: KVCacheLayout, itemsize: int) -> "TransferStrides":
        return cls(kv=layout.get_kv_stride() * itemsize,
                   block=layout.get_block_stride() * itemsize,
                   layer=layout.get_layer_stride() * itemsize,
                   chunk=layout.get_chunk_size() * itemsize)


def gpu_strides_from_tensor(shape: Sequence[int], stride: Sequence[int],
                            tokens_per_block: int, itemsize: int,
                            kv_dim: int) -> Optional[Tuple[int, int, int]]:
    """(kv_stride, block_stride, layer_stride) in bytes of one per-layer engine
    tensor, from its real shape/stride (worker.py:262-306).

    Engines order the first three axes of the 5-D per-layer tensor differently
    (``[2, N, T, H, D]`` for flash-attn, ``[N, 2, T, H, D]`` for
    triton/flashinfer).  The axis of extent 2 is K/V, the axis whose extent is
    ``tokens_per_block`` is the token axis, the remaining one is the block
    axis.  Returns None (caller falls back to the layout's closed forms) when
    ``kv_dim == 1``, the tensor is not 5-D, or the axes cannot be told apart.
    """
    if kv_dim == 1 or len(shape) != 5:
        return None
    lead = list(shape[:3])
    kv_axis = next((i for i in range(3) if lead[i] == 2), None)
    if kv_axis is None:
        return None
    tok_axis = next((i for i in range(3) if i != kv_axis and lead[i] == tokens_per_block),
                    None)
    blk_axis = next((i for i in range(3) if i != kv_axis and i != tok_axis), None)
    if blk_axis is None:
        return None
    numel = 1
    for e in shape:
        numel *= e
    return (stride[kv_axis] * itemsize, stride[blk_axis] * itemsize, numel * itemsize)


def gpu_block_type_from_tensor_count(num_tensors: int, num_layers: int) -> int:
    """1 tensor -> TRT-LLM, L tensors -> vLLM, 2L tensors -> SGLang
    (worker.py:804-814; csrc/tp_transfer_thread_group.cpp:71-80)."""
    if num_tensors == 1:
        return GPU_BLOCK_TYPE_TRTLLM
    if num_tensors == num_layers:
        return GPU_BLOCK_TYPE_VLLM
    if num_tensors == 2 * num_layers:
        return GPU_BLOCK_TYPE_SGLANG
    raise ValueError(f"Invalid GPU block type: {num_tensors} tensors for {num_layers} layers")
