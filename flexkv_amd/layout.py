"""KV-cache layouts and the byte strides the transfer path is driven with.

Host-side mirror of the part of FlexKV's ``flexkv/common/storage.py`` that the
GPU<->CPU transfer workers consume (``KVCacheLayout`` and its stride getters,
storage.py:87-247), of the stride probe the worker runs on a real engine
tensor (``flexkv/transfer/worker.py:262-306``) and of the rule that derives the
GPU addressing mode from the number of engine tensors (``worker.py:804-814``,
``csrc/tp_transfer_thread_group.cpp:71-80``).

All getters return ELEMENT counts like the reference; multiply by
``dtype.itemsize`` for bytes (``TransferStrides`` does that).

Models whose layers do not share one KV shape (a latent cache plus an indexer
cache on the same layer, groups compressed along the token axis) are described
by ``LayerGroupSpec`` / ``LayerMemberMap`` (``flexkv/common/config.py:33-119``)
and stored in byte-flat host blocks, ``MultiGroupBlockLayout``
(storage.py:87-127, 249-286); ``multi_group_tables`` produces the per-group
arrays the layerwise restore is constructed with
(``flexkv/transfer/layerwise.py:431-537``).
"""
from __future__ import annotations

import enum
from dataclasses import dataclass, replace
from typing import Dict, List, Optional, Sequence, Tuple


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


# ---- heterogeneous layer groups -------------------------------------------------

@dataclass(frozen=True)
class LayerGroupSpec:
    """Layers that share one KV shape (config.py:33-65).

    ``layer_indices[k]`` is the original layer the group's k-th layer belongs to;
    several groups may name the same original layer.  ``itemsize`` is the byte
    width of the group's storage dtype; ``compress_ratio`` divides
    ``tokens_per_block`` for this group.
    """
    num_layers: int
    num_kv_heads: int
    head_size: int
    layer_indices: Tuple[int, ...]
    itemsize: int = 2
    compress_ratio: int = 1

    def __post_init__(self) -> None:
        object.__setattr__(self, "layer_indices", tuple(self.layer_indices))
        if self.num_layers != len(self.layer_indices):
            raise ValueError("num_layers must equal len(layer_indices)")
        if len(set(self.layer_indices)) != len(self.layer_indices):
            raise ValueError("layer_indices must not repeat inside one group")


@dataclass(frozen=True)
class LayerMemberMap:
    """``members[i]``: the (group, layer-inside-group) pairs of original layer i,
    by ascending group (config.py:68-99)."""
    members: Tuple[Tuple[Tuple[int, int], ...], ...]

    @property
    def num_original_layers(self) -> int:
        return len(self.members)

    def members_of(self, original_layer_id: int) -> Tuple[Tuple[int, int], ...]:
        return self.members[original_layer_id]


def build_layer_member_map(layer_groups: Sequence[LayerGroupSpec],
                           num_original_layers: int) -> LayerMemberMap:
    """config.py:102-119."""
    buckets: List[List[Tuple[int, int]]] = [[] for _ in range(num_original_layers)]
    for gi, g in enumerate(layer_groups):
        for local_id, orig in enumerate(g.layer_indices):
            if not 0 <= orig < num_original_layers:
                raise ValueError(f"layer_groups[{gi}] names original layer {orig} outside "
                                 f"[0, {num_original_layers})")
            buckets[orig].append((gi, local_id))
    return LayerMemberMap(tuple(tuple(sorted(b, key=lambda m: m[0])) for b in buckets))


@dataclass(frozen=True)
class MultiGroupBlockLayout:
    """Byte-flat BLOCKFIRST host pool of a multi-group model: block b holds, group
    after group, ``[layer-in-group, kv, token, head, dim]`` of every group, once
    per tensor-parallel rank (storage.py:87-127)."""
    num_block: int
    tokens_per_block: int
    layer_groups: Tuple[LayerGroupSpec, ...]
    kv_dim: int = 1
    tp_size: int = 1

    def __post_init__(self) -> None:
        object.__setattr__(self, "layer_groups", tuple(self.layer_groups))
        for gi, g in enumerate(self.layer_groups):
            if self.tokens_per_block % g.compress_ratio:
                raise ValueError(
                    f"layer_groups[{gi}].compress_ratio={g.compress_ratio} does not divide "
                    f"tokens_per_block={self.tokens_per_block}")

    def group_chunk_bytes(self, gi: int) -> int:
        g = self.layer_groups[gi]
        return (self.tokens_per_block // g.compress_ratio) * g.num_kv_heads * g.head_size \
            * g.itemsize

    def get_block_stride(self) -> int:
        """Bytes per block (storage.py:120-127, 222-226)."""
        return self.tp_size * sum(g.num_layers * self.kv_dim * self.group_chunk_bytes(gi)
                                  for gi, g in enumerate(self.layer_groups))

    @property
    def kv_shape(self) -> Tuple[int, int]:
        return (self.num_block, self.get_block_stride())

    def get_group_strides(self) -> List[Dict[str, int]]:
        """Per group, in bytes: offset inside a block, layer / kv strides and chunk
        size (storage.py:249-286, there in elements of the group's dtype)."""
        out, offset = [], 0
        for gi, g in enumerate(self.layer_groups):
            chunk = self.group_chunk_bytes(gi)
            layer_stride = self.kv_dim * chunk
            out.append({"num_layers": g.num_layers, "offset_bytes": offset,
                        "layer_stride": layer_stride, "kv_stride": chunk, "chunk_size": chunk})
            offset += g.num_layers * layer_stride
        return out


def multi_group_tables(cpu_layout: MultiGroupBlockLayout, num_original_layers: int,
                       gpu_layouts_per_group: Sequence[Sequence[KVCacheLayout]],
                       tp_group_size: int = 1) -> Dict[str, object]:
    """The per-group arrays of the multi-group ``LayerwiseTransferGroup``
    constructor and of ``init_swa_multi_group`` (layerwise.py:431-537).
    ``gpu_layouts_per_group[gi][d]`` is the device layout of group gi on GPU d;
    the per-GPU arrays are flattened group-major."""
    member_map = build_layer_member_map(cpu_layout.layer_groups, num_original_layers)
    block_stride = cpu_layout.get_block_stride()
    tp_stride = block_stride // tp_group_size
    t: Dict[str, list] = {k: [] for k in (
        "group_num_layers", "group_cpu_offset_bytes", "group_ssd_offset_bytes",
        "group_cpu_layer_strides", "group_cpu_kv_strides", "group_ssd_layer_strides",
        "group_ssd_kv_strides", "group_chunk_sizes", "group_h2d_cpu_kv_strides",
        "group_h2d_cpu_layer_strides", "group_cpu_block_strides", "group_cpu_tp_strides",
        "group_gpu_kv_strides", "group_gpu_block_strides", "group_gpu_layer_strides",
        "group_gpu_chunk_sizes")}
    for gi, (g, st) in enumerate(zip(cpu_layout.layer_groups, cpu_layout.get_group_strides())):
        t["group_num_layers"].append(g.num_layers)
        t["group_cpu_offset_bytes"].append(st["offset_bytes"])
        t["group_ssd_offset_bytes"].append(st["offset_bytes"])
        for k in ("group_cpu_layer_strides", "group_ssd_layer_strides",
                  "group_h2d_cpu_layer_strides"):
            t[k].append(st["layer_stride"])
        for k in ("group_cpu_kv_strides", "group_ssd_kv_strides", "group_h2d_cpu_kv_strides"):
            t[k].append(st["kv_stride"])
        t["group_chunk_sizes"].append(st["chunk_size"])
        t["group_cpu_block_strides"].append(block_stride)
        t["group_cpu_tp_strides"].append(tp_stride)
        for layout in gpu_layouts_per_group[gi]:
            s = TransferStrides.from_layout(layout, g.itemsize)
            t["group_gpu_kv_strides"].append(s.kv)
            t["group_gpu_block_strides"].append(s.block)
            t["group_gpu_layer_strides"].append(s.layer)
            t["group_gpu_chunk_sizes"].append(s.chunk)
    out: Dict[str, object] = dict(t)
    out["layer_members"] = [list(m) for m in member_map.members]
    out["layer_member_map"] = member_map
    out["cpu_block_stride"] = block_stride
    out["cpu_tp_stride"] = tp_stride
    return out
