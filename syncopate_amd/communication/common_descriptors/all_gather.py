"""All-gather plan builders: 1-D swizzle (direct), ring, double ring.

Behavioural restatement of syncopate/communication/common_descriptors/all_gather.py
(1-D swizzle :14-115, ring :129-218, double ring :221-372).  In all three,
`shape` is the shape of the GATHERED buffer; the gather axis is cut into
`mesh_size` shards and rank r owns shard r.
"""

from __future__ import annotations

from typing import Callable, List, Literal, Sequence, Tuple

import torch

from ..descriptor import BufferRegion, DevicePlan, Transfer, TransferOp, XferDependency
from .utils import axis_box, normalize_axis, row_major_strides


def _gather_setup(shape: Sequence[int], dtype: torch.dtype, axis: int, mesh_size: int, rank: int,
                  buffer_name: str, *, need_nonempty: bool
                  ) -> Tuple[DevicePlan, Callable[[int], BufferRegion], BufferRegion]:
    """Argument checks shared by the builders, the plan with the local shard registered,
    and shard_index -> BufferRegion."""
    elem_size = dtype.itemsize
    if mesh_size <= 0:
        raise ValueError("mesh_size must be positive")
    if elem_size <= 0:
        raise ValueError("elem_size must be positive")
    shape = tuple(shape)
    if not shape:
        raise ValueError("all_gather expects at least one dimension")
    axis = normalize_axis(axis, len(shape))
    if shape[axis] % mesh_size:
        raise ValueError(
            f"axis length {shape[axis]} along dim {axis} must be divisible by mesh_size {mesh_size}")
    chunk = shape[axis] // mesh_size
    if need_nonempty and chunk == 0:
        raise ValueError("all-gather requires non-empty slices along the gather axis")
    strides = row_major_strides(shape)

    def shard(index: int) -> BufferRegion:
        return BufferRegion.from_slices(elem_size=elem_size, strides=strides,
                                        slices=axis_box(shape, {axis: (index * chunk, (index + 1) * chunk)}))

    plan = DevicePlan(dev=rank)
    plan.tensors_involved[buffer_name] = (torch.Size(shape), dtype)
    own = shard(rank)
    plan.local_regions.setdefault(buffer_name, []).append(own)
    return plan, shard, own


def build_all_gather_plan_1d_swizzle(
    shape: Sequence[int],
    dtype: torch.dtype,
    axis: int,
    mesh_size: int,
    rank: int,
    buffer_name: str = "buffer",
    transfer_kind: Literal["push", "pull"] = "pull",
) -> DevicePlan:
    """Every rank talks to peers (rank+1), (rank+2), ... in turn: it pulls each peer's
    shard, or pushes its own shard to each peer (all_gather.py:79-113)."""
    # the reference validates transfer_kind after it has built the local region
    plan, shard, own = _gather_setup(shape, dtype, axis, mesh_size, rank, buffer_name, need_nonempty=False)
    if transfer_kind not in {"push", "pull"}:
        raise ValueError("transfer_kind must be 'push' or 'pull'")
    for step in range(1, mesh_size):
        peer = (rank + step) % mesh_size
        if transfer_kind == "pull":
            theirs = shard(peer)
            op = Transfer(op=TransferOp.PULL, src_buf=buffer_name, src_region=theirs, dst_buf=buffer_name,
                          dst_region=theirs, chunk_idx=peer, peer=peer)
        else:
            op = Transfer(op=TransferOp.PUSH, src_buf=buffer_name, src_region=own, dst_buf=buffer_name,
                          dst_region=own, chunk_idx=rank, peer=peer)
        plan.add_op(op)
    return plan


def build_ring_all_gather_plan(
    shape: Sequence[int],
    dtype: torch.dtype,
    axis: int,
    mesh_size: int,
    rank: int,
    buffer_name: str = "buffer",
) -> DevicePlan:
    """Ring of pushes to (rank+1): step s forwards the shard of rank (rank-s), which (for
    s > 0) must first have arrived from (rank-1)'s step s-1 (all_gather.py:189-216)."""
    plan, shard, _ = _gather_setup(shape, dtype, axis, mesh_size, rank, buffer_name, need_nonempty=True)
    if mesh_size == 1:
        return plan
    downstream = (rank + 1) % mesh_size
    upstream = (rank - 1) % mesh_size
    for step in range(mesh_size - 1):
        owner = (rank - step) % mesh_size
        waits: List[XferDependency] = []
        if step > 0:
            waits.append(XferDependency(depend_rank=upstream, depend_xfer_stream=0, depend_xfer_idx=step - 1))
        region = shard(owner)
        plan.add_op(Transfer(op=TransferOp.PUSH, src_buf=buffer_name, src_region=region, dst_buf=buffer_name,
                             dst_region=region, chunk_idx=owner, peer=downstream, dependency=waits))
    return plan


def build_double_ring_all_gather_plan(
    shape: Sequence[int],
    dtype: torch.dtype,
    axis: int,
    mesh_size: int,
    inner_mesh_size: int,
    rank: int,
    buffer_name: str = "buffer",
) -> DevicePlan:
    """Two-level ring (all_gather.py:290-370).  Ranks form contiguous groups of
    `inner_mesh_size`.  For outer step o the shards of group (g-o) circulate once round
    the inner ring (inner_mesh_size-1 pushes to the inner neighbour) and, except on the
    last outer step, one more push hands a shard on to the same inner position of group
    g+1.  Every rank therefore issues inner_mesh_size ops per outer step, which is what
    the dependency indices below count in."""
    if mesh_size > 0 and inner_mesh_size <= 0:
        raise ValueError("inner_mesh_size must be positive")
    if mesh_size > 0 and inner_mesh_size > 0 and mesh_size % inner_mesh_size:
        raise ValueError("mesh_size must be divisible by inner_mesh_size")
    plan, shard, _ = _gather_setup(shape, dtype, axis, mesh_size, rank, buffer_name, need_nonempty=True)
    if mesh_size == 1:
        return plan

    inner = inner_mesh_size
    groups = mesh_size // inner
    g, i = divmod(rank, inner)
    inner_next = g * inner + (i + 1) % inner
    inner_prev = g * inner + (i - 1) % inner
    outer_next = ((g + 1) % groups) * inner + i
    outer_prev = ((g - 1) % groups) * inner + i
    per_outer = inner

    def after(peer: int, op_idx: int) -> List[XferDependency]:
        return [XferDependency(depend_rank=peer, depend_xfer_stream=0, depend_xfer_idx=op_idx)]

    for o in range(groups):
        source_group = (g - o) % groups
        # the shard this outer step starts from arrived over the outer ring (none for o == 0)
        from_outer: List[XferDependency] = after(outer_prev, o * per_outer - 1) if o > 0 else []
        tag = source_group * inner + i

        for s in range(inner - 1):
            owner = source_group * inner + (i + o - s) % inner
            waits = from_outer if s == 0 else after(inner_prev, o * per_outer + s - 1)
            region = shard(owner)
            plan.add_op(Transfer(op=TransferOp.PUSH, src_buf=buffer_name, src_region=region,
                                 dst_buf=buffer_name, dst_region=region, chunk_idx=tag, peer=inner_next,
                                 dependency=waits))

        if o < groups - 1:
            owner = source_group * inner + (i + o + 1) % inner
            waits = from_outer if inner == 1 else after(inner_prev, o * per_outer + (inner - 2))
            region = shard(owner)
            plan.add_op(Transfer(op=TransferOp.PUSH, src_buf=buffer_name, src_region=region,
                                 dst_buf=buffer_name, dst_region=region, chunk_idx=tag, peer=outer_next,
                                 dependency=waits))
    return plan


__all__ = [
    "build_all_gather_plan_1d_swizzle",
    "build_ring_all_gather_plan",
    "build_double_ring_all_gather_plan",
]
