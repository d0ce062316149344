"""Reduce-scatter plan builders.

Direct-reduce form: every rank ships (with a reduce op) the chunk each peer owns straight into
that peer's output, then reduces its own chunk locally - `build_reduce_scatter_direct_reduce_plan`
(syncopate/communication/common_descriptors/reduce_scatter.py:161-304).

Collective form: the tensor is cut into slabs along an axis other than the scattered one and every
slab becomes one library reduce-scatter - `build_reduce_scatter_collective_plan`
(reduce_scatter.py:22-158).
"""

from __future__ import annotations

from typing import Literal, Optional, Sequence

import torch

from ..descriptor import (
    BufferRegion,
    Collective,
    CollectiveOp,
    ComputeDependency,
    DevicePlan,
    ReduceOp,
    Transfer,
    TransferOp,
)
from .utils import axis_box, ensure_divisible, row_major_strides


def build_reduce_scatter_direct_reduce_plan(
    shape: Sequence[int],
    *,
    dtype: torch.dtype,
    axis: int,
    mesh_size: int,
    rank: int,
    src_buffer: str,
    dst_buffer: str,
    reduce_op: ReduceOp = ReduceOp.SUM,
    transfer_kind: Literal["push", "pull"] = "push",
) -> DevicePlan:
    elem_size = dtype.itemsize
    if mesh_size <= 0:
        raise ValueError("mesh_size must be positive")
    if elem_size <= 0:
        raise ValueError("elem_size must be positive")
    if rank < 0 or rank >= mesh_size:
        raise ValueError("rank must be in [0, mesh_size)")
    shape = tuple(shape)
    ndim = len(shape)
    if ndim == 0:
        raise ValueError("reduce_scatter expects at least one dimension")
    if axis < 0:
        axis += ndim
    if not 0 <= axis < ndim:
        raise IndexError(f"axis {axis} out of range for tensor with {ndim} dims")
    ensure_divisible(shape[axis], mesh_size, axis)
    per_rank = shape[axis] // mesh_size
    if per_rank == 0:
        raise ValueError("reduce_scatter requires non-empty slices along the reduce axis")
    if transfer_kind not in {"push", "pull"}:
        raise ValueError("transfer_kind must be 'push' or 'pull'")

    dst_shape = tuple(per_rank if a == axis else extent for a, extent in enumerate(shape))
    src_strides = row_major_strides(shape)
    dst_strides = row_major_strides(dst_shape)

    plan = DevicePlan(dev=rank)
    plan.tensors_involved[src_buffer] = (torch.Size(shape), dtype)
    plan.tensors_involved[dst_buffer] = (torch.Size(dst_shape), dtype)
    # the whole partial result is resident in the source buffer
    plan.local_regions.setdefault(src_buffer, []).append(
        BufferRegion.from_slices(elem_size=elem_size, strides=src_strides, slices=axis_box(shape, {})))

    def chunk_of(owner: int) -> BufferRegion:
        return BufferRegion.from_slices(
            elem_size=elem_size, strides=src_strides,
            slices=axis_box(shape, {axis: (owner * per_rank, (owner + 1) * per_rank)}))

    whole_dst = BufferRegion.from_slices(elem_size=elem_size, strides=dst_strides,
                                         slices=axis_box(dst_shape, {}))
    own_chunk = chunk_of(rank)

    for step in range(mesh_size - 1):
        peer = (rank + step + 1) % mesh_size
        if transfer_kind == "push":
            outgoing = chunk_of(peer)
            plan.add_op(Transfer(op=TransferOp.PUSH, src_buf=src_buffer, src_region=outgoing,
                                 dst_buf=dst_buffer, dst_region=whole_dst, chunk_idx=step, peer=peer,
                                 dependency=[ComputeDependency(compute_rank=rank, src_region=outgoing)],
                                 reduce_op=reduce_op))
        else:
            plan.add_op(Transfer(op=TransferOp.PULL, src_buf=src_buffer, src_region=own_chunk,
                                 dst_buf=dst_buffer, dst_region=whole_dst, chunk_idx=step, peer=peer,
                                 dependency=[ComputeDependency(compute_rank=peer, src_region=own_chunk)],
                                 reduce_op=reduce_op))

    plan.add_op(Transfer(op=TransferOp.LOCAL_COPY, src_buf=src_buffer, src_region=own_chunk,
                         dst_buf=dst_buffer, dst_region=whole_dst, chunk_idx=mesh_size - 1,
                         dependency=[ComputeDependency(compute_rank=rank, src_region=own_chunk)],
                         reduce_op=reduce_op))
    return plan


def build_reduce_scatter_collective_plan(
    shape: Sequence[int],
    *,
    dtype: torch.dtype,
    axis: int,
    split_axis: Optional[int] = None,
    mesh_size: int,
    rank: int,
    src_buffer: str,
    dst_buffer: str,
    num_reduce_scatters: int = 1,
    compute_producer: bool = False,
) -> DevicePlan:
    """Reduce along `axis` and scatter it over the mesh, `num_reduce_scatters` collectives over
    equal slabs of `split_axis` (any axis but `axis`; the one behind `axis`, else the first, when
    there is a single collective and none is named)."""
    elem_size = dtype.itemsize
    if mesh_size <= 0:
        raise ValueError("mesh_size must be positive")
    if elem_size <= 0:
        raise ValueError("elem_size must be positive")
    if num_reduce_scatters <= 0:
        raise ValueError("num_reduce_scatters must be positive")
    shape = tuple(shape)
    ndim = len(shape)
    if ndim == 0:
        raise ValueError("reduce_scatter expects at least one dimension")
    if axis < 0:
        axis += ndim
    if not 0 <= axis < ndim:
        raise IndexError(f"axis {axis} out of range for tensor with {ndim} dims")
    ensure_divisible(shape[axis], mesh_size, axis)
    per_rank = shape[axis] // mesh_size

    if split_axis is None:
        if num_reduce_scatters != 1:
            raise ValueError("split_axis is required when num_reduce_scatters > 1")
        split_axis = (axis + 1) % ndim
    if split_axis < 0:
        split_axis += ndim
    if not 0 <= split_axis < ndim:
        raise IndexError(f"split_axis {split_axis} out of range for tensor with {ndim} dims")
    if split_axis == axis:
        raise ValueError("split_axis must differ from reduce axis")
    ensure_divisible(shape[split_axis], num_reduce_scatters, "num_reduce_scatters")
    width = shape[split_axis] // num_reduce_scatters
    if width == 0:
        raise ValueError("split produces empty chunks")

    dst_shape = tuple(per_rank if a == axis else extent for a, extent in enumerate(shape))
    src_strides = row_major_strides(shape)
    dst_strides = row_major_strides(dst_shape)

    plan = DevicePlan(dev=rank)
    plan.tensors_involved[src_buffer] = (torch.Size(shape), dtype)
    plan.tensors_involved[dst_buffer] = (torch.Size(dst_shape), dtype)
    plan.local_regions.setdefault(src_buffer, []).append(
        BufferRegion.from_slices(elem_size=elem_size, strides=src_strides, slices=axis_box(shape, {})))

    for i in range(num_reduce_scatters):
        cut = {split_axis: (i * width, (i + 1) * width)}
        src_region = BufferRegion.from_slices(elem_size=elem_size, strides=src_strides,
                                              slices=axis_box(shape, cut))
        dst_region = BufferRegion.from_slices(elem_size=elem_size, strides=dst_strides,
                                              slices=axis_box(dst_shape, cut))
        gate = [ComputeDependency(compute_rank=rank, src_region=src_region)] if compute_producer else []
        plan.add_op(Collective(op=CollectiveOp.REDUCE_SCATTER, src_buf=src_buffer, src_region=src_region,
                               dst_buf=dst_buffer, dst_region=dst_region, dependency=gate))
    return plan


__all__ = ["build_reduce_scatter_collective_plan", "build_reduce_scatter_direct_reduce_plan"]
