"""All-reduce plan builders: the tensor is cut into `num_all_reduces` slabs along `split_axis`
and every slab becomes one library collective, optionally gated on the local producer's tiles.

Behavioural restatement of `build_all_reduce_plan` (in place, one buffer) and
`build_all_reduce_nvsharp_plan` (separate source and destination buffers, for a switch-reduced
all-reduce) - syncopate/communication/common_descriptors/all_reduce.py:13-113 and :116-212.
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from ..descriptor import BufferRegion, Collective, CollectiveOp, ComputeDependency, DevicePlan
from .utils import axis_box, ensure_divisible, row_major_strides


def split_slabs(shape: Sequence[int], split_axis: Optional[int], pieces: int, what: str,
                kind: str) -> Tuple[int, List[Tuple[int, int]]]:
    """Normalised split axis and the (start, end) of each of `pieces` equal slabs along it."""
    ndim = len(shape)
    if ndim == 0:
        raise ValueError(f"{kind} expects at least one dimension")
    if split_axis is None:
        if pieces != 1:
            raise ValueError(f"split_axis is required when {what} > 1")
        split_axis = 0
    if split_axis < 0:
        split_axis += ndim
    if not 0 <= split_axis < ndim:
        raise IndexError(f"split_axis {split_axis} out of range for tensor with {ndim} dims")
    ensure_divisible(shape[split_axis], pieces, what)
    width = shape[split_axis] // pieces
    if width == 0:
        raise ValueError("split produces empty chunks")
    return split_axis, [(i * width, (i + 1) * width) for i in range(pieces)]


def _check_counts(dtype: torch.dtype, mesh_size: int, pieces: int, what: str) -> int:
    if mesh_size <= 0:
        raise ValueError("mesh_size must be positive")
    if dtype.itemsize <= 0:
        raise ValueError("elem_size must be positive")
    if pieces <= 0:
        raise ValueError(f"{what} must be positive")
    return dtype.itemsize


def _all_reduce(shape: Sequence[int], dtype: torch.dtype, mesh_size: int, rank: int, src: str, dst: str,
                op: CollectiveOp, pieces: int, split_axis: Optional[int], compute_producer: bool,
                resident: bool) -> DevicePlan:
    elem_size = _check_counts(dtype, mesh_size, pieces, "num_all_reduces")
    shape = tuple(shape)
    split_axis, slabs = split_slabs(shape, split_axis, pieces, "num_all_reduces", "all_reduce")
    strides = row_major_strides(shape)
    plan = DevicePlan(dev=rank)
    for name in (src, dst):
        plan.tensors_involved[name] = (torch.Size(shape), dtype)
    if resident:
        plan.local_regions.setdefault(src, []).append(
            BufferRegion.from_slices(elem_size=elem_size, strides=strides, slices=axis_box(shape, {})))
    for cut in slabs:
        region = BufferRegion.from_slices(elem_size=elem_size, strides=strides,
                                          slices=axis_box(shape, {split_axis: cut}))
        gate = [ComputeDependency(compute_rank=rank, src_region=region)] if compute_producer else []
        plan.add_op(Collective(op=op, src_buf=src, src_region=region, dst_buf=dst, dst_region=region,
                               dependency=gate))
    return plan


def build_all_reduce_plan(shape: Sequence[int], *, dtype: torch.dtype, mesh_size: int, rank: int,
                          buffer_name: str, num_all_reduces: int = 1, split_axis: Optional[int] = None,
                          compute_producer: bool = False) -> DevicePlan:
    """In-place all-reduce of `buffer_name`, one collective per slab."""
    return _all_reduce(shape, dtype, mesh_size, rank, buffer_name, buffer_name, CollectiveOp.ALL_REDUCE,
                       num_all_reduces, split_axis, compute_producer, resident=True)


def build_all_reduce_nvsharp_plan(shape: Sequence[int], *, dtype: torch.dtype, mesh_size: int, rank: int,
                                  src_name: str, dst_name: str, num_all_reduces: int = 1,
                                  split_axis: Optional[int] = None,
                                  compute_producer: bool = False) -> DevicePlan:
    """All-reduce from `src_name` into `dst_name` (two buffers), one collective per slab."""
    return _all_reduce(shape, dtype, mesh_size, rank, src_name, dst_name, CollectiveOp.ALL_REDUCE_NVSHARP,
                       num_all_reduces, split_axis, compute_producer, resident=False)


__all__ = ["build_all_reduce_plan", "build_all_reduce_nvsharp_plan"]
