"""All-to-all plan builders.

Behavioural restatement of syncopate/communication/common_descriptors/all_to_all.py:
`build_all_to_all_plan` (dim-0 sharded, :11-169), `build_all_to_all_plan_dim`
(moves the sharding from one axis to another, :179-370), `build_all_to_all_plan_dim_waves`
(the same, with every destination shard delivered in waves, :373-572) and
`build_all_to_all_plan_axis` (exchange along one axis, source and destination of one shape,
:575-735).

Op order matters to everything downstream (signal offsets, arrival waves):
when communication produces the data a compute kernel will read
(compute_producer=False) the local copy is issued first; when a compute kernel
produces the data communication ships (compute_producer=True) every op waits
on a ComputeDependency and the local copy is issued last.
"""

from __future__ import annotations

from typing import Callable, List, Literal, Sequence

import torch

from ..descriptor import BufferRegion, ComputeDependency, DevicePlan, Transfer, TransferOp
from .utils import axis_box, block_nbytes, ensure_divisible, normalize_axis, row_major_strides


def _emit_exchange(
    plan: DevicePlan,
    *,
    rank: int,
    mesh_size: int,
    peers: Sequence[int],
    src_buffer: str,
    dst_buffer: str,
    src_region_for: Callable[[int], BufferRegion],
    dst_region_for: Callable[[int], BufferRegion],
    transfer_kind: str,
    compute_producer: bool,
) -> DevicePlan:
    """The op list common to both builders (all_to_all.py:95-169 / :291-370)."""
    own_src = src_region_for(rank)
    own_dst = dst_region_for(rank)

    def produced_by(compute_rank: int, region: BufferRegion) -> List:
        if not compute_producer:
            return []
        return [ComputeDependency(compute_rank=compute_rank, src_region=region, signal=None)]

    local_copy = Transfer(op=TransferOp.LOCAL_COPY, src_buf=src_buffer, dst_buf=dst_buffer,
                          src_region=own_src, dst_region=own_dst, chunk_idx=-1,
                          dependency=produced_by(rank, own_src))
    if not compute_producer:
        plan.add_op(local_copy, stream_idx=0)

    for peer in peers:
        if transfer_kind == "push":
            # my slice for `peer` lands in the slot of `rank` in peer's destination
            outgoing = src_region_for(peer)
            op = Transfer(op=TransferOp.PUSH, src_buf=src_buffer, src_region=outgoing, peer=peer,
                          chunk_idx=rank * mesh_size + peer, dst_buf=dst_buffer, dst_region=own_dst,
                          dependency=produced_by(rank, src_region_for(peer)))
        else:
            # peer's slice for me (same box as my own source slice) lands in peer's slot here
            op = Transfer(op=TransferOp.PULL, dst_buf=dst_buffer, dst_region=dst_region_for(peer), peer=peer,
                          chunk_idx=peer * mesh_size + rank, src_buf=src_buffer, src_region=own_src,
                          dependency=produced_by(peer, own_src))
        plan.add_op(op)

    if compute_producer:
        plan.add_op(local_copy)
    return plan


def build_all_to_all_plan(
    shape: Sequence[int],
    *,
    dtype: torch.dtype,
    mesh_size: int,
    rank: int,
    src_buffer: str,
    dst_buffer: str,
    transfer_kind: Literal["push", "pull"] = "push",
    compute_producer: bool = False,
) -> DevicePlan:
    """`shape` is the local source tensor, dim 0 split into one slice per destination;
    the destination is laid out (mesh_size, shape[0]/mesh_size, *shape[1:]) with slot s
    holding what rank s sent."""
    elem_size = dtype.itemsize
    if mesh_size <= 0:
        raise ValueError("mesh_size must be positive")
    if elem_size <= 0:
        raise ValueError("elem_size must be positive")
    shape = tuple(shape)
    if not shape:
        raise ValueError("all_to_all expects at least one dimension in the source shape")
    ensure_divisible(shape[0], mesh_size, axis=0)
    chunk = shape[0] // mesh_size
    if chunk == 0:
        raise ValueError("all-to-all requires non-empty slices along dim0")
    if block_nbytes(shape, elem_size, {0: chunk}) == 0:
        raise ValueError("all-to-all transfer would be empty")

    dst_shape = (mesh_size, chunk, *shape[1:])
    src_strides = row_major_strides(shape)
    dst_strides = row_major_strides(dst_shape)

    def src_region_for(dest_peer: int) -> BufferRegion:
        return BufferRegion.from_slices(
            elem_size=elem_size, strides=src_strides,
            slices=axis_box(shape, {0: (dest_peer * chunk, (dest_peer + 1) * chunk)}))

    def dst_region_for(source_rank: int) -> BufferRegion:
        return BufferRegion.from_slices(
            elem_size=elem_size, strides=dst_strides,
            slices=axis_box(dst_shape, {0: (source_rank, source_rank + 1)}))

    plan = DevicePlan(dev=rank)
    plan.src_shape = shape          # read by callers (and the reference's tests)
    plan.dst_shape = dst_shape
    plan.tensors_involved[src_buffer] = (torch.Size(shape), dtype)
    plan.tensors_involved[dst_buffer] = (torch.Size(dst_shape), dtype)
    plan.local_regions.setdefault(src_buffer, []).append(src_region_for(rank))

    if transfer_kind not in {"push", "pull"}:
        raise ValueError("transfer_kind must be 'push' or 'pull'")
    peers = [(rank + step) % mesh_size for step in range(1, mesh_size)]
    return _emit_exchange(plan, rank=rank, mesh_size=mesh_size, peers=peers, src_buffer=src_buffer,
                          dst_buffer=dst_buffer, src_region_for=src_region_for,
                          dst_region_for=dst_region_for, transfer_kind=transfer_kind,
                          compute_producer=compute_producer)


def build_all_to_all_plan_dim(
    shape: Sequence[int],
    *,
    dtype: torch.dtype,
    mesh_size: int,
    rank: int,
    src_buffer: str,
    dst_buffer: str,
    src_split_axis: int,
    dst_split_axis: int,
    transfer_kind: Literal["push", "pull"] = "push",
    compute_producer: bool = False,
    peer_order: Literal["clockwise", "counter-clockwise"] = "clockwise",
) -> DevicePlan:
    """Re-shard from `src_split_axis` to `dst_split_axis`, e.g. [B, S/w, H, D] -> [B, S, H/w, D].
    `shape` is the local source shape (already cut along src_split_axis); the destination
    has the full src axis and 1/mesh_size of the dst axis."""
    elem_size = dtype.itemsize
    if mesh_size <= 0:
        raise ValueError("mesh_size must be positive")
    if elem_size <= 0:
        raise ValueError("elem_size must be positive")
    shape = tuple(shape)
    if not shape:
        raise ValueError("all_to_all expects at least one dimension in the source shape")
    ndim = len(shape)
    src_split_axis = normalize_axis(src_split_axis, ndim)
    dst_split_axis = normalize_axis(dst_split_axis, ndim)
    if src_split_axis == dst_split_axis:
        raise ValueError("src_split_axis and dst_split_axis must differ")
    src_chunk = shape[src_split_axis]
    if src_chunk <= 0:
        raise ValueError("all-to-all requires non-empty slices along the split axis")
    ensure_divisible(shape[dst_split_axis], mesh_size, axis=dst_split_axis)
    dst_chunk = shape[dst_split_axis] // mesh_size
    if dst_chunk == 0:
        raise ValueError("all-to-all requires non-empty slices along the destination axis")
    if block_nbytes(shape, elem_size, {src_split_axis: src_chunk, dst_split_axis: dst_chunk}) == 0:
        raise ValueError("all-to-all transfer would be empty")

    dst_shape = list(shape)
    dst_shape[src_split_axis] = src_chunk * mesh_size
    dst_shape[dst_split_axis] = dst_chunk
    src_strides = row_major_strides(shape)
    dst_strides = row_major_strides(dst_shape)

    def src_region_for(dest_peer: int) -> BufferRegion:
        return BufferRegion.from_slices(
            elem_size=elem_size, strides=src_strides,
            slices=axis_box(shape, {src_split_axis: (0, src_chunk),
                                    dst_split_axis: (dest_peer * dst_chunk, (dest_peer + 1) * dst_chunk)}))

    def dst_region_for(source_rank: int) -> BufferRegion:
        return BufferRegion.from_slices(
            elem_size=elem_size, strides=dst_strides,
            slices=axis_box(dst_shape, {src_split_axis: (source_rank * src_chunk, (source_rank + 1) * src_chunk),
                                        dst_split_axis: (0, dst_chunk)}))

    plan = DevicePlan(dev=rank)
    plan.src_shape = shape
    plan.dst_shape = tuple(dst_shape)
    plan.tensors_involved[src_buffer] = (torch.Size(shape), dtype)
    plan.tensors_involved[dst_buffer] = (torch.Size(dst_shape), dtype)
    plan.local_regions.setdefault(src_buffer, []).append(src_region_for(rank))

    if transfer_kind not in {"push", "pull"}:
        raise ValueError("transfer_kind must be 'push' or 'pull'")
    if peer_order not in {"clockwise", "counter-clockwise"}:
        raise ValueError("peer_order must be 'clockwise' or 'counter-clockwise'")
    direction = 1 if peer_order == "clockwise" else -1
    peers = [(rank + direction * step) % mesh_size for step in range(1, mesh_size)]
    return _emit_exchange(plan, rank=rank, mesh_size=mesh_size, peers=peers, src_buffer=src_buffer,
                          dst_buffer=dst_buffer, src_region_for=src_region_for,
                          dst_region_for=dst_region_for, transfer_kind=transfer_kind,
                          compute_producer=compute_producer)


__all__ = ["build_all_to_all_plan", "build_all_to_all_plan_dim"]


def build_all_to_all_plan_axis(
    shape: Sequence[int],
    *,
    dtype: torch.dtype,
    mesh_size: int,
    rank: int,
    src_buffer: str,
    dst_buffer: str,
    split_axis: int,
    transfer_kind: Literal["push", "pull"] = "push",
    compute_producer: bool = False,
) -> DevicePlan:
    """All-to-all along `split_axis`, the same axis before and after: `shape` is the local source
    tensor, slice p of the axis goes to rank p and lands there in slice `rank` of a destination
    of the same shape, e.g. attention output [B, S, H/w, D] -> [B, w * S/w, H/w, D] with the
    sequence blocks regrouped by sender."""
    elem_size = dtype.itemsize
    if mesh_size <= 0:
        raise ValueError("mesh_size must be positive")
    if elem_size <= 0:
        raise ValueError("elem_size must be positive")
    shape = tuple(shape)
    if not shape:
        raise ValueError("all_to_all expects at least one dimension in the source shape")
    split_axis = normalize_axis(split_axis, len(shape))
    ensure_divisible(shape[split_axis], mesh_size, axis=split_axis)
    chunk = shape[split_axis] // mesh_size
    if chunk == 0:
        raise ValueError("all-to-all requires non-empty slices along the split axis")
    if block_nbytes(shape, elem_size, {split_axis: chunk}) == 0:
        raise ValueError("all-to-all transfer would be empty")
    strides = row_major_strides(shape)

    def slice_of(index: int) -> BufferRegion:
        return BufferRegion.from_slices(
            elem_size=elem_size, strides=strides,
            slices=axis_box(shape, {split_axis: (index * chunk, (index + 1) * chunk)}))

    plan = DevicePlan(dev=rank)
    plan.src_shape = shape
    plan.dst_shape = shape
    plan.tensors_involved[src_buffer] = (torch.Size(shape), dtype)
    plan.tensors_involved[dst_buffer] = (torch.Size(shape), dtype)
    plan.local_regions.setdefault(src_buffer, []).append(slice_of(rank))

    if transfer_kind not in {"push", "pull"}:
        raise ValueError("transfer_kind must be 'push' or 'pull'")
    peers = [(rank + step) % mesh_size for step in range(1, mesh_size)]
    return _emit_exchange(plan, rank=rank, mesh_size=mesh_size, peers=peers, src_buffer=src_buffer,
                          dst_buffer=dst_buffer, src_region_for=slice_of, dst_region_for=slice_of,
                          transfer_kind=transfer_kind, compute_producer=compute_producer)


def build_all_to_all_plan_dim_waves(
    shape: Sequence[int],
    *,
    dtype: torch.dtype,
    mesh_size: int,
    rank: int,
    src_buffer: str,
    dst_buffer: str,
    src_split_axis: int,
    dst_split_axis: int,
    num_waves: int,
    transfer_kind: Literal["push", "pull"] = "push",
    compute_producer: bool = False,
    peer_order: Literal["clockwise", "counter-clockwise"] = "clockwise",
) -> DevicePlan:
    """`build_all_to_all_plan_dim` with every destination shard cut into `num_waves` slices along
    `dst_split_axis`, so that a receiver can start on the first slices while the rest is on its
    way.  Wave-major op order: for each wave, one op per peer starting with the rank itself (a
    local copy, treated like any other peer: first in the round, with its own compute dependency
    when a kernel produces the source)."""
    elem_size = dtype.itemsize
    if mesh_size <= 0:
        raise ValueError("mesh_size must be positive")
    if elem_size <= 0:
        raise ValueError("elem_size must be positive")
    if num_waves <= 0:
        raise ValueError("num_waves must be positive")
    shape = tuple(shape)
    if not shape:
        raise ValueError("all_to_all expects at least one dimension in the source shape")
    ndim = len(shape)
    src_split_axis = normalize_axis(src_split_axis, ndim)
    dst_split_axis = normalize_axis(dst_split_axis, ndim)
    if src_split_axis == dst_split_axis:
        raise ValueError("src_split_axis and dst_split_axis must differ")
    src_chunk = shape[src_split_axis]
    if src_chunk <= 0:
        raise ValueError("all-to-all requires non-empty slices along the split axis")
    ensure_divisible(shape[dst_split_axis], mesh_size, axis=dst_split_axis)
    dst_chunk = shape[dst_split_axis] // mesh_size
    if dst_chunk == 0:
        raise ValueError("all-to-all requires non-empty slices along the destination axis")
    ensure_divisible(dst_chunk, num_waves, "num_waves")
    wave_chunk = dst_chunk // num_waves
    if wave_chunk == 0:
        raise ValueError("wave splitting produced an empty chunk along dst_split_axis")
    if block_nbytes(shape, elem_size, {src_split_axis: src_chunk, dst_split_axis: wave_chunk}) == 0:
        raise ValueError("all-to-all transfer would be empty")

    dst_shape = list(shape)
    dst_shape[src_split_axis] = src_chunk * mesh_size
    dst_shape[dst_split_axis] = dst_chunk
    src_strides = row_major_strides(shape)
    dst_strides = row_major_strides(dst_shape)

    def outgoing(dest_peer: int, wave: int) -> BufferRegion:
        """Wave `wave` of what this rank holds for `dest_peer` (wave None: all of it)."""
        lo = dest_peer * dst_chunk + (0 if wave is None else wave * wave_chunk)
        hi = lo + (dst_chunk if wave is None else wave_chunk)
        return BufferRegion.from_slices(
            elem_size=elem_size, strides=src_strides,
            slices=axis_box(shape, {src_split_axis: (0, src_chunk), dst_split_axis: (lo, hi)}))

    def landing(source_rank: int, wave: int) -> BufferRegion:
        """Where wave `wave` of `source_rank`'s contribution lands in a destination buffer."""
        return BufferRegion.from_slices(
            elem_size=elem_size, strides=dst_strides,
            slices=axis_box(dst_shape, {src_split_axis: (source_rank * src_chunk, (source_rank + 1) * src_chunk),
                                        dst_split_axis: (wave * wave_chunk, (wave + 1) * wave_chunk)}))

    plan = DevicePlan(dev=rank)
    plan.src_shape = shape
    plan.dst_shape = tuple(dst_shape)
    plan.tensors_involved[src_buffer] = (torch.Size(shape), dtype)
    plan.tensors_involved[dst_buffer] = (torch.Size(dst_shape), dtype)
    plan.local_regions.setdefault(src_buffer, []).append(outgoing(rank, None))

    if transfer_kind not in {"push", "pull"}:
        raise ValueError("transfer_kind must be 'push' or 'pull'")
    if peer_order not in {"clockwise", "counter-clockwise"}:
        raise ValueError("peer_order must be 'clockwise' or 'counter-clockwise'")
    direction = 1 if peer_order == "clockwise" else -1
    peers = [(rank + direction * step) % mesh_size for step in range(mesh_size)]     # the rank itself first

    def produced_by(compute_rank: int, region: BufferRegion) -> List:
        if not compute_producer:
            return []
        return [ComputeDependency(compute_rank=compute_rank, src_region=region, signal=None)]

    for wave in range(num_waves):
        for peer in peers:
            if peer == rank:
                piece = outgoing(rank, wave)
                op = Transfer(op=TransferOp.LOCAL_COPY, src_buf=src_buffer, dst_buf=dst_buffer, src_region=piece,
                              dst_region=landing(rank, wave),
                              chunk_idx=(rank * mesh_size + rank) * num_waves + wave,
                              dependency=produced_by(rank, piece))
            elif transfer_kind == "push":
                piece = outgoing(peer, wave)
                op = Transfer(op=TransferOp.PUSH, src_buf=src_buffer, src_region=piece, peer=peer,
                              chunk_idx=(rank * mesh_size + peer) * num_waves + wave, dst_buf=dst_buffer,
                              dst_region=landing(rank, wave), dependency=produced_by(rank, piece))
            else:
                piece = outgoing(rank, wave)       # the same box of the peer's source
                op = Transfer(op=TransferOp.PULL, dst_buf=dst_buffer, dst_region=landing(peer, wave), peer=peer,
                              chunk_idx=(peer * mesh_size + rank) * num_waves + wave, src_buf=src_buffer,
                              src_region=piece, dependency=produced_by(peer, piece))
            plan.add_op(op)
    return plan
