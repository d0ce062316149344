"""Small shape helpers shared by the plan builders
(reference: syncopate/communication/common_descriptors/utils.py)."""

from __future__ import annotations

from typing import Dict, List, Mapping, Sequence, Union


def ensure_divisible(length: int, mesh_size: int, axis: Union[str, int]) -> None:
    if length % mesh_size:
        raise ValueError(f"axis '{axis}' length {length} must be divisible by mesh size {mesh_size}")


def lookup_mesh_size(mesh: Dict[str, int], mesh_axis: str) -> int:
    if mesh_axis not in mesh:
        raise ValueError(f"mesh axis '{mesh_axis}' not found in mesh")
    size = mesh[mesh_axis]
    if size <= 0:
        raise ValueError(f"mesh axis '{mesh_axis}' must be positive")
    return size


def row_major_strides(shape: Sequence[int]) -> List[int]:
    """Element strides of a C-contiguous tensor of `shape`."""
    strides = [1] * len(shape)
    for axis in range(len(shape) - 2, -1, -1):
        strides[axis] = strides[axis + 1] * shape[axis + 1]
    return strides


def compute_offset(strides: Sequence[int], starts: Mapping[int, int]) -> int:
    return sum(starts.get(axis, 0) * stride for axis, stride in enumerate(strides))


def block_nbytes(shape: Sequence[int], elem_size: int, lengths: Mapping[int, int]) -> int:
    """Bytes of a box that spans `lengths[axis]` on the listed axes and the full extent elsewhere."""
    count = 1
    for axis, extent in enumerate(shape):
        count *= lengths.get(axis, extent)
    return count * elem_size


def normalize_axis(axis: int, ndim: int, what: str = "tensor") -> int:
    if axis < 0:
        axis += ndim
    if not 0 <= axis < ndim:
        raise IndexError(f"axis {axis} out of range for {what} with {ndim} dims")
    return axis


def axis_box(shape: Sequence[int], cuts: Mapping[int, tuple]):
    """(start, end) per axis: `cuts[axis]` where given, the whole axis elsewhere."""
    return [cuts.get(axis, (0, extent)) for axis, extent in enumerate(shape)]


__all__ = [
    "block_nbytes",
    "compute_offset",
    "ensure_divisible",
    "lookup_mesh_size",
    "row_major_strides",
]
