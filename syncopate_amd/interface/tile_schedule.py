"""Schedule data model: tiles, blocks, waves, and the flat lists kernels take.

Same classes, fields and results as the reference
(syncopate/interface/tile_schedule.py: TileCoord :14, TileBlock :40-61,
RawSchedule :65-171, SimplifiedSchedule :177, Mod1DSchedule :214-273).
"""

from __future__ import annotations

import abc
from dataclasses import dataclass
from typing import Iterator, List, Literal, Optional, Tuple

from ..communication.descriptor import ReduceOp, Signal

TileRole = Literal["producer", "consumer"]


@dataclass
class TileCoord:
    """Origin and extent of a box of an N-D tensor, in elements."""

    offsets: Tuple[int, ...]
    shape: Tuple[int, ...]

    def __post_init__(self) -> None:
        if len(self.offsets) != len(self.shape):
            raise ValueError("offsets and shape must have identical length")
        if any(o < 0 for o in self.offsets):
            raise ValueError("offsets must be non-negative")
        if any(s <= 0 for s in self.shape):
            raise ValueError("shape must contain strictly positive sizes")

    @property
    def ndim(self) -> int:
        return len(self.offsets)

    def as_ranges(self) -> Tuple[Tuple[int, int], ...]:
        return tuple((o, o + s) for o, s in zip(self.offsets, self.shape))

    def __repr__(self) -> str:
        return f"TileCoord(offsets={self.offsets}, shape={self.shape})"


@dataclass
class TileBlock:
    """A tile plus how it becomes ready and whom it is exchanged with."""

    tile: TileCoord
    signal: Optional[Signal] = None           # flag that publishes the tile (None: resident)
    peer_rank: Optional[int] = None           # rank on the other end (None: purely local)
    reduce_op: Optional[ReduceOp] = None      # set when the transfer accumulates
    role: Optional[TileRole] = None           # what the fused compute kernel does with the tile
    dst_offsets: Optional[Tuple[int, ...]] = None   # where the tile sits in the peer's allocation


@dataclass
class RawSchedule:
    """Time-ordered waves of blocks for one buffer on one rank."""

    num_waves: int
    block_infos: List[List[TileBlock]]
    global_shape: Tuple[int, ...]

    def __post_init__(self) -> None:
        if self.num_waves <= 0:
            raise ValueError("num_waves must be positive")
        if len(self.block_infos) != self.num_waves:
            raise ValueError("block_infos length must match num_waves")
        if any(len(wave) == 0 for wave in self.block_infos):
            raise ValueError("each wave must contain at least one block")
        if any(b.tile.ndim != len(self.global_shape) for b in self._blocks()):
            raise ValueError("all blocks must have the same number of dimensions as global_shape")

    def _blocks(self) -> Iterator[TileBlock]:
        for wave in self.block_infos:
            yield from wave

    def __repr__(self) -> str:
        return (f"RawSchedule(num_waves={self.num_waves}, global_shape={self.global_shape}, "
                f"block_infos=[{self.block_infos}])")

    # ---- one row per block, waves in order: the kernel-argument tables ----

    def gen_block_offset_lists(self) -> List[List[int]]:
        return [list(b.tile.offsets) for b in self._blocks()]

    def gen_block_shape_lists(self) -> List[List[int]]:
        return [list(b.tile.shape) for b in self._blocks()]

    def gen_signal_lists(self) -> List[int]:
        """Flag index per block, -1 where the block needs no flag."""
        return [-1 if b.signal is None else b.signal.dst_offset for b in self._blocks()]

    def gen_target_rank_list(self) -> List[int]:
        """Peer rank per block, -1 for purely local blocks."""
        return [-1 if b.peer_rank is None else b.peer_rank for b in self._blocks()]

    def gen_dst_offset_lists(self) -> List[List[int]]:
        """Peer-side offsets per block; a block without a remote counterpart reports its
        own offsets, which leaves a rewritten access where it was."""
        return [list(b.tile.offsets if b.dst_offsets is None else b.dst_offsets) for b in self._blocks()]

    def is_reduce(self) -> bool:
        return any(b.reduce_op is not None for b in self._blocks())

    def role(self) -> Optional[TileRole]:
        """The one role all role-carrying blocks share (None if none carries one)."""
        seen: Optional[TileRole] = None
        for b in self._blocks():
            if b.role is None:
                continue
            if seen is not None and seen != b.role:
                raise ValueError(f"schedule blocks disagree on role: {seen!r} vs {b.role!r}")
            seen = b.role
        return seen


@dataclass
class SimplifiedSchedule:
    """Try to express a RawSchedule by a closed form (so a kernel need not read tables)."""

    origin_schedule: RawSchedule
    simplified_schedule: "None | SimpleSchedule" = None

    def simplify(self) -> bool:
        for candidate in sorted(SimpleSchedule.__subclasses__(), key=lambda c: c.priority):
            try:
                self.simplified_schedule = candidate(self.origin_schedule)
            except Exception as exc:
                print(f"Failed to simplify schedule to {candidate.__name__}: {exc}")
                continue
            print(f"Simplified schedule to {candidate.__name__}")
            return True
        return False


class SimpleSchedule(abc.ABC):
    priority = 99

    @abc.abstractmethod
    def __init__(self, raw_schedule: RawSchedule):
        pass

    @abc.abstractmethod
    def __repr__(self) -> str:
        pass


class Mod1DSchedule(SimpleSchedule):
    """One equal-shaped block per wave, stepping along a single axis, flags 0, 1, 2, ...
    after an unflagged first (local) wave: what ring and swizzled all-gathers lower to."""

    priority = 1

    num_waves: int
    global_shape: Tuple[int, ...]
    stride: int
    starting_offset: int
    schedule_axis: int

    def __init__(self, raw_schedule: RawSchedule):
        self.num_waves = raw_schedule.num_waves
        self.global_shape = raw_schedule.global_shape
        waves = raw_schedule.block_infos
        if any(len(wave) != 1 for wave in waves):
            raise ValueError("all waves must contain exactly one block")
        blocks = [wave[0] for wave in waves]
        shape = blocks[0].tile.shape
        if any(b.tile.shape != shape for b in blocks):
            raise ValueError("all blocks must have the same shape")
        partial = [a for a in range(len(self.global_shape)) if shape[a] < self.global_shape[a]]
        if len(partial) != 1:
            raise ValueError("schedule must be defined along exactly one axis")
        self.schedule_axis = partial[0]
        self.stride = shape[self.schedule_axis]
        self.starting_offset = blocks[0].tile.offsets[self.schedule_axis]
        if blocks[0].signal is not None:
            raise ValueError("first block (local) must not have any signals")
        for w, b in enumerate(blocks[1:], start=1):
            if b.signal is None or b.signal.dst_offset != w - 1:
                raise ValueError("signal offsets do not match expected pattern")

    def __post_init__(self) -> None:
        if self.schedule_axis < 0 or self.schedule_axis >= len(self.global_shape):
            raise ValueError("schedule_axis must be a valid axis index")
        if self.stride * self.num_waves != self.global_shape[self.schedule_axis]:
            raise ValueError("stride * num_waves must equal the size of the schedule_axis in global_shape")

    def __repr__(self) -> str:
        return (f"Mod1DSchedule(num_waves={self.num_waves}, global_shape={self.global_shape}, "
                f"stride={self.stride}, starting_offset={self.starting_offset}, "
                f"schedule_axis={self.schedule_axis})")
