"""Lower a planned CommPlan to per-rank, per-buffer wave schedules.

Behavioural restatement of syncopate/interface/lowering.py
(`lower_comm_plan_to_raw_schedules` :91-331 and its helpers :334-451).  The
result — which blocks form which wave, in which order, with which signal,
peer, role, reduce op and peer-side offsets — is what the compute kernels are
driven by, so the ordering rules below are kept exactly:

* ops are visited by (period start, device, stream, index);
* every op touches a buffer on its own device and (push/pull) one on the peer;
  a touch where communication WRITES the buffer becomes an event at the op's
  start time, a touch where communication READS it is kept only at its
  earliest (time, order key) per identical tile, and dropped altogether if the
  same buffer is also written by communication;
* resident regions form a leading wave unless communication only reads the buffer;
* events of one device are sorted by (time, buffer, order key, offsets, shape)
  and cut into waves wherever the time changes (tolerance 1e-9).
"""

from __future__ import annotations

import math
from collections import defaultdict
from dataclasses import dataclass
from typing import Dict, Iterable, Iterator, List, NamedTuple, Optional, Tuple

from ..communication.descriptor import (
    BufferRegion,
    Collective,
    CommOp,
    CommPlan,
    ReduceOp,
    Signal,
    Transfer,
    TransferOp,
)
from .tile_schedule import RawSchedule, TileBlock, TileCoord

_TIME_TOL = 1e-9


class _ScheduleError(ValueError):
    """A plan that cannot be lowered (missing regions, inconsistent shapes, ...)."""


def _same_time(a: float, b: float) -> bool:
    return math.isclose(a, b, rel_tol=_TIME_TOL, abs_tol=_TIME_TOL)


def _region_to_tiles(region: Optional[BufferRegion]) -> List[TileCoord]:
    """One tile per non-empty box of the region (lowering.py:443-451)."""
    if region is None:
        return []
    tiles = []
    for box in region.regions:
        extent = tuple(ax.length() for ax in box)
        if extent and all(n > 0 for n in extent):
            tiles.append(TileCoord(offsets=tuple(ax.start for ax in box), shape=extent))
    return tiles


class _Touch(NamedTuple):
    """One side of an op as seen from the device that holds `buffer`."""

    device: int
    side: int                      # 0: the op's own device, 1: its peer
    buffer: str
    region: BufferRegion
    comm_reads: bool               # True: communication reads the buffer (compute produced it)
    peer: Optional[int]
    peer_region: Optional[BufferRegion]


def _need(name: str, region: Optional[BufferRegion]) -> BufferRegion:
    if region is None:
        raise _ScheduleError(f"transfer for buffer '{name}' lacks a concrete region")
    return region


def _touches(origin: int, op: CommOp) -> Iterator[_Touch]:
    """Local touches first, then remote ones (lowering.py:334-419)."""
    if isinstance(op, Collective):
        yield _Touch(origin, 0, op.src_buf, _need(op.src_buf, op.src_region), True, None, None)
        yield _Touch(origin, 0, op.dst_buf, _need(op.dst_buf, op.dst_region), False, None, None)
        return
    if not isinstance(op, Transfer):
        raise _ScheduleError(f"unsupported op type: {type(op)}")
    src = _need(op.src_buf, op.src_region)
    dst = _need(op.dst_buf, op.dst_region)
    if op.op == TransferOp.LOCAL_COPY:
        # no cross-device peer, but the destination side is still recorded so that a fused
        # producer sees where its local wave lands
        yield _Touch(origin, 0, op.src_buf, src, True, None, dst)
        if op.dst_buf != op.src_buf or op.dst_region != op.src_region:
            yield _Touch(origin, 0, op.dst_buf, dst, False, None, src)
        return
    if op.peer is None:
        raise _ScheduleError(f"{op.op.value} transfer lacks peer device")
    if op.op == TransferOp.PUSH:
        yield _Touch(origin, 0, op.src_buf, src, True, op.peer, dst)
        yield _Touch(op.peer, 1, op.dst_buf, dst, False, origin, src)
    elif op.op == TransferOp.PULL:
        yield _Touch(origin, 0, op.dst_buf, dst, False, op.peer, src)
        yield _Touch(op.peer, 1, op.src_buf, src, True, origin, dst)
    else:
        raise _ScheduleError(f"unsupported transfer operation: {op.op}")


def _signal_for(op: CommOp, device: int, comm_reads: bool) -> Optional[Signal]:
    """The flag `device` can watch for this touch: for data read by communication the
    first dependency signal addressed to it, for data written the first completion
    signal addressed to it (lowering.py:428-440)."""
    if comm_reads:
        candidates = (getattr(dep, "signal", None) for dep in op.dependency)
    else:
        candidates = iter(op.set_signals)
    for sig in candidates:
        if sig is not None and sig.dst_rank == device:
            return sig
    return None


@dataclass
class _Event:
    time: float
    buffer: str
    order: Tuple[int, ...]
    block: TileBlock

    def sort_key(self):
        return (self.time, self.buffer, self.order, self.block.tile.offsets, self.block.tile.shape)


class _BufferWaves:
    """Waves collected for one buffer of one device."""

    def __init__(self, expected_shape: Optional[Tuple[int, ...]]) -> None:
        if expected_shape is not None and any(d <= 0 for d in expected_shape):
            raise _ScheduleError("expected_shape must contain positive dimensions")
        self.expected_shape = expected_shape
        self.waves: List[List[TileBlock]] = []

    def append_wave(self, blocks: Iterable[TileBlock]) -> None:
        blocks = list(blocks)
        if blocks:
            self.waves.append(blocks)

    def build(self) -> RawSchedule:
        if not self.waves:
            raise _ScheduleError("cannot build schedule with no waves")
        extent: Optional[List[int]] = None
        for wave in self.waves:
            for block in wave:
                tile = block.tile
                if extent is None:
                    extent = [0] * tile.ndim
                elif len(extent) != tile.ndim:
                    raise _ScheduleError("inconsistent dimensionality encountered while lowering")
                for axis, (lo, n) in enumerate(zip(tile.offsets, tile.shape)):
                    extent[axis] = max(extent[axis], lo + n)
        if extent is None:
            raise _ScheduleError("buffer extent is unknown after lowering")
        if self.expected_shape is None:
            shape = tuple(extent)
        else:
            if len(self.expected_shape) != len(extent):
                raise _ScheduleError("mismatched dimensionality between tiles and expected shape")
            for axis, (seen, allowed) in enumerate(zip(extent, self.expected_shape)):
                if seen > allowed:
                    raise _ScheduleError(
                        f"observed extent {seen} exceeds expected shape {allowed} on axis {axis}")
            shape = tuple(self.expected_shape)
        return RawSchedule(num_waves=len(self.waves), block_infos=[list(w) for w in self.waves],
                           global_shape=shape)


def lower_comm_plan_to_raw_schedules(comm_plan: CommPlan) -> Dict[int, Dict[str, RawSchedule]]:
    """{rank: {buffer name: RawSchedule}} for every rank and buffer that has waves."""
    comm_plan.estimate_period()
    plans = comm_plan.device_plans

    collected: Dict[int, Dict[str, _BufferWaves]] = {}

    def waves_of(device: int, buffer: str) -> _BufferWaves:
        per_device = collected.setdefault(device, {})
        if buffer not in per_device:
            hint = plans[device].tensors_involved.get(buffer) if device in plans else None
            per_device[buffer] = _BufferWaves(tuple(hint[0]) if hint is not None else None)
        return per_device[buffer]

    # data resident before any transfer runs
    resident: Dict[Tuple[int, str], List[TileBlock]] = {}
    for dev, plan in plans.items():
        for buffer, regions in plan.local_regions.items():
            blocks = [TileBlock(tile=t) for region in regions for t in _region_to_tiles(region)]
            if blocks:
                resident.setdefault((dev, buffer), []).extend(blocks)

    timeline = []
    for dev, plan in plans.items():
        for s, stream in enumerate(plan.xfer):
            for i, op in enumerate(stream):
                if op.period.start is None:
                    raise _ScheduleError("transfer period start is unknown; run period estimation first")
                timeline.append((op.period.start, dev, s, i, op))
    timeline.sort(key=lambda item: item[:4])

    events: Dict[int, List[_Event]] = defaultdict(list)
    # (device, buffer) -> {(offsets, shape): earliest read event of that tile}
    first_reads: Dict[Tuple[int, str], Dict[Tuple, _Event]] = defaultdict(dict)
    written = defaultdict(bool)     # (device, buffer) written by communication
    read = defaultdict(bool)        # (device, buffer) read by communication

    for start, origin, s, i, op in timeline:
        reduce_op: Optional[ReduceOp] = op.reduce_op if isinstance(op, Transfer) else None
        for touch in _touches(origin, op):
            if touch.side == 1 and touch.device not in plans:
                continue
            tiles = _region_to_tiles(touch.region)
            if not tiles:
                continue
            peer_tiles = _region_to_tiles(touch.peer_region)
            signal = _signal_for(op, touch.device, touch.comm_reads)
            key = (touch.device, touch.buffer)
            if touch.comm_reads:
                read[key] = True
            else:
                written[key] = True
            for t, tile in enumerate(tiles):
                block = TileBlock(
                    tile=tile,
                    signal=signal,
                    peer_rank=touch.peer,
                    reduce_op=reduce_op,
                    # the holder's compute role is the inverse of communication's
                    role="producer" if touch.comm_reads else "consumer",
                    # i-th local tile pairs with the i-th peer-side tile, if there is one
                    dst_offsets=peer_tiles[t].offsets if t < len(peer_tiles) else None,
                )
                event = _Event(start, touch.buffer, (origin, touch.side, s, i, t), block)
                if not touch.comm_reads:
                    events[touch.device].append(event)
                    continue
                slot = first_reads[key]
                tile_key = (tile.offsets, tile.shape)
                seen = slot.get(tile_key)
                if (seen is None or start < seen.time - _TIME_TOL
                        or (_same_time(start, seen.time) and event.order < seen.order)):
                    slot[tile_key] = event

    for key, slot in first_reads.items():
        if not written[key]:
            events[key[0]].extend(slot.values())

    # resident data leads, unless communication only ever reads the buffer
    for (dev, buffer), blocks in resident.items():
        touched = (dev, buffer) in read or (dev, buffer) in written
        reads, writes = read.get((dev, buffer), False), written.get((dev, buffer), False)
        if touched and reads and not writes:
            continue
        if touched and writes and not reads:
            role: Optional[str] = "consumer"
        else:
            role = None
        waves_of(dev, buffer).append_wave(
            TileBlock(tile=b.tile, signal=b.signal, peer_rank=dev, reduce_op=b.reduce_op, role=role)
            for b in blocks)

    for dev, dev_events in events.items():
        dev_events.sort(key=_Event.sort_key)
        wave_time: Optional[float] = None
        wave: Dict[str, List[TileBlock]] = {}

        def flush() -> None:
            for buffer, blocks in wave.items():
                waves_of(dev, buffer).append_wave(blocks)
            wave.clear()

        for ev in dev_events:
            if wave_time is None or not _same_time(ev.time, wave_time):
                flush()
                wave_time = ev.time
            wave.setdefault(ev.buffer, []).append(ev.block)
        flush()

    lowered: Dict[int, Dict[str, RawSchedule]] = {}
    for dev, per_device in collected.items():
        built = {buffer: bw.build() for buffer, bw in per_device.items() if bw.waves}
        if built:
            lowered[dev] = built
    return lowered


__all__ = ["lower_comm_plan_to_raw_schedules"]
