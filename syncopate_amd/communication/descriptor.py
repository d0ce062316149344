"""Communication IR: byte regions, transfers, per-device plans, signal planning, timing.

Host-side (pure Python) restatement of the reference's IR module
(syncopate/communication/descriptor.py).  Class names, fields, method names and
every observable result (segment lists, region text, signal offsets, period
starts, error types) follow the reference so that plans built against it build
unchanged here; the implementation is this project's own.

Reference map:
    MemorySegment, AxisSlice, BufferRegion      descriptor.py:26-373
    XferDependency .. Signal, ReduceOp          descriptor.py:393-433
    Transfer (+ to_memcpys), Collective         descriptor.py:435-639
    DevicePlan                                  descriptor.py:643-745
    CommPlan (plan_signals, estimate_period)    descriptor.py:747-1061
"""

from __future__ import annotations

import copy
from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from itertools import product
from typing import Dict, Iterable, List, Optional, Sequence, Tuple, Union

import torch


def cdiv(a: int, b: int) -> int:
    """Ceiling division of non-negative integers (the reference borrows triton.cdiv)."""
    return -(-a // b)


# --------------------------------------------------------------------------- time


@dataclass
class Period:
    """Scheduling interval of an op or signal; `start` is filled by estimate_period."""

    start: Optional[float] = None
    duration: float = 1.0

    def split(self, num_splits: int) -> "Period":
        assert self.start is None, "Cannot split a Period with known start time."
        if num_splits <= 1:
            return self
        return Period(start=None, duration=self.duration / num_splits)


# --------------------------------------------------------------------------- regions


@dataclass(frozen=True)
class MemorySegment:
    """Contiguous byte span [offset, offset + nbytes) of a logical buffer."""

    offset: int
    nbytes: int

    def __post_init__(self) -> None:
        if self.offset < 0:
            raise ValueError("segment offset must be non-negative")
        if self.nbytes < 0:
            raise ValueError("segment nbytes must be non-negative")

    @property
    def end(self) -> int:
        return self.offset + self.nbytes


@dataclass(frozen=True)
class AxisSlice:
    """Half-open index range [start, end) along one logical axis."""

    start: int
    end: int

    def __post_init__(self) -> None:
        if self.start < 0:
            raise ValueError("axis slice start must be non-negative")
        if self.end < self.start:
            raise ValueError("axis slice end must be >= start")

    def length(self) -> int:
        return self.end - self.start


SliceSpec = Union[AxisSlice, slice, Tuple[int, int]]


def _as_axis_slice(spec: SliceSpec) -> AxisSlice:
    if isinstance(spec, AxisSlice):
        return spec
    if isinstance(spec, slice):
        if spec.step not in (None, 1):
            raise ValueError("slice step other than 1 is not supported")
        if spec.stop is None:
            raise ValueError("slice stop must be provided")
        return AxisSlice(spec.start or 0, spec.stop)
    lo, hi = spec
    return AxisSlice(lo, hi)


def _merge_adjacent_segments(segments: Sequence[MemorySegment]) -> Tuple[MemorySegment, ...]:
    """Fuse neighbours of an offset-sorted list that touch end-to-start."""
    fused: List[MemorySegment] = []
    for seg in segments:
        if fused and fused[-1].end == seg.offset:
            fused[-1] = MemorySegment(fused[-1].offset, fused[-1].nbytes + seg.nbytes)
        else:
            fused.append(seg)
    return tuple(fused)


@dataclass
class BufferRegion:
    """Union of axis-aligned boxes of a strided buffer, with its byte-segment view.

    `regions` is a tuple of boxes, each a tuple of AxisSlice (one per axis);
    `strides` are in elements.  `_segments` is the offset-sorted, merged list of
    contiguous byte spans the boxes cover (descriptor.py:87-92,192-234).
    """

    regions: Tuple[Tuple[AxisSlice, ...], ...]
    elem_size: int
    strides: Tuple[int, ...]
    base_offset: int = 0
    _segments: Tuple[MemorySegment, ...] = field(init=False, repr=False)

    def __post_init__(self) -> None:
        if not self.regions:
            raise ValueError("BufferRegion requires at least one region")
        if self.elem_size <= 0:
            raise ValueError("elem_size must be positive")
        if self.base_offset < 0:
            raise ValueError("base_offset must be non-negative")
        rank = len(self.regions[0])
        if len(self.strides) != rank:
            raise ValueError("strides length must match number of axes")
        if any(len(box) != rank for box in self.regions):
            raise ValueError("all regions must have the same number of axes")
        spans: List[MemorySegment] = []
        for box in self.regions:
            spans.extend(self._box_segments(box))
        spans.sort(key=lambda s: s.offset)
        self._segments = _merge_adjacent_segments(spans)

    # ---- constructors ------------------------------------------------------

    @classmethod
    def contiguous(cls, offset: int, nbytes: int) -> "BufferRegion":
        return cls.from_segments([(offset, nbytes)])

    @classmethod
    def from_segments(cls, segments: Iterable[Union[MemorySegment, Tuple[int, int]]]) -> "BufferRegion":
        spans = [s if isinstance(s, MemorySegment) else MemorySegment(*s) for s in segments]
        if not spans:
            raise ValueError("from_segments expects at least one segment")
        boxes = tuple((AxisSlice(s.offset, s.end),) for s in spans)
        return cls(regions=boxes, elem_size=1, strides=(1,), base_offset=0)

    @classmethod
    def from_slices(cls, *, elem_size: int, strides: Sequence[int], slices: Sequence[SliceSpec],
                    base_offset: int = 0) -> "BufferRegion":
        box = tuple(_as_axis_slice(s) for s in slices)
        return cls(regions=(box,), elem_size=elem_size, strides=tuple(strides), base_offset=base_offset)

    @classmethod
    def from_multi_slices(cls, *, elem_size: int, strides: Sequence[int],
                          regions: Sequence[Sequence[SliceSpec]], base_offset: int = 0) -> "BufferRegion":
        boxes = tuple(tuple(_as_axis_slice(s) for s in box) for box in regions)
        if not boxes:
            raise ValueError("from_multi_slices expects at least one region")
        return cls(regions=boxes, elem_size=elem_size, strides=tuple(strides), base_offset=base_offset)

    @classmethod
    def strided(cls, base_offset: int, segment_bytes: int, stride: int, count: int) -> "BufferRegion":
        if count <= 0:
            raise ValueError("count must be positive for strided region")
        if segment_bytes <= 0:
            raise ValueError("segment_bytes must be positive")
        if stride < 0:
            raise ValueError("stride must be non-negative")
        return cls.from_segments(MemorySegment(base_offset + i * stride, segment_bytes) for i in range(count))

    @staticmethod
    def _normalize_region(slices: Sequence[SliceSpec]) -> Tuple[AxisSlice, ...]:
        return tuple(_as_axis_slice(s) for s in slices)

    # ---- byte view ---------------------------------------------------------

    def _box_segments(self, box: Tuple[AxisSlice, ...]) -> List[MemorySegment]:
        """Contiguous spans of one box (descriptor.py:192-234): trailing axes whose
        byte stride equals the run length so far extend the run; the first axis
        that does not is the split axis, and every index combination of axes
        0..split yields one run."""
        if any(ax.length() == 0 for ax in box):
            return []
        run = self.elem_size
        split = -1
        for axis in reversed(range(len(box))):
            if self.strides[axis] * self.elem_size != run:
                split = axis
                break
            run *= box[axis].length()
        if split < 0:
            first = sum(ax.start * st for ax, st in zip(box, self.strides))
            return [MemorySegment(self.base_offset + first * self.elem_size, run)]
        tail = sum(box[a].start * self.strides[a] * self.elem_size for a in range(split + 1, len(box)))
        byte_strides = [self.strides[a] * self.elem_size for a in range(split + 1)]
        spans = []
        for index in product(*(range(box[a].start, box[a].end) for a in range(split + 1))):
            head = sum(i * s for i, s in zip(index, byte_strides))
            spans.append(MemorySegment(self.base_offset + head + tail, run))
        return spans

    def total_nbytes(self) -> int:
        return sum(s.nbytes for s in self._segments)

    def is_contiguous(self) -> bool:
        return len(self._segments) == 1

    def to_segments(self) -> Tuple[MemorySegment, ...]:
        return self._segments

    def as_slice(self) -> Optional[slice]:
        plain_bytes = (self.strides == (1,) and self.elem_size == 1 and self.base_offset == 0
                       and len(self.regions) == 1 and len(self.regions[0]) == 1)
        if not plain_bytes:
            return None
        only = self.regions[0][0]
        return slice(only.start, only.end)

    # ---- splitting ---------------------------------------------------------

    def split(self, num_splits: int, axis: Optional[int] = None) -> List["BufferRegion"]:
        if num_splits <= 1:
            return [self]
        if axis is None:
            return self._split_by_bytes(num_splits)
        return self._split_along_axis(num_splits, axis)

    def _split_by_bytes(self, num_splits: int) -> List["BufferRegion"]:
        """Cut the segment list into pieces of cdiv(total, n) bytes (descriptor.py:263-301)."""
        total = self.total_nbytes()
        if total == 0:
            return [self]
        quota = cdiv(total, num_splits)
        pending = deque(self._segments)
        pieces: List[BufferRegion] = []
        left = total
        for _ in range(num_splits):
            want = min(quota, left)
            if want <= 0:
                break
            taken: List[MemorySegment] = []
            while want > 0:
                if not pending:
                    raise RuntimeError("not enough data to satisfy split request")
                seg = pending.popleft()
                take = min(want, seg.nbytes)
                taken.append(MemorySegment(seg.offset, take))
                if take < seg.nbytes:
                    pending.appendleft(MemorySegment(seg.offset + take, seg.nbytes - take))
                want -= take
                left -= take
            pieces.append(BufferRegion.from_segments(taken))
        return pieces

    def _split_along_axis(self, num_splits: int, axis: int) -> List["BufferRegion"]:
        rank = len(self.strides)
        if axis < 0:
            axis += rank
        if not 0 <= axis < rank:
            raise IndexError(f"axis {axis} out of range for BufferRegion with {rank} dims")
        if len(self.regions) != 1:
            raise NotImplementedError(
                "Axis-aligned splitting currently supports regions with a single contiguous block")
        box = self.regions[0]
        span = box[axis]
        if span.length() == 0:
            return [self]
        step = cdiv(span.length(), num_splits)
        pieces = []
        for lo in range(span.start, span.end, step):
            if len(pieces) == num_splits:
                break
            cut = box[:axis] + (AxisSlice(lo, min(span.end, lo + step)),) + box[axis + 1:]
            pieces.append(BufferRegion(regions=(cut,), elem_size=self.elem_size, strides=self.strides,
                                       base_offset=self.base_offset))
        return pieces or [self]

    # ---- text --------------------------------------------------------------

    def describe(self) -> str:
        def one(box: Tuple[AxisSlice, ...]) -> str:
            return "[" + ", ".join(f"{ax.start}:{ax.end}" for ax in box) + "]"

        if len(self.regions) == 1:
            return one(self.regions[0])
        return "{" + ", ".join(one(box) for box in self.regions) + "}"


# --------------------------------------------------------------------------- high-level descriptor


@dataclass
class DataPlacement:
    rank: int
    region: Optional[BufferRegion] = None


@dataclass
class CommDescriptor:
    """Data-only description of a collective (no scheduling)."""

    data_info: Dict[int, Optional[int]]
    before_placement: Dict[int, DataPlacement]
    after_placement: Dict[int, DataPlacement]


# --------------------------------------------------------------------------- ops


class TransferOp(Enum):
    PUSH = "push"
    PULL = "pull"
    LOCAL_COPY = "local_copy"


class SignalType(Enum):
    RECEIVE_DATA = "receive_data"            # raised at the receiver when data has landed
    COMPUTE_DONE = "compute_done"            # raised by a compute kernel
    REMOTE_DATA_READY = "remote_data_ready"  # transfer finished, told to a non-receiver


class ReduceOp(Enum):
    SUM = 1
    MAX = 2


class CollectiveOp(Enum):
    REDUCE_SCATTER = "reduce_scatter"
    ALL_REDUCE = "all_reduce"
    ALL_GATHER = "all_gather"
    ALL_REDUCE_NVSHARP = "all_reduce_nvsharp"


@dataclass
class Signal:
    dst_rank: int     # rank whose flag array holds the word
    dst_offset: int   # index of the word in that array
    type: SignalType
    period: Period = field(default_factory=Period)


@dataclass
class XferDependency:
    """This op may start only after op (depend_rank, depend_xfer_stream, depend_xfer_idx)."""

    depend_rank: int
    depend_xfer_stream: int
    depend_xfer_idx: int
    signal: Optional[Signal] = None   # filled by plan_signals


@dataclass
class ComputeDependency:
    """This op may start only after compute on `compute_rank` has produced `src_region`."""

    compute_rank: int
    src_region: Optional[BufferRegion]
    signal: Optional[Signal] = None   # filled by plan_signals (or by the caller)

    def __post_init__(self) -> None:
        if self.signal is not None:
            assert self.signal.type == SignalType.COMPUTE_DONE


Dependency = Union[XferDependency, ComputeDependency]


@dataclass
class Transfer:
    """A push, pull or local copy of one region into another."""

    op: TransferOp
    src_buf: str
    src_region: Optional[BufferRegion]
    dst_buf: str
    dst_region: Optional[BufferRegion]
    chunk_idx: int
    dependency: List[Dependency] = field(default_factory=list)
    set_signals: List[Signal] = field(default_factory=list)
    peer: Optional[int] = None
    period: Period = field(default_factory=Period)
    reduce_op: Optional[ReduceOp] = None

    def __post_init__(self) -> None:
        if self.op in (TransferOp.PULL, TransferOp.PUSH):
            assert self.peer is not None
        else:
            assert self.peer is None

    # -- contiguous fast-path views (None when a side is scattered or dynamic) --

    @property
    def nbytes(self) -> Optional[int]:
        if self.src_region is None or self.dst_region is None:
            return None
        if not (self.src_region.is_contiguous() and self.dst_region.is_contiguous()):
            return None
        n_src, n_dst = self.src_region.total_nbytes(), self.dst_region.total_nbytes()
        if n_src != n_dst:
            raise ValueError("source and destination regions disagree on total bytes")
        return n_src

    @property
    def src_off(self) -> Optional[int]:
        if self.src_region and self.src_region.is_contiguous():
            return self.src_region.to_segments()[0].offset
        return None

    @property
    def dst_off(self) -> Optional[int]:
        if self.dst_region and self.dst_region.is_contiguous():
            return self.dst_region.to_segments()[0].offset
        return None

    def split(self, num_splits: int) -> List["Transfer"]:
        if num_splits <= 1:
            return [self]
        if self.src_region is None or self.dst_region is None:
            raise ValueError("Cannot split a Transfer with dynamic regions.")
        src_parts = self.src_region.split(num_splits)
        dst_parts = self.dst_region.split(num_splits)
        if len(src_parts) != len(dst_parts):
            raise ValueError("Source and destination splits differ in count")
        self.period.split(num_splits)   # checks the period is still unscheduled; pieces keep 1.0
        pieces = []
        for i, (s, d) in enumerate(zip(src_parts, dst_parts)):
            # splitting is only defined before dependencies and signals are planned
            assert len(self.dependency) == 0
            assert len(self.set_signals) == 0
            pieces.append(Transfer(op=self.op, src_buf=self.src_buf, src_region=s, dst_buf=self.dst_buf,
                                   dst_region=d, chunk_idx=self.chunk_idx * num_splits + i,
                                   dependency=copy.deepcopy(self.dependency), peer=self.peer,
                                   set_signals=copy.deepcopy(self.set_signals)))
        return pieces

    def to_memcpys(self) -> List[Tuple[int, int, int]]:
        """(src_offset, dst_offset, nbytes) copies that move src_region onto dst_region,
        walking both segment lists in lockstep and fusing a piece into the previous one
        when it is adjacent on both sides (descriptor.py:513-590)."""
        if self.src_region is None or self.dst_region is None:
            raise ValueError("Cannot materialize memcpy plan for dynamic regions.")
        src, dst = self.src_region.to_segments(), self.dst_region.to_segments()
        if not src or not dst:
            return []
        if len(src) == 1 and len(dst) == 1:
            if src[0].nbytes != dst[0].nbytes:
                raise ValueError("Source and destination byte counts differ.")
            return [(src[0].offset, dst[0].offset, src[0].nbytes)] if src[0].nbytes else []
        if sum(s.nbytes for s in src) != sum(d.nbytes for d in dst):
            raise ValueError("Source and destination regions disagree on total bytes.")
        if sum(s.nbytes for s in src) == 0:
            return []
        if any(s.nbytes == 0 for s in src) or any(d.nbytes == 0 for d in dst):
            raise RuntimeError("Encountered zero-length segment while constructing memcpy plan.")
        copies: List[Tuple[int, int, int]] = []
        si = di = 0
        s_used = d_used = 0     # bytes already consumed of src[si] / dst[di]
        while si < len(src) and di < len(dst):
            n = min(src[si].nbytes - s_used, dst[di].nbytes - d_used)
            s_at, d_at = src[si].offset + s_used, dst[di].offset + d_used
            if copies and copies[-1][0] + copies[-1][2] == s_at and copies[-1][1] + copies[-1][2] == d_at:
                copies[-1] = (copies[-1][0], copies[-1][1], copies[-1][2] + n)
            else:
                copies.append((s_at, d_at, n))
            s_used += n
            d_used += n
            if s_used == src[si].nbytes:
                si, s_used = si + 1, 0
            if d_used == dst[di].nbytes:
                di, d_used = di + 1, 0
        return copies


@dataclass
class Collective:
    """A library collective over one region pair."""

    op: CollectiveOp
    src_buf: str
    src_region: Optional[BufferRegion]
    dst_buf: str
    dst_region: Optional[BufferRegion]
    dependency: List[Dependency] = field(default_factory=list)
    set_signals: List[Signal] = field(default_factory=list)
    period: Period = field(default_factory=Period)

    def split(self, num_splits: int) -> List["Collective"]:
        if num_splits <= 1:
            return [self]
        if self.src_region is None or self.dst_region is None:
            raise ValueError("Cannot split a Collective with dynamic regions.")
        src_parts = self.src_region.split(num_splits)
        dst_parts = self.dst_region.split(num_splits)
        if len(src_parts) != len(dst_parts):
            raise ValueError("Source and destination splits differ in count")
        piece_period = self.period.split(num_splits)
        pieces = []
        for s, d in zip(src_parts, dst_parts):
            assert len(self.dependency) == 0
            assert len(self.set_signals) == 0
            pieces.append(Collective(op=self.op, src_buf=self.src_buf, src_region=s, dst_buf=self.dst_buf,
                                     dst_region=d, dependency=copy.deepcopy(self.dependency),
                                     set_signals=copy.deepcopy(self.set_signals), period=piece_period))
        return pieces


CommOp = Union[Transfer, Collective]


# --------------------------------------------------------------------------- per-device plan


def _region_text(buf: str, region: Optional[BufferRegion]) -> str:
    return f"{buf}[?]" if region is None else f"{buf}{region.describe()}"


def _op_text(op: CommOp) -> str:
    route = f"{_region_text(op.src_buf, op.src_region)} -> {_region_text(op.dst_buf, op.dst_region)}"
    if isinstance(op, Collective):
        return f"collective {op.op.value} {route}"
    if op.op == TransferOp.LOCAL_COPY:
        return f"copy {route}"
    peer = "?" if op.peer is None else op.peer
    return f"{op.op.value} peer={peer} {route}"


def _format_signal(signal: Signal) -> str:
    return f"{signal.type.value}@{signal.dst_rank}[{signal.dst_offset}]"


@dataclass
class DevicePlan:
    """Everything one rank does: streams of ops, what is resident up front, buffer shapes."""

    dev: int
    xfer: List[List[CommOp]] = field(default_factory=list)
    local_regions: Dict[str, List[BufferRegion]] = field(default_factory=dict)
    # (signal received here, signal to forward): the receiver of a push relays
    # completion to a third rank
    transit_signals: List[Tuple[Signal, Signal]] = field(default_factory=list)
    tensors_involved: Dict[str, Tuple[torch.Size, torch.dtype]] = field(default_factory=dict)

    def __post_init__(self) -> None:
        if not self.xfer:
            self.xfer.append([])

    def _ensure_stream(self, idx: int) -> List[CommOp]:
        if idx < 0:
            raise ValueError("stream index must be non-negative")
        while len(self.xfer) <= idx:
            self.xfer.append([])
        return self.xfer[idx]

    def add_op(self, op: CommOp, *, stream_idx: int = 0) -> None:
        self._ensure_stream(stream_idx).append(op)

    def add_stream(self) -> int:
        self.xfer.append([])
        return len(self.xfer) - 1

    def _ops(self) -> Iterable[CommOp]:
        for stream in self.xfer:
            yield from stream

    @property
    def xfers(self) -> List[Transfer]:
        return [op for op in self._ops()
                if isinstance(op, Transfer) and op.op in (TransferOp.PUSH, TransferOp.PULL)]

    @property
    def local_copies(self) -> List[Transfer]:
        return [op for op in self._ops() if isinstance(op, Transfer) and op.op == TransferOp.LOCAL_COPY]

    def pretty(self) -> str:
        lines = [f"DevicePlan(dev={self.dev})"]
        for s, stream in enumerate(self.xfer):
            lines.append(f"  Stream {s}:")
            if not stream:
                lines.append("    (none)")
            for i, op in enumerate(stream):
                lines.append(f"    [{i}] {_op_text(op)}")
        return "\n".join(lines)

    def __str__(self) -> str:
        return self.pretty()

    def split_xfers(self, num_splits: int) -> "DevicePlan":
        streams: List[List[CommOp]] = []
        for stream in self.xfer:
            out: List[CommOp] = []
            for op in stream:
                cross = isinstance(op, Transfer) and op.op in (TransferOp.PUSH, TransferOp.PULL)
                if cross or isinstance(op, Collective):
                    out.extend(op.split(num_splits))
                else:
                    out.append(copy.deepcopy(op))
            streams.append(out)
        return DevicePlan(dev=self.dev, xfer=streams, local_regions=copy.deepcopy(self.local_regions),
                          transit_signals=copy.deepcopy(self.transit_signals),
                          tensors_involved=copy.deepcopy(self.tensors_involved))

    def check_no_dependency(self) -> bool:
        # `dependency` is always a list, so any cross-device transfer or collective makes
        # this False — the reference behaves the same (descriptor.py:738-745)
        for op in self._ops():
            cross = isinstance(op, Transfer) and op.op in (TransferOp.PUSH, TransferOp.PULL)
            if (cross or isinstance(op, Collective)) and op.dependency is not None:
                return False
        return True


# --------------------------------------------------------------------------- whole plan


class CommPlan:
    """All device plans plus the signal counters that planning hands out."""

    def __init__(self, device_plans: Optional[Dict[int, DevicePlan]] = None) -> None:
        self.device_plans: Dict[int, DevicePlan] = device_plans or {}
        self.receive_signal_counters: Dict[int, int] = {dev: 0 for dev in self.device_plans}
        self.transit_signal_counters: Dict[int, int] = {dev: 0 for dev in self.device_plans}
        self.compute_signal_counters: Dict[int, int] = {dev: 0 for dev in self.device_plans}

    def add_device_plan(self, plan: DevicePlan) -> None:
        if plan.dev in self.device_plans:
            raise ValueError(f"device plan for dev {plan.dev} already exists")
        self.device_plans[plan.dev] = plan

    @property
    def xfers(self) -> List[Transfer]:
        return [t for plan in self.device_plans.values() for t in plan.xfers]

    def _walk(self):
        """(dev, stream index, op index, op) in planning order: devices as inserted,
        streams and ops in list order."""
        for dev, plan in self.device_plans.items():
            for s, stream in enumerate(plan.xfer):
                for i, op in enumerate(stream):
                    yield dev, s, i, op

    # ---- text --------------------------------------------------------------

    def pretty(self, include_signals: bool = False) -> str:
        lines = [f"CommPlan(devices={len(self.device_plans)})"]
        for dev in sorted(self.device_plans):
            plan = self.device_plans[dev]
            lines.extend("  " + ln for ln in plan.pretty().splitlines())
            if include_signals:
                lines.extend(self._format_signal_details(plan))
        return "\n".join(lines)

    def visualize_signals(self) -> str:
        lines = ["CommPlan Signals:"]
        for dev in sorted(self.device_plans):
            lines.append(f"  Device {dev}:")
            lines.extend(self._format_signal_details(self.device_plans[dev]) or ["    (no signal activity)"])
        return "\n".join(lines)

    def _format_signal_details(self, dev_plan: DevicePlan) -> List[str]:
        lines: List[str] = []
        for s, stream in enumerate(dev_plan.xfer):
            if not stream:
                lines.append(f"    Stream {s}: (none)")
                continue
            lines.append(f"    Stream {s}:")
            for i, op in enumerate(stream):
                raised = ", ".join(_format_signal(sig) for sig in op.set_signals) or "(none)"
                lines.append(f"      op[{i}] {op.op.value} -> signals: {raised}")
                for d, dep in enumerate(op.dependency or []):
                    waits = "pending" if dep.signal is None else _format_signal(dep.signal)
                    if isinstance(dep, XferDependency):
                        src = f"xfer({dep.depend_rank},{dep.depend_xfer_stream},{dep.depend_xfer_idx})"
                    elif isinstance(dep, ComputeDependency):
                        src = f"compute({dep.compute_rank})"
                    else:
                        continue
                    lines.append(f"        dep[{d}] <- {src} -> {waits}")
        if dev_plan.transit_signals:
            lines.append("    Transit signals:")
            for got, forward in dev_plan.transit_signals:
                lines.append(f"      {_format_signal(got)} -> {_format_signal(forward)}")
        return lines

    # ---- signal planning ---------------------------------------------------

    def _check_compute_dependency_signals_set(self, plan_compute_signals: bool) -> bool:
        for _, _, _, op in self._walk():
            for dep in op.dependency:
                if isinstance(dep, ComputeDependency) and (dep.signal is not None) == plan_compute_signals:
                    return False
        return True

    def _take(self, counters: Dict[int, int], dev: int) -> int:
        if dev not in counters:
            raise ValueError(f"device {dev} not in signal counter")
        counters[dev] += 1
        return counters[dev] - 1

    def plan_signals(self, plan_compute_signals: bool = True) -> None:
        """Assign a flag word to every completion and every dependency
        (descriptor.py:860-988).

        Pass 1: each op raises one RECEIVE_DATA signal at the rank where its data
        lands (the peer for a push, the op's own rank otherwise); offsets are the
        running per-rank counter in planning order.  Pass 2: an XferDependency
        reuses that signal when the waiting rank is the one it is raised at,
        otherwise a REMOTE_DATA_READY signal is added (relayed by the push
        receiver as a transit signal, or raised directly by a pull / local copy);
        a ComputeDependency gets a COMPUTE_DONE signal from the waiting rank's
        compute counter.
        """
        assert all(not p.transit_signals for p in self.device_plans.values()), \
            "transit_signals should be empty before planning signals"
        assert all(not op.set_signals for _, _, _, op in self._walk()), \
            "set_signals should be empty before planning signals"
        assert self._check_compute_dependency_signals_set(plan_compute_signals), \
            "if plan_compute_signals is True, compute dependency signals should be None before " \
            "planning; if False, they should be already set"

        for dev, _, _, op in self._walk():
            lands_at = op.peer if isinstance(op, Transfer) and op.op == TransferOp.PUSH else dev
            if isinstance(op, Transfer) and op.op == TransferOp.PUSH:
                assert op.peer is not None
            op.set_signals.append(Signal(dst_rank=lands_at,
                                         dst_offset=self._take(self.receive_signal_counters, lands_at),
                                         type=SignalType.RECEIVE_DATA))

        for dev, _, _, op in self._walk():
            for dep in op.dependency:
                if isinstance(dep, ComputeDependency):
                    if plan_compute_signals:
                        dep.signal = Signal(dst_rank=dep.compute_rank,
                                            dst_offset=self._take(self.compute_signal_counters, dev),
                                            type=SignalType.COMPUTE_DONE)
                    continue
                if not isinstance(dep, XferDependency):
                    raise ValueError(f"unknown dependency type: {type(dep)}")
                if isinstance(op, Collective):
                    raise ValueError("Collective operations cannot have XferDependency for now")
                upstream_plan = self.device_plans.get(dep.depend_rank)
                assert upstream_plan is not None, f"depend_rank {dep.depend_rank} not found in device_plans"
                upstream = upstream_plan.xfer[dep.depend_xfer_stream][dep.depend_xfer_idx]
                if not isinstance(upstream, Transfer):
                    raise ValueError("XferDependency can only depend on Collective operations for now")
                landed = upstream.set_signals[0]      # the RECEIVE_DATA signal is always first
                if upstream.op == TransferOp.PUSH:
                    if dev == upstream.peer:
                        assert landed.type == SignalType.RECEIVE_DATA
                        dep.signal = landed
                    else:
                        assert upstream.peer is not None
                        relay = Signal(dst_rank=dev,
                                       dst_offset=self._take(self.transit_signal_counters, dev),
                                       type=SignalType.REMOTE_DATA_READY)
                        self.device_plans[upstream.peer].transit_signals.append((landed, relay))
                        dep.signal = relay
                else:
                    if dev == dep.depend_rank:
                        assert landed.type == SignalType.RECEIVE_DATA
                        dep.signal = landed
                    else:
                        extra = Signal(dst_rank=dev,
                                       dst_offset=self._take(self.receive_signal_counters, dev),
                                       type=SignalType.REMOTE_DATA_READY)
                        upstream.set_signals.append(extra)
                        dep.signal = extra

    # ---- timing ------------------------------------------------------------

    def estimate_period(self) -> None:
        """Earliest start of every op given stream order and XferDependency edges
        (compute dependencies ignored); Kahn's algorithm with FIFO ready queue
        (descriptor.py:990-1061).  Signals start when their op completes."""
        ops: List[CommOp] = []
        index: Dict[Tuple[int, int, int], int] = {}
        parents: List[set] = []
        children: List[List[int]] = []

        def link(parent: int, child: int) -> None:
            if parent not in parents[child]:
                parents[child].add(parent)
                children[parent].append(child)

        for dev, s, i, op in self._walk():
            node = len(ops)
            ops.append(op)
            index[(dev, s, i)] = node
            parents.append(set())
            children.append([])
            if i > 0:
                link(index[(dev, s, i - 1)], node)
        if not ops:
            return
        for dev, s, i, op in self._walk():
            for dep in op.dependency:
                if not isinstance(dep, XferDependency):
                    continue
                key = (dep.depend_rank, dep.depend_xfer_stream, dep.depend_xfer_idx)
                if key not in index:
                    raise ValueError(f"dependency target {key} not found in communication plan")
                link(index[key], index[(dev, s, i)])

        waiting = [len(p) for p in parents]
        ready_at = [0.0] * len(ops)
        queue = deque(n for n, w in enumerate(waiting) if w == 0)
        done = 0
        while queue:
            node = queue.popleft()
            done += 1
            op = ops[node]
            op.period.start = ready_at[node]
            finish = ready_at[node] + op.period.duration
            for sig in op.set_signals:
                sig.period.start = finish
            for child in children[node]:
                waiting[child] -= 1
                ready_at[child] = max(ready_at[child], finish)
                if waiting[child] == 0:
                    queue.append(child)
        if done != len(ops):
            raise RuntimeError("cycle detected in transfer dependencies")


__all__ = [
    "CommPlan",
    "DevicePlan",
    "Transfer",
    "TransferOp",
    "Collective",
    "CollectiveOp",
    "CommOp",
    "Signal",
    "SignalType",
    "ReduceOp",
    "Period",
    "CommDescriptor",
    "DataPlacement",
    "XferDependency",
    "ComputeDependency",
    "MemorySegment",
    "BufferRegion",
    "AxisSlice",
    "cdiv",
]
