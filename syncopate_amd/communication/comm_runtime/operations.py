"""Flat op records a CommInfo is made of: what one rank's comm streams execute, in order.

Same record types and fields as the reference
(syncopate/communication/comm_runtime/operations.py:6-106).
"""

from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..descriptor import AxisSlice, CollectiveOp, ReduceOp, SignalType


class _Record:
    """Keyword-initialised record with a stable text form."""

    _shown: Tuple[str, ...] = ()

    def __init__(self, **fields) -> None:
        for name, value in fields.items():
            setattr(self, name, value)

    def __str__(self) -> str:
        body = ", ".join(f"{self._label(n)}={getattr(self, n, None)}" for n in self._shown)
        return f"{type(self).__name__}({body})"

    @staticmethod
    def _label(name: str) -> str:
        return name


class CopyEngineOp(_Record):
    """A contiguous byte copy between two ranks' buffers (hipMemcpyAsync)."""

    src: str
    dst: str
    src_rank: int
    dst_rank: int
    src_offset: int
    dst_offset: int
    size: int
    _shown = ("src_rank", "dst_rank", "src_offset", "dst_offset", "size")


class SMCopyOp(_Record):
    """A strided box copy done by a compute-unit kernel, optionally accumulating."""

    src: str
    dst: str
    src_rank: int
    dst_rank: int
    src_slice: Tuple[AxisSlice, ...]
    dst_slice: Tuple[AxisSlice, ...]
    reduce_op: Optional[ReduceOp] = None
    use_tma: bool = True
    _shown = ("src_rank", "dst_rank", "src_slice", "dst_slice", "reduce_op")


class CollectiveComm(_Record):
    op: CollectiveOp
    src: str
    dst: str
    src_slice: Tuple[AxisSlice, ...]
    dst_slice: Tuple[AxisSlice, ...]
    _shown = ("op", "src", "dst", "src_slice", "dst_slice")


class IntraNodeSignal(_Record):
    """Set flag word `offset` of `rank`'s array of `signal_type` to 1."""

    signal_type: SignalType
    offset: int
    rank: int
    _shown = ("signal_type", "offset", "rank")

    @staticmethod
    def _label(name: str) -> str:
        return "type" if name == "signal_type" else name


class WaitIntraNodeSignal(_Record):
    """Stall the stream until flag word `offset` of `rank`'s array of `signal_type` equals 1."""

    signal_type: SignalType
    offset: int
    rank: int
    _shown = ("signal_type", "offset", "rank")

    @staticmethod
    def _label(name: str) -> str:
        return "type" if name == "signal_type" else name


class CommInfo:
    """Everything a runtime needs to execute a planned communication."""

    world_size: int
    local_world_size: int
    recv_signal_num: int
    transit_signal_num: int
    compute_signal_num: int
    comm_buffer_sizes: Dict[str, Tuple[torch.Size, torch.dtype]]
    operations: List[List[List]]   # [rank][stream] -> ops in issue order
    num_copy_sms: int
    need_green_ctx: bool

    def __init__(self) -> None:
        self.world_size = 0
        self.local_world_size = 0
        self.recv_signal_num = 0
        self.transit_signal_num = 0
        self.compute_signal_num = 0
        self.comm_buffer_sizes = {}
        self.operations = []
        self.num_copy_sms = 0
        self.need_green_ctx = False

    def __str__(self) -> str:
        lines = [
            f"world_size={self.world_size}",
            f"local_world_size={self.local_world_size}",
            f"recv_signal_num={self.recv_signal_num}",
            f"transit_signal_num={self.transit_signal_num}",
            f"compute_signal_num={self.compute_signal_num}",
        ]
        if self.comm_buffer_sizes:
            lines.append("comm_buffers:")
            lines.extend(f"  {name}: shape={tuple(shape)} dtype={dtype}"
                         for name, (shape, dtype) in self.comm_buffer_sizes.items())
        else:
            lines.append("comm_buffers: none")
        for rank, streams in enumerate(self.operations):
            lines.append(f"rank {rank}:")
            for s, ops in enumerate(streams):
                lines.append(f"  stream {s}:")
                lines.extend(f"    {op}" for op in ops)
        return "\n".join(lines)
