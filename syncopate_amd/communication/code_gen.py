"""Plan -> flat op lists per rank and stream (wait*, copy*, signal* for every op).

Behavioural restatement of syncopate/communication/code_gen.py
(`CodeGenOptions` :7-30, `CommGenerator.generate_code_for_plan` :36-181,
`_get_buffer_info` :184-199).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Tuple

from .comm_runtime.operations import (
    CollectiveComm,
    CommInfo,
    CopyEngineOp,
    IntraNodeSignal,
    SMCopyOp,
    WaitIntraNodeSignal,
)
from .descriptor import (
    AxisSlice,
    BufferRegion,
    Collective,
    CollectiveOp,
    CommPlan,
    ComputeDependency,
    SignalType,
    Transfer,
    TransferOp,
    XferDependency,
)


@dataclass
class CodeGenOptions:
    copy_engine: bool = True               # contiguous byte copies (hipMemcpyAsync) vs box copies on CUs
    low_latency: bool = False
    use_tma: bool = True                   # carried on SMCopyOp records; no meaning on CDNA4
    fuse_with_compute_intra: bool = False
    fuse_with_compute_inter: bool = False

    def validate(self) -> None:
        if self.low_latency:
            raise NotImplementedError("low_latency codegen is not implemented yet")
        if self.copy_engine and self.fuse_with_compute_intra:
            raise ValueError("copy_engine and fuse_with_compute_intra cannot be both enabled")
        if self.fuse_with_compute_inter and not self.fuse_with_compute_intra:
            raise ValueError("fuse_with_compute_inter requires fuse_with_compute_intra to be enabled")


def _boxes_in_buffer_coordinates(region: BufferRegion) -> List[Tuple[AxisSlice, ...]]:
    """The region's boxes with base_offset folded into the axis indices (code_gen.py:49-67)."""
    shifts = [0] * len(region.strides)
    if region.base_offset:
        if region.base_offset % region.elem_size:
            raise ValueError("base_offset must align with elem_size for TMA copy")
        rest = region.base_offset // region.elem_size
        for axis, stride in enumerate(region.strides):
            shifts[axis], rest = divmod(rest, stride)
        if rest:
            raise ValueError("base_offset not representable by strides for TMA copy")
    return [tuple(AxisSlice(ax.start + sh, ax.end + sh) for ax, sh in zip(box, shifts))
            for box in region.regions]


def _endpoints(op: Transfer, dev: int) -> Tuple[int, int]:
    """(source rank, destination rank) of a transfer issued by `dev`."""
    if op.op == TransferOp.LOCAL_COPY:
        return dev, dev
    assert op.peer is not None
    return (dev, op.peer) if op.op == TransferOp.PUSH else (op.peer, dev)


class CommGenerator(CommPlan):
    """A CommPlan that can also be flattened into the op lists a runtime replays."""

    options: CodeGenOptions

    def generate_code_for_plan(self, options: CodeGenOptions = CodeGenOptions()) -> CommInfo:
        options.validate()
        info = CommInfo()
        info.world_size = len(self.device_plans)
        (info.recv_signal_num, info.transit_signal_num, info.compute_signal_num,
         info.comm_buffer_sizes) = self._get_buffer_info()

        for dev, plan in self.device_plans.items():
            info.operations.append([])
            for stream in plan.xfer:
                ops: List = []
                info.operations[dev].append(ops)
                for op in stream:
                    ops.extend(self._waits(op))
                    if isinstance(op, Collective):
                        ops.extend(self._collective(op))
                    elif isinstance(op, Transfer):
                        ops.extend(self._copies(op, plan.dev, options))
                    for sig in op.set_signals:
                        # intra-node only: a stream-ordered flag write reaches the target
                        assert sig.type == SignalType.RECEIVE_DATA
                        ops.append(IntraNodeSignal(signal_type=sig.type, offset=sig.dst_offset,
                                                   rank=sig.dst_rank))
        return info

    @staticmethod
    def _waits(op) -> List[WaitIntraNodeSignal]:
        waits = []
        for dep in op.dependency:
            if isinstance(dep, ComputeDependency):
                assert dep.signal is not None
                waits.append(WaitIntraNodeSignal(signal_type=SignalType.COMPUTE_DONE,
                                                 offset=dep.signal.dst_offset, rank=dep.signal.dst_rank))
            elif isinstance(dep, XferDependency):
                if dep.signal is None:
                    raise ValueError("XferDependency requires planned signals before codegen")
                waits.append(WaitIntraNodeSignal(signal_type=dep.signal.type, offset=dep.signal.dst_offset,
                                                 rank=dep.signal.dst_rank))
            else:
                raise NotImplementedError("dependency handling is not implemented yet")
        return waits

    @staticmethod
    def _collective(op: Collective) -> List[CollectiveComm]:
        if op.src_region is None or op.dst_region is None:
            raise ValueError("Collective requires materialized regions.")
        if op.op == CollectiveOp.ALL_REDUCE and op.src_buf != op.dst_buf:
            raise ValueError("ALL_REDUCE must use the same buffer for src and dst.")
        src_boxes = _boxes_in_buffer_coordinates(op.src_region)
        dst_boxes = _boxes_in_buffer_coordinates(op.dst_region)
        if len(src_boxes) != len(dst_boxes):
            raise ValueError("source and destination region counts differ for collective")
        return [CollectiveComm(op=op.op, src=op.src_buf, dst=op.dst_buf, src_slice=s, dst_slice=d)
                for s, d in zip(src_boxes, dst_boxes)]

    @staticmethod
    def _copies(op: Transfer, dev: int, options: CodeGenOptions) -> List:
        src_rank, dst_rank = _endpoints(op, dev)
        if options.copy_engine:
            if op.reduce_op is not None:
                raise ValueError("Copy engine transfer cannot do reduction.")
            return [CopyEngineOp(src_rank=src_rank, dst_rank=dst_rank, src=op.src_buf, dst=op.dst_buf,
                                 src_offset=s, dst_offset=d, size=n) for s, d, n in op.to_memcpys()]
        assert op.src_region is not None and op.dst_region is not None
        src_boxes = _boxes_in_buffer_coordinates(op.src_region)
        dst_boxes = _boxes_in_buffer_coordinates(op.dst_region)
        if len(src_boxes) != len(dst_boxes):
            raise ValueError("source and destination region counts differ for TMA copy")
        return [SMCopyOp(use_tma=options.use_tma, src_rank=src_rank, dst_rank=dst_rank, src=op.src_buf,
                         dst=op.dst_buf, src_slice=s, dst_slice=d, reduce_op=op.reduce_op)
                for s, d in zip(src_boxes, dst_boxes)]

    def _get_buffer_info(self) -> Tuple[int, int, int, dict]:
        """Flag-array lengths (the largest counter any rank reached) and buffer shapes."""
        def most(counters) -> int:
            return max(counters.values()) if counters else 0

        buffers = {}
        for plan in self.device_plans.values():
            for name, spec in plan.tensors_involved.items():
                if buffers.setdefault(name, spec) != spec:
                    raise ValueError(f"Buffer {name} has inconsistent size or dtype across devices.")
        return (most(self.receive_signal_counters), most(self.transit_signal_counters),
                most(self.compute_signal_counters), buffers)
