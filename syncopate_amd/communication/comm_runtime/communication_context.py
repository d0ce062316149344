"""Single-GPU executor of a CommInfo: replays one rank's op list on side streams.

Counterpart of the reference runtime
(syncopate/communication/comm_runtime/communication_context.py: `__init__`
:31-76, `reset_signals` :90-96, `start_after`/`end_before` :98-106, `execute`
:108-235, `get_graph` :242-249), with the other ranks simulated on the same
MI355X: every rank's "symmetric" buffers and flag arrays are ordinary device
tensors of this process, a cross-rank copy is a hipMemcpyAsync between two of
them, a flag write is a one-wavefront kernel doing a system-scope release
store and a flag wait is a one-wavefront kernel spinning (with a time-out) on
the word.  Only the ops of `rank` are executed, in exactly the order the op
list prescribes, so a consumer kernel launched on the compute stream really
overlaps with data arriving chunk by chunk.

`execute_mesh` replays the op lists of ALL ranks on one stream, in an order that
honours every flag wait, for plans whose data reaches this rank through its
neighbours' forwarding (ring, double ring).

On a multi-GPU node the same op list would be replayed with the peers'
buffers mapped through IPC and one stream per peer link; that path is not
built here.
"""

from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ... import _lib
from ..descriptor import CollectiveOp, ReduceOp, SignalType
from .operations import (
    CollectiveComm,
    CommInfo,
    CopyEngineOp,
    IntraNodeSignal,
    SMCopyOp,
    WaitIntraNodeSignal,
)
from ...computation._launch import trust_flags
from .cu_partition import split_device_cu_mask
from .persistent_copy import persistent_copy_last_contig
from .streams import pick_side_streams

SIGNAL_DTYPE = torch.int64   # 8-byte flag words, value 1 = set


class CommContext:
    rank: int
    info: CommInfo
    recv_signal_bufs: List[torch.Tensor]
    transit_signal_bufs: List[torch.Tensor]
    compute_signal_bufs: List[torch.Tensor]
    comm_buffers: Dict[str, List[torch.Tensor]]
    streams: List[torch.cuda.Stream]

    def __init__(self, rank: int, info: CommInfo, multi_info: bool = False, *,
                 device: Optional[torch.device] = None, link_delay_us: int = 0,
                 wait_timeout_us: int = 2_000_000, copy_blocks: int = 0, flag_sets: int = 1,
                 compute_stream: Optional[torch.cuda.Stream] = None, fuse_flags: bool = False,
                 lead_copy_blocks: int = 0, flag_write_values: bool = False, list_blocks: int = 0) -> None:
        if info.local_world_size <= 0:
            info.local_world_size = info.world_size
        if info.local_world_size != info.world_size:
            raise NotImplementedError("the single-GPU executor simulates one node: "
                                      "local_world_size must equal world_size")
        if not 0 <= rank < info.world_size:
            raise ValueError(f"rank {rank} outside world of {info.world_size}")
        self.rank = rank
        self.local_rank = rank % info.local_world_size
        self.node_id = rank // info.local_world_size
        self.info = info
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
        self.link_delay_us = int(link_delay_us)
        self.wait_timeout_us = int(wait_timeout_us)
        # 0: contiguous copies go through hipMemcpyAsync; > 0: through a streaming copy kernel of
        # that many 256-thread workgroups (16-byte aligned copies only)
        self.copy_blocks = int(copy_blocks)
        # with copy_blocks > 0: a copy that is followed by its flag write in the op list becomes
        # ONE kernel that copies and then sets the flag (execute() only)
        self.fuse_flags = bool(fuse_flags)
        if self.fuse_flags and self.copy_blocks <= 0:
            raise ValueError("fuse_flags needs the copy kernel: copy_blocks > 0")
        # > 0: among the leading ops of execute(lead_ops=n), a copy that is followed by its flag
        # write is ONE kernel of that many workgroups that copies and then sets the flag.  The
        # compute kernel has not been launched yet, so these copies may take the whole device.
        self.lead_copy_blocks = int(lead_copy_blocks)
        # flag writes as stream memory operations instead of one-wavefront kernels (outside graph capture)
        self.flag_write_values = bool(flag_write_values)
        # > 0: an op list that is nothing but (copy, flag write) pairs is issued by execute() as ONE kernel
        # of that many workgroups which walks the list (two kernels with lead_ops: the leading pairs, with
        # lead_copy_blocks workgroups if given, and the rest).  No kernel starts or ends on the device while
        # the consumer runs, so nothing writes back or invalidates the L2s its operands are cached in.
        self.list_blocks = int(list_blocks)
        self._list_records: Dict[tuple, tuple] = {}
        self._list_tickets: Dict[int, torch.Tensor] = {}
        self._lib = _lib.load()
        world = info.local_world_size

        def flag_arrays(count: int) -> List[torch.Tensor]:
            if count <= 0:
                return []
            return [torch.zeros((count,), dtype=SIGNAL_DTYPE, device=self.device) for _ in range(world)]

        # One set of flag arrays is the reference's arrangement: reset_signals() zeroes it in front
        # of every iteration, and the compute kernel can only be launched behind that fill.  With
        # two sets reset_signals() switches to the other (already zero) set and the one just left
        # is zeroed at the tail of the next execute(), off the compute stream's path: iterations
        # then follow each other without a fill between the kernels.
        if flag_sets not in (1, 2):
            raise ValueError("flag_sets must be 1 or 2")
        self._flag_sets = [
            (flag_arrays(info.recv_signal_num), flag_arrays(info.transit_signal_num),
             flag_arrays(info.compute_signal_num))
            for _ in range(flag_sets)
        ]
        # this executor's copies are the only writers of its buffers and its flags are reset between iterations:
        # kernels that wait on these arrays may skip the acquire fence when a flag is already up
        for flag_set in self._flag_sets:
            for group in flag_set:
                trust_flags(*group)
        self._cur_set = 0
        self._stale_set: Optional[int] = None
        self._stale_whole_mesh = False
        self.recv_signal_bufs, self.transit_signal_bufs, self.compute_signal_bufs = self._flag_sets[0]
        self.comm_buffers = {
            name: [torch.zeros(tuple(shape), dtype=dtype, device=self.device) for _ in range(world)]
            for name, (shape, dtype) in info.comm_buffer_sizes.items()
        }
        self.status = torch.zeros(_lib.SYN_STATUS_WORDS, dtype=torch.int32, device=self.device)
        self._sole_writer_ops = self._find_sole_writer_ops()
        # one workgroup counter per communication stream for the fused copy + flag kernel
        self._tickets = torch.zeros(max(1, len(info.operations[self.rank])), dtype=torch.int32, device=self.device)
        # one stream per op list, none of them on the hardware queue of the stream the compute
        # kernels are launched on (the current stream unless `compute_stream` names it): a flag
        # wait spinning on a shared queue would hold back the very kernel that sets the flag
        if info.need_green_ctx:
            # the device split in two (communication_context.py:66-72): `num_copy_sms` compute
            # units (rounded up to a whole number per XCD) for the one communication stream, the
            # rest for `self.compute_stream`, on which the caller launches its kernels
            if len(info.operations[self.rank]) != 1:
                raise ValueError("a split device carries one communication stream")
            if info.num_copy_sms <= 0:
                raise ValueError("a split device needs CommInfo.num_copy_sms compute units for communication")
            (comm, rest), self.cu_split = split_device_cu_mask(self.device, 1, info.num_copy_sms)
            self.streams = [comm]
            self.compute_stream = rest
        else:
            self.cu_split = None
            self.compute_stream = (torch.cuda.current_stream(self.device) if compute_stream is None
                                   else compute_stream)
            self.streams = pick_side_streams(len(info.operations[self.rank]), self.compute_stream, self.device)

    # ---- flags and stream ordering -------------------------------------------

    def _zero_set(self, index: int, whole_mesh: bool) -> None:
        for group in self._flag_sets[index]:
            if group:
                for r in (range(len(group)) if whole_mesh else (self.local_rank,)):
                    group[r].fill_(0)

    def reset_signals(self, whole_mesh: bool = False) -> None:
        """Zero this rank's flag words (every simulated rank's with `whole_mesh`).

        With two flag sets: make the other set current (`recv_signal_bufs` etc. then name ITS
        arrays - pass them to the kernels after this call) and leave the old one to be zeroed at
        the end of the next execute().  That is only safe in the reference's call order,
        reset_signals -> start_after(compute stream) -> execute -> kernels -> end_before: the
        communication streams then start after the previous iteration's kernels, the last readers
        of the old set."""
        if len(self._flag_sets) == 1:
            self._zero_set(0, whole_mesh)
            return
        self._stale_set = self._cur_set
        self._stale_whole_mesh = whole_mesh
        self._cur_set = 1 - self._cur_set
        self.recv_signal_bufs, self.transit_signal_bufs, self.compute_signal_bufs = self._flag_sets[self._cur_set]

    def _zero_stale_set(self) -> None:
        if self._stale_set is None or not self.streams:
            return
        with torch.cuda.stream(self.streams[-1]):
            self._zero_set(self._stale_set, self._stale_whole_mesh)
        self._stale_set = None

    def start_after(self, stream: Optional[torch.cuda.Stream] = None) -> None:
        """Communication streams start once `stream` has reached this point."""
        stream = torch.cuda.current_stream(self.device) if stream is None else stream
        for comm_stream in self.streams:
            comm_stream.wait_stream(stream)

    def end_before(self, stream: Optional[torch.cuda.Stream] = None) -> None:
        """`stream` continues only after all communication streams have drained.  Call it after
        the compute kernels have been launched: a join enqueued before them on a stream that
        happens to share their hardware queue would hold them back, and with them the flags the
        communication streams are waiting for."""
        stream = torch.cuda.current_stream(self.device) if stream is None else stream
        for comm_stream in self.streams:
            stream.wait_stream(comm_stream)

    # ---- replay --------------------------------------------------------------

    def _flags(self, signal_type: SignalType, rank: int) -> torch.Tensor:
        if signal_type == SignalType.COMPUTE_DONE:
            return self.compute_signal_bufs[rank]
        if signal_type == SignalType.RECEIVE_DATA:
            return self.recv_signal_bufs[rank]
        raise NotImplementedError(f"Signal type {signal_type} not implemented yet.")

    def execute(self, neglect_local: bool = False, lead_ops: int = 0,
                lead_on: Optional[torch.cuda.Stream] = None) -> None:
        """Enqueue this rank's ops, stream by stream, in list order.

        `lead_ops` > 0 records an event behind the first `lead_ops` ops of every stream;
        `wait_lead(stream)` makes a stream wait for them.  Launch order gives the copies that
        head start over the compute kernel when everything is launched from the host; inside a
        replayed graph the kernel and the first copy become ready at the same moment, the kernel
        takes the compute units, and every chunk of the iteration arrives later.

        `lead_on` (with `lead_ops`): the leading ops are enqueued on THAT stream - the compute
        stream, in front of the kernel - and the communication stream carries on behind them.
        A kernel that waits for an event of another hardware queue starts some 10 us after the
        event; behind ops of its own stream it starts at once.  Only for leading ops that wait
        for nothing the compute stream's later kernels set."""
        self._lead_events = []
        self._check_copy_units(self.info.operations[self.rank])
        for lane, (stream, ops) in enumerate(zip(self.streams, self.info.operations[self.rank])):
            lead = min(lead_ops, len(ops))
            if self.list_blocks > 0 and self._issue_as_list(lane, stream, ops, lead, lead_on, neglect_local):
                continue
            index = 0
            while index < len(ops):
                op, done = ops[index], 1
                on = lead_on if (lead_on is not None and index < lead) else stream
                handle = int(on.cuda_stream)
                blocks = self.copy_blocks if self.fuse_flags else 0
                if self.lead_copy_blocks > 0 and index + 1 < lead:
                    blocks = self.lead_copy_blocks
                if (blocks > 0 and isinstance(op, CopyEngineOp) and index + 1 < len(ops)
                        and isinstance(ops[index + 1], IntraNodeSignal)
                        and self._issue_copy_with_flag(op, ops[index + 1], lane, handle, neglect_local, blocks)):
                    done = 2
                else:
                    self._issue(op, self.rank, on, handle, neglect_local)
                if lead_ops > 0 and index < lead <= index + done:
                    event = torch.cuda.Event()
                    event.record(on)
                    if lead_on is not None:
                        stream.wait_event(event)      # the rest of the list follows the leading ops
                    else:
                        self._lead_events.append(event)
                index += done
        self._zero_stale_set()

    def _issue_as_list(self, lane: int, stream: torch.cuda.Stream, ops, lead: int,
                       lead_on: Optional[torch.cuda.Stream], neglect_local: bool) -> bool:
        """The whole op list as one kernel (two with leading ops); False if the list is not made of
        (copy, flag write) pairs that the list kernel can take."""
        world = self.info.local_world_size
        if len(ops) == 0 or len(ops) % 2:
            return False
        # the records hold addresses and sizes: they are good for exactly this op list, these buffers and this delay
        key = (lane, self._cur_set, neglect_local)
        stamp = (tuple(map(id, ops)), self.link_delay_us,
                 tuple(t.data_ptr() for name in sorted(self.comm_buffers) for t in self.comm_buffers[name]),
                 tuple(t.data_ptr() for t in self.recv_signal_bufs))
        cached = self._list_records.get(key)
        records = cached[1] if cached is not None and cached[0] == stamp else None
        if records is None:
            rows = []
            for i in range(0, len(ops), 2):
                op, flag_op = ops[i], ops[i + 1]
                if not (isinstance(op, CopyEngineOp) and isinstance(flag_op, IntraNodeSignal)
                        and flag_op.signal_type == SignalType.RECEIVE_DATA):
                    return False
                src = self.comm_buffers[op.src][op.src_rank % world]
                dst = self.comm_buffers[op.dst][op.dst_rank % world]
                if op.src_offset + op.size > src.numel() * src.element_size() or \
                        op.dst_offset + op.size > dst.numel() * dst.element_size():
                    raise ValueError(f"{op} runs past the end of its buffer")
                dst_ptr, src_ptr = dst.data_ptr() + op.dst_offset, src.data_ptr() + op.src_offset
                if op.size <= 0 or op.size % 16 or dst_ptr % 16 or src_ptr % 16:
                    return False
                flags = self.recv_signal_bufs[flag_op.rank % world]
                if not 0 <= flag_op.offset < flags.numel():
                    raise ValueError(f"{flag_op} is outside the flag array")
                skip = op.src_rank == op.dst_rank and neglect_local
                delay = self.link_delay_us * 100 if (self.link_delay_us and op.src_rank != op.dst_rank) else 0
                rows.append([dst_ptr, src_ptr, 0 if skip else op.size // 16, flags.data_ptr() + 8 * flag_op.offset, 1, delay])
            records = torch.tensor(rows, dtype=torch.int64, device=self.device)
            self._list_records[key] = (stamp, records)
        tickets = self._list_tickets.get(lane)
        if tickets is None or tickets.numel() < records.shape[0]:
            tickets = torch.zeros(records.shape[0], dtype=torch.int32, device=self.device)
            self._list_tickets[lane] = tickets
        lib = self._lib
        count = records.shape[0]
        lead_pairs = min(lead // 2, count)
        if lead_pairs > 0:
            on = lead_on if lead_on is not None else stream
            blocks = self.lead_copy_blocks if self.lead_copy_blocks > 0 else self.list_blocks
            _lib.check("syn_copy_flag_list_async",
                       lib.syn_copy_flag_list_async(records.data_ptr(), lead_pairs, tickets.data_ptr(), blocks,
                                                    int(on.cuda_stream)))
            if lead_on is None:
                event = torch.cuda.Event()
                event.record(on)
                self._lead_events.append(event)
            # with lead_on the rest of the list does NOT wait for the leading chunks: both kernels start
            # together, the leading one with many workgroups in front of the compute kernel, the other with
            # few beside it.  Chunks then land in list order in practice (the leading kernel is an order of
            # magnitude faster) but not by construction; every chunk has its own flag, so a consumer does
            # not depend on the order.
        if count > lead_pairs:
            _lib.check("syn_copy_flag_list_async",
                       lib.syn_copy_flag_list_async(records.data_ptr() + 48 * lead_pairs, count - lead_pairs,
                                                    tickets.data_ptr() + 4 * lead_pairs, self.list_blocks,
                                                    int(stream.cuda_stream)))
        return True

    def wait_lead(self, stream: Optional[torch.cuda.Stream] = None) -> None:
        """`stream` continues once the leading ops of the last execute(lead_ops=...) are done."""
        stream = torch.cuda.current_stream(self.device) if stream is None else stream
        for event in getattr(self, "_lead_events", []):
            stream.wait_event(event)

    def execute_mesh(self, neglect_local: bool = False) -> None:
        """Enqueue EVERY rank's ops on this rank's first communication stream, in an order that
        respects each list and every flag wait (an op that waits for a flag is issued only after
        the op that writes it).  Plans in which a neighbour forwards what it has received itself
        (ring, double ring) only deliver this rank's data when the whole mesh is replayed; on one
        GPU that is one stream doing all the mesh's copies in turn.  Waits for another rank's
        COMPUTE_DONE flags are taken as satisfied (only this rank's compute kernel runs); this
        rank's own are real waits on the flags its kernel writes.  A library collective
        (CollectiveComm) is carried out once for the mesh, at the point where every rank's list
        has arrived at it."""
        if not self.streams:
            return
        stream = self.streams[0]
        handle = int(stream.cuda_stream)
        world = self.info.local_world_size
        lists = [(r, ops) for r in range(world) for ops in self.info.operations[r]]
        self._check_copy_units(ops for _, ops in lists)
        cursor = [0] * len(lists)
        written = set()                  # (signal type, rank, offset) already enqueued as a write
        for r in range(world):
            if r != self.rank and self.compute_signal_bufs:
                self.compute_signal_bufs[r].fill_(1)
        remaining = sum(len(ops) for _, ops in lists)
        # the k-th library collective of every list is one collective of the mesh: it is carried
        # out once, when every list that has a k-th collective has arrived at it
        nth = [0] * len(lists)                           # collectives passed, per list
        counts = [sum(isinstance(op, CollectiveComm) for op in ops) for _, ops in lists]
        arrived: Dict[int, Dict[int, CollectiveComm]] = {}
        done_collectives = set()
        while remaining:
            progressed = False
            for idx, (owner, ops) in enumerate(lists):
                while cursor[idx] < len(ops):
                    op = ops[cursor[idx]]
                    if isinstance(op, WaitIntraNodeSignal) and op.signal_type != SignalType.COMPUTE_DONE:
                        if (op.signal_type, op.rank % world, op.offset) not in written:
                            break            # its writer has not been enqueued yet
                    if isinstance(op, CollectiveComm):
                        k = nth[idx]
                        if k not in done_collectives:
                            here = arrived.setdefault(k, {})
                            if owner not in here:
                                here[owner] = op
                                progressed = True
                            if len(here) < sum(1 for c in counts if c > k):
                                break        # the other ranks have not reached it yet
                            self._mesh_collective(here, stream)
                            done_collectives.add(k)
                        nth[idx] += 1
                        cursor[idx] += 1
                        remaining -= 1
                        progressed = True
                        continue
                    self._issue(op, owner, stream, handle, neglect_local)
                    if isinstance(op, IntraNodeSignal):
                        written.add((op.signal_type, op.rank % world, op.offset))
                    cursor[idx] += 1
                    remaining -= 1
                    progressed = True
            if not progressed:
                raise RuntimeError("the op lists wait for flags nobody writes: the plan cannot be replayed")
        self._zero_stale_set()

    def _mesh_collective(self, per_rank: Dict[int, CollectiveComm], stream: torch.cuda.Stream) -> None:
        """One library collective of the simulated mesh, carried out on `stream` over the ranks'
        buffers of this process with the box copy / accumulate kernel (sums in rank order, one
        rounding in the element type per addition, the way a ring adds them up).  The reference
        hands these records to NCCL / NVSHMEM (communication_context.py:190-236), which needs one
        process per rank; here they exist so that plans with collectives replay end to end."""
        ranks = sorted(per_rank)
        first = per_rank[ranks[0]]
        for r in ranks:
            o = per_rank[r]
            if (o.op, o.src, o.dst, tuple(o.src_slice), tuple(o.dst_slice)) != \
                    (first.op, first.src, first.dst, tuple(first.src_slice), tuple(first.dst_slice)):
                raise ValueError(f"ranks disagree about a collective: {first} against {o}")
        world = self.info.local_world_size
        if ranks != list(range(world)):
            raise ValueError(f"collective {first} is issued by ranks {ranks} of {world}")
        units = self.info.num_copy_sms if self.info.num_copy_sms > 0 else 64
        src_idx = tuple(slice(ax.start, ax.end) for ax in first.src_slice)
        dst_idx = tuple(slice(ax.start, ax.end) for ax in first.dst_slice)
        srcs = [self.comm_buffers[first.src][r][src_idx] for r in ranks]
        dsts = [self.comm_buffers[first.dst][r][dst_idx] for r in ranks]

        def total_into(out: torch.Tensor, parts: List[torch.Tensor]) -> None:
            persistent_copy_last_contig(parts[0], out, num_sms=units, stream=stream)
            for part in parts[1:]:
                persistent_copy_last_contig(part, out, num_sms=units, reduce_op=ReduceOp.SUM, stream=stream,
                                            exclusive=True)

        if first.op == CollectiveOp.REDUCE_SCATTER:
            # the scattered axis: the one where the source is `world` times the destination
            axes = [a for a, (s, d) in enumerate(zip(srcs[0].shape, dsts[0].shape)) if s != d]
            if len(axes) != 1 or srcs[0].shape[axes[0]] != world * dsts[0].shape[axes[0]]:
                raise ValueError(f"{first}: source {tuple(srcs[0].shape)} is not {world} destination blocks "
                                 f"{tuple(dsts[0].shape)} along one axis")
            axis, width = axes[0], dsts[0].shape[axes[0]]
            for q in ranks:
                total_into(dsts[q], [s.narrow(axis, q * width, width) for s in srcs])
        elif first.op == CollectiveOp.ALL_REDUCE:
            if first.src != first.dst or src_idx != dst_idx:
                raise ValueError("the in-place all-reduce needs one buffer and one slice for source and result")
            with torch.cuda.stream(stream):
                total = torch.empty(srcs[0].shape, dtype=srcs[0].dtype, device=self.device)
            total_into(total, srcs)
            for q in ranks:
                persistent_copy_last_contig(total, dsts[q], num_sms=units, stream=stream)
        elif first.op == CollectiveOp.ALL_REDUCE_NVSHARP:
            if first.src == first.dst:
                raise ValueError("the two-buffer all-reduce needs different source and result buffers")
            total_into(dsts[0], srcs)
            for q in ranks[1:]:
                persistent_copy_last_contig(dsts[0], dsts[q], num_sms=units, stream=stream)
        else:
            raise NotImplementedError(f"collective {first.op} in the single-GPU executor")

    def _find_sole_writer_ops(self) -> set:
        """Accumulating box copies whose destination box nobody outside their own op list writes
        (the lists of every rank are known here).  One list is one stream, so such a box has one
        writer at a time and the sum need not be atomic: reduce-scatter by direct reduction in
        its pull form, where each rank adds its peers' chunks into its own result.  In the push
        form every rank adds into every other rank's result and the sums stay atomic."""
        writers = []          # (list key, buffer name, rank, box or None for a byte-range copy)
        for r, lists in enumerate(self.info.operations):
            for i, ops in enumerate(lists):
                for op in ops:
                    if isinstance(op, SMCopyOp):
                        box = tuple((ax.start, ax.end) for ax in op.dst_slice)
                        writers.append(((r, i), op.dst, op.dst_rank, box, op))
                    elif isinstance(op, CopyEngineOp):
                        writers.append(((r, i), op.dst, op.dst_rank, None, op))

        def overlap(a, b) -> bool:
            if a is None or b is None or len(a) != len(b):
                return True
            return all(lo1 < hi2 and lo2 < hi1 for (lo1, hi1), (lo2, hi2) in zip(a, b))

        sole = set()
        for key, name, rank, box, op in writers:
            if not isinstance(op, SMCopyOp) or op.reduce_op is None:
                continue
            if all(k == key or n != name or rk != rank or not overlap(box, bx)
                   for k, n, rk, bx, _ in writers):
                sole.add(id(op))
        return sole

    def _check_copy_units(self, op_lists) -> None:
        # before anything is enqueued (communication_context.py:164 asserts it per op)
        if self.info.num_copy_sms <= 0 and any(isinstance(op, SMCopyOp) for ops in op_lists for op in ops):
            raise ValueError("box copies run on compute units: set CommInfo.num_copy_sms first")

    def _issue_copy_with_flag(self, op: CopyEngineOp, flag_op: IntraNodeSignal, lane: int, handle: int,
                              neglect_local: bool, blocks: int) -> bool:
        """A copy and the flag write behind it as one kernel; False if the pair does not qualify
        (then both are issued on their own)."""
        world = self.info.local_world_size
        if op.src_rank == op.dst_rank and neglect_local:
            return False
        if flag_op.signal_type != SignalType.RECEIVE_DATA:
            return False
        src = self.comm_buffers[op.src][op.src_rank % world]
        dst = self.comm_buffers[op.dst][op.dst_rank % world]
        if op.src_offset + op.size > src.numel() * src.element_size() or \
                op.dst_offset + op.size > dst.numel() * dst.element_size():
            raise ValueError(f"{op} runs past the end of its buffer")
        dst_ptr, src_ptr = dst.data_ptr() + op.dst_offset, src.data_ptr() + op.src_offset
        if op.size <= 0 or op.size % 16 or dst_ptr % 16 or src_ptr % 16:
            return False
        flags = self.recv_signal_bufs[flag_op.rank % world]
        if not 0 <= flag_op.offset < flags.numel():
            raise ValueError(f"{flag_op} is outside the flag array")
        lib = self._lib
        if self.link_delay_us and op.src_rank != op.dst_rank:
            _lib.check("syn_delay_us", lib.syn_delay_us(self.link_delay_us, handle))
        _lib.check("syn_copy_flag_async",
                   lib.syn_copy_flag_async(dst_ptr, src_ptr, op.size, flags.data_ptr() + 8 * flag_op.offset, 1,
                                           self._tickets.data_ptr() + 4 * lane, blocks, handle))
        return True

    def _issue(self, op, owner: int, stream: torch.cuda.Stream, handle: int, neglect_local: bool) -> None:
        """Enqueue one op of rank `owner`'s list on `stream`."""
        lib = self._lib
        world = self.info.local_world_size
        if isinstance(op, CopyEngineOp):
            assert op.src_rank == owner or op.dst_rank == owner
            if op.src_rank == op.dst_rank and neglect_local:
                return
            src = self.comm_buffers[op.src][op.src_rank % world]
            dst = self.comm_buffers[op.dst][op.dst_rank % world]
            assert src.is_contiguous() and dst.is_contiguous()
            nbytes_src = src.numel() * src.element_size()
            nbytes_dst = dst.numel() * dst.element_size()
            if op.src_offset + op.size > nbytes_src or op.dst_offset + op.size > nbytes_dst:
                raise ValueError(f"{op} runs past the end of its buffer")
            if self.link_delay_us and op.src_rank != op.dst_rank:
                _lib.check("syn_delay_us", lib.syn_delay_us(self.link_delay_us, handle))
            dst_ptr, src_ptr = dst.data_ptr() + op.dst_offset, src.data_ptr() + op.src_offset
            kernel_ok = self.copy_blocks > 0 and not (op.size % 16 or dst_ptr % 16 or src_ptr % 16)
            if kernel_ok:
                _lib.check("syn_copy_kernel_async",
                           lib.syn_copy_kernel_async(dst_ptr, src_ptr, op.size, self.copy_blocks, handle))
            else:
                _lib.check("syn_copy_async", lib.syn_copy_async(dst_ptr, src_ptr, op.size, handle))
        elif isinstance(op, IntraNodeSignal):
            assert op.signal_type == SignalType.RECEIVE_DATA
            flags = self.recv_signal_bufs[op.rank % world]
            if not 0 <= op.offset < flags.numel():
                raise ValueError(f"{op} is outside the flag array")
            if self.flag_write_values and not torch.cuda.is_current_stream_capturing():
                _lib.check("syn_flag_write_value", lib.syn_flag_write_value(flags.data_ptr() + 8 * op.offset, 1, handle))
            else:
                _lib.check("syn_flag_set", lib.syn_flag_set(flags.data_ptr() + 8 * op.offset, 1, handle))
        elif isinstance(op, WaitIntraNodeSignal):
            flags = self._flags(op.signal_type, op.rank % world)
            if not 0 <= op.offset < flags.numel():
                raise ValueError(f"{op} is outside the flag array")
            _lib.check("syn_flag_wait",
                       lib.syn_flag_wait(flags.data_ptr() + 8 * op.offset, 1, self.wait_timeout_us,
                                         self.status.data_ptr(), handle))
        elif isinstance(op, SMCopyOp):
            assert op.src_rank == owner or op.dst_rank == owner
            if op.src_rank == op.dst_rank and neglect_local:
                return
            src = self.comm_buffers[op.src][op.src_rank % world]
            dst = self.comm_buffers[op.dst][op.dst_rank % world]
            src_box = src[tuple(slice(ax.start, ax.end) for ax in op.src_slice)]
            dst_box = dst[tuple(slice(ax.start, ax.end) for ax in op.dst_slice)]
            if op.reduce_op is not None and op.reduce_op != ReduceOp.SUM:
                raise NotImplementedError(f"reduce op {op.reduce_op} in a box copy")
            if self.link_delay_us and op.src_rank != op.dst_rank:
                _lib.check("syn_delay_us", lib.syn_delay_us(self.link_delay_us, handle))
            persistent_copy_last_contig(src_box, dst_box, num_sms=self.info.num_copy_sms,
                                        reduce_op=op.reduce_op, stream=stream,
                                        exclusive=id(op) in self._sole_writer_ops)
        elif isinstance(op, CollectiveComm):
            raise NotImplementedError(
                "a library collective involves every rank: replay the whole mesh with execute_mesh()")
        else:
            raise TypeError(f"unknown op record {type(op).__name__}")

    def check_status(self) -> None:
        """Synchronise and raise if a stream-side flag wait gave up."""
        torch.cuda.synchronize(self.device)
        words = self.status.tolist()
        if words[0] != 0:
            self.status.zero_()
            raise RuntimeError(f"communication stream flag wait timed out (status {words})")

    def get_comm_sms(self) -> int:
        return self.info.num_copy_sms

    def get_graph(self) -> torch.cuda.CUDAGraph:
        """Capture start_after / execute / end_before into a HIP graph.  The op list
        consists of memcpy nodes and small kernels only (no memset nodes).

        A graph holds the flag pointers of the set that is current at capture.  With two flag
        sets `reset_signals()` switches sets between iterations, and a replay would keep
        writing the first set while the kernels wait on the other: refused.  (Capture two
        iterations, reset_signals() included, into a graph of one's own instead.)"""
        if len(self._flag_sets) != 1:
            raise RuntimeError("get_graph() captures one flag set: not with flag_sets=2, where reset_signals() "
                               "alternates between two (capture two whole iterations instead)")
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.start_after(torch.cuda.current_stream(self.device))
            self.execute()
            self.end_before(torch.cuda.current_stream(self.device))
        return graph
