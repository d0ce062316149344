"""Launchers of the GEMM forms that bind an operand to a peer per wave (MI355X HIP, C ABI).

* ``gemm_ag_direct_read`` — the GEMM reads the A rows of every wave straight from the shard of
  the rank that owns them instead of from a gathered buffer
  (syncopate/computation/gemm/template_ag.py:43-187, launcher :190-260).
* ``gemm_rs_producer_persistent`` — the C tile of every wave is atomically added into the
  [M / W, N] result of the rank that owns those rows
  (syncopate/computation/gemm/template_rs.py:37-209, launcher :212-290).
* ``gemm_remote`` — the call form the transform pass generates for a descriptor with a
  RemoteBinding: ``target_rank`` and ``dst_offsets`` per wave, store or atomic add
  (syncopate/computation/transform/transformer.py:1158-1178; use in
  tests/test_gemm_rs_direct_reduce.py:166-189).

The reference resolves a peer's buffer with ``dl.symm_at(ptr, rank)`` on an NVSHMEM heap.  Here
the caller passes the peers' buffers themselves (``a`` / ``c`` as a list with one tensor per
rank): on one MI355X they are tensors of the same process, on a node they would be peer-mapped
allocations.  Everything else (tables in elements, B stored [N, K]) is as in ``template.py``.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from ... import _lib
from .._launch import (TableLike, acquire_always, as_device_table, host_copy, host_ptr, launches_on_stream, recall_note,
                       remember_note, require_cuda, status_words)

_pointer_tables: dict = {}


def _pointer_table(tensors: Sequence[torch.Tensor], dev: torch.device) -> torch.Tensor:
    """Device array of the tensors' addresses (kept per set of addresses: a launch must not
    allocate in steady state)."""
    key = (dev.index, tuple(t.data_ptr() for t in tensors))
    table = _pointer_tables.get(key)
    if table is None:
        if len(_pointer_tables) > 64:
            _pointer_tables.clear()
        table = torch.tensor(list(key[1]), dtype=torch.int64, device=dev)
        _pointer_tables[key] = table
    return table


def _check_ranks(name: str, ranks: torch.Tensor, count: int, num_waves: int) -> None:
    host = host_copy(ranks)
    if host.numel() < num_waves:
        raise ValueError(f"{name} is shorter than the wave tables")
    if int(host[:num_waves].min()) < 0 or int(host[:num_waves].max()) >= count:
        raise ValueError(f"{name} names a rank outside 0..{count - 1}")


@launches_on_stream
def _prepare_binding(lib, sizes, offsets, signals, flags, num_waves, M, N, K, block_m, block_n, block_k, cum_tiles,
                     a_list, a_target_rank, c_list, target_rank, dst_offsets, atomic_add, k_ranges, dev):
    """The host's share of a bound launch: table checks, and the device tables the kernel reads (pointer tables,
    ranks, destination offsets, k ranges).  Returns the fields of the remote descriptor and the tensors they point into."""
    hs, ho, hg = host_copy(sizes), host_copy(offsets), host_copy(signals)
    _lib.check("syn_gemm_check_waves",
               lib.syn_gemm_check_waves(host_ptr(hs), host_ptr(ho), host_ptr(hg), num_waves, M, N, K,
                                        block_m, block_n, block_k, int(cum_tiles), flags.numel()))
    fields, keep = {}, []
    if a_list is not None:
        if a_target_rank is None:
            raise ValueError("a list of A shards needs a_target_rank")
        a_ranks = as_device_table(a_target_rank, dev, None)
        _check_ranks("a_target_rank", a_ranks, len(a_list), num_waves)
        shard_rows = min(t.shape[0] for t in a_list)
        if int(hs[:, 0].max()) > shard_rows:
            raise ValueError("a wave has more rows than an A shard")
        table = _pointer_table(a_list, dev)
        keep += [a_ranks, table]
        fields.update(a_peers=table.data_ptr(), a_target_rank=a_ranks.data_ptr())
    if c_list is not None:
        if target_rank is None or dst_offsets is None:
            raise ValueError("a list of C buffers needs target_rank and dst_offsets")
        c_ranks = as_device_table(target_rank, dev, None)
        dst = as_device_table(dst_offsets, dev, 2)
        _check_ranks("target_rank", c_ranks, len(c_list), num_waves)
        ldc = c_list[0].shape[1]
        rows = min(t.shape[0] for t in c_list)
        if any(t.shape[1] != ldc for t in c_list) or ldc % 4:
            raise ValueError("peer C buffers must share one row length, a multiple of 4")
        hd = host_copy(dst)
        if dst.shape[0] < num_waves or int(hd.min()) < 0:
            raise ValueError("dst_offsets must hold one non-negative (row, col) pair per wave")
        if int((hd[:num_waves, 0] + hs[:, 0]).max()) > rows or int((hd[:num_waves, 1] + hs[:, 1]).max()) > ldc:
            raise ValueError("a wave's destination region does not fit the peer C buffer")
        if int(hd[:num_waves, 1].max()) % 4:
            raise ValueError("dst column offsets must be multiples of 4 elements")
        table = _pointer_table(c_list, dev)
        keep += [c_ranks, dst, table]
        fields.update(c_peers=table.data_ptr(), c_target_rank=c_ranks.data_ptr(), c_dst_offsets=dst.data_ptr(), c_ld=ldc,
                      c_atomic_add=1 if atomic_add else 0)
    elif atomic_add:
        raise ValueError("atomic_add needs c bound to peers")
    if k_ranges is not None:
        if c_list is None or not atomic_add:
            raise ValueError("k_ranges produce partial products: c must be bound and added into (atomic_add)")
        ranges = as_device_table(k_ranges, dev, 2)
        hk = host_copy(ranges)
        if ranges.shape[0] < num_waves:
            raise ValueError("k_ranges is shorter than the wave tables")
        k0, kn = hk[:num_waves, 0], hk[:num_waves, 1]
        if int(k0.min()) < 0 or int(kn.min()) <= 0 or int((k0 % 64).max()) or int((kn % 64).max()):
            raise ValueError("k ranges must start at and span positive multiples of 64")
        if int((k0 + kn).max()) > K:
            raise ValueError("a k range runs past K")
        keep.append(ranges)
        fields["k_ranges"] = ranges.data_ptr()
    return fields, keep


def gemm_remote(
    a,
    b: torch.Tensor,
    c,
    num_gemm_sms: int,
    BLOCK_SIZE_M: int = 128,
    BLOCK_SIZE_N: int = 256,
    BLOCK_SIZE_K: int = 64,
    GROUP_SIZE_M: int = 8,
    STAGES: int = 3,
    *,
    cur_wave_sizes: TableLike,
    wave_offsets: TableLike,
    M: int,
    a_target_rank: Optional[TableLike] = None,
    target_rank: Optional[TableLike] = None,
    dst_offsets: Optional[TableLike] = None,
    atomic_add: bool = False,
    k_ranges: Optional[TableLike] = None,
    signal_ptr: Optional[torch.Tensor] = None,
    signal_offsets: Optional[TableLike] = None,
    cum_tiles: int = 0,
    visit_log: Optional[torch.Tensor] = None,
    xcd_remap: bool = True,
    eight_waves: bool = False,
    stream: Optional[torch.cuda.Stream] = None,
) -> None:
    """C = A @ B.T over an [M, N] tile space walked in wave order, with per-wave peer bindings.

    `a` is a tensor [M, K], or a list of per-rank shards [rows, K] together with
    `a_target_rank` (then the A rows of wave w are rows `tile row inside the wave` of shard
    a_target_rank[w]).  `c` is a tensor [M, N], or a list of per-rank buffers [rows, ldc]
    together with `target_rank` and `dst_offsets` ([num_waves, 2] element offsets of the wave's
    region in the peer buffer); `atomic_add` adds instead of storing.  `k_ranges` ([num_waves, 2]:
    first k and count, multiples of 64) makes a wave contract over part of K only; its partial
    product has to be added (`atomic_add`) into a C that starts at zero.
    """
    a_list = list(a) if isinstance(a, (list, tuple)) else None
    c_list = list(c) if isinstance(c, (list, tuple)) else None
    if a_list is None and c_list is None:
        raise ValueError("neither a nor c is bound to peers: use gemm / gemm_consumer")
    first_a = a_list[0] if a_list is not None else a
    first_c = c_list[0] if c_list is not None else c
    dev = require_cuda(first_a, b, first_c)
    K, N = b.shape[1], b.shape[0]
    for t in (a_list or [a]):
        if t.dim() != 2 or t.shape[1] != K or t.dtype != b.dtype or not t.is_contiguous() or t.device != dev:
            raise ValueError("every A operand must be a contiguous [rows, K] tensor of b's type and device")
    for t in (c_list or [c]):
        if t.dim() != 2 or t.dtype != b.dtype or not t.is_contiguous() or t.device != dev:
            raise ValueError("every C operand must be a contiguous 2-D tensor of b's type and device")
    if not b.is_contiguous():
        raise ValueError("b must be contiguous [N, K]")
    if a_list is None and tuple(a.shape) != (M, K):
        raise ValueError(f"a must be ({M}, {K})")
    if c_list is None and tuple(c.shape) != (M, N):
        raise ValueError(f"c must be ({M}, {N})")

    sizes = as_device_table(cur_wave_sizes, dev, 2)
    offsets = as_device_table(wave_offsets, dev, 2)
    num_waves = sizes.shape[0]
    if offsets.shape[0] != num_waves:
        raise ValueError("wave size and offset tables disagree on the number of waves")
    if signal_offsets is None:
        signals = torch.full((num_waves,), -1, dtype=torch.int32, device=dev)
        flags = torch.zeros((1,), dtype=torch.int64, device=dev) if signal_ptr is None else signal_ptr
    else:
        if signal_ptr is None:
            raise ValueError("signal_offsets without signal_ptr")
        signals = as_device_table(signal_offsets, dev, None)
        flags = signal_ptr

    lib = _lib.load()
    # What the host works out from the tables - the checks, the pointer tables, the converted rank and offset
    # tables - is kept with the caller's device tables (per tensor objects and versions), so that a launch repeated
    # on the same operands costs no device-to-host copy.
    given = [t for t in (cur_wave_sizes, wave_offsets, signal_offsets, a_target_rank, target_rank, dst_offsets, k_ranges)
             if t is not None]
    caller_owned = all(isinstance(t, torch.Tensor) and t.is_cuda for t in given)
    params = (M, N, K, BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, int(cum_tiles), flags.numel(), bool(atomic_add),
              None if a_list is None else tuple((t.data_ptr(), t.shape[0]) for t in a_list),
              None if c_list is None else tuple((t.data_ptr(), tuple(t.shape)) for t in c_list))
    prepared = recall_note(given, "remote binding") if caller_owned else None
    if prepared is None or prepared[0] != params:
        prepared = (params, _prepare_binding(lib, sizes, offsets, signals, flags, num_waves, M, N, K, BLOCK_SIZE_M, BLOCK_SIZE_N,
                                             BLOCK_SIZE_K, cum_tiles, a_list, a_target_rank, c_list, target_rank, dst_offsets,
                                             atomic_add, k_ranges, dev))
        if caller_owned:
            remember_note(given, "remote binding", prepared)
    fields, keep = prepared[1]
    remote = _lib.GemmRemote()
    for name, value in fields.items():
        setattr(remote, name, value)

    if visit_log is not None:
        tiles = (int(cum_tiles) if cum_tiles else M * N) // (BLOCK_SIZE_M * BLOCK_SIZE_N)
        if visit_log.dtype != torch.int32 or visit_log.numel() < 4 * tiles or not visit_log.is_contiguous():
            raise ValueError(f"visit_log must be a contiguous int32 tensor of at least {4 * tiles} words")
    desc = _lib.GemmDesc(
        a=None if a_list is not None else a.data_ptr(), b=b.data_ptr(),
        c=None if c_list is not None else c.data_ptr(), flags=flags.data_ptr(),
        wave_sizes=sizes.data_ptr(), wave_offsets=offsets.data_ptr(), signal_offsets=signals.data_ptr(),
        counters=None, visit_log=None if visit_log is None else visit_log.data_ptr(),
        status=status_words(dev).data_ptr(), num_waves=num_waves, M=M, N=N, K=K,
        dtype=_lib.dtype_code(b.dtype), block_m=BLOCK_SIZE_M, block_n=BLOCK_SIZE_N, block_k=BLOCK_SIZE_K,
        group_m=GROUP_SIZE_M, num_sms=num_gemm_sms, cum_tiles=int(cum_tiles), spin_timeout_us=0,
        options=(_lib.SYN_GEMM_XCD_REMAP if xcd_remap else 0) | (_lib.SYN_GEMM_EIGHT_WAVES if eight_waves else 0)
        | (_lib.SYN_GEMM_ACQUIRE_ALWAYS if signal_ptr is not None and acquire_always(signal_ptr) else 0),
    )
    with torch.cuda.device(dev):
        _lib.check("syn_gemm_remote_binding",
                   lib.syn_gemm_remote_binding(ctypes.byref(desc), ctypes.byref(remote), _lib.stream_handle(stream)))
    del keep, prepared


def gemm_ag_direct_read(
    a,
    b,
    c,
    cur_wave_size,
    wave_offset,
    target_rank,
    world_size,
    local_world_size,
    num_gemm_sms,
    use_a_tma: bool = True,
    BLOCK_SIZE_M=128,
    BLOCK_SIZE_N=256,
    BLOCK_SIZE_K=64,
    GROUP_SIZE_M=8,
    STAGES=3,
    **kwargs,
):
    """AG+GEMM without a gathered buffer: `a` is the list of the ranks' [M / W, K] shards
    (index = rank); wave w reads shard target_rank[w]; c is the local [M, N] result
    (reference: template_ag.py:190-260).  `use_a_tma` is accepted and ignored."""
    shards = list(a)
    if len(shards) != world_size:
        raise ValueError("a must list one shard per rank")
    local_m = shards[0].shape[0]
    assert local_m * world_size == c.shape[0], (
        f"c must hold gathered rows (expected {local_m * world_size}, got {c.shape[0]})")
    assert c.shape[1] == b.shape[0]
    gemm_remote(shards, b, c, num_gemm_sms, BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, GROUP_SIZE_M, STAGES,
                cur_wave_sizes=cur_wave_size, wave_offsets=wave_offset, M=local_m * world_size,
                a_target_rank=target_rank, cum_tiles=c.shape[0] * c.shape[1], **kwargs)


def gemm_rs_producer_persistent(
    a,
    b,
    c,
    cur_wave_size,
    wave_offset,
    target_rank,
    world_size,
    local_world_size,
    num_gemm_sms,
    BLOCK_SIZE_M=128,
    BLOCK_SIZE_N=256,
    BLOCK_SIZE_K=64,
    GROUP_SIZE_M=8,
    STAGES=3,
    use_c_tma: bool = True,
    **kwargs,
):
    """GEMM+RS by remote atomics: a [M, K_local], b [N, K_local]; `c` is the list of the ranks'
    [M / W, N] results (index = rank), zeroed by the caller's side of the collective; the tile of
    wave w is added into c[target_rank[w]] at its wave-local row (reference:
    template_rs.py:212-290; unlike it this launcher neither zeroes c nor barriers: on one GPU
    the caller launches every rank's kernel in turn on one stream)."""
    bufs = list(c)
    if len(bufs) != world_size:
        raise ValueError("c must list one buffer per rank")
    m = a.shape[0]
    m_per_rank = m // world_size
    assert m_per_rank % BLOCK_SIZE_M == 0
    # rows are wave-local in the owner's buffer, columns keep their global position
    # (template_rs.py:157-166: offs_cm from the wave-local pid_m, offs_bn from the global pid_n)
    owned = isinstance(wave_offset, torch.Tensor) and wave_offset.is_cuda
    dst = recall_note([wave_offset], "owner slot offsets") if owned else None
    if dst is None:
        dst = as_device_table(wave_offset, a.device, 2).clone()
        dst[:, 0] = 0
        if owned:
            remember_note([wave_offset], "owner slot offsets", dst)      # the same tensor next time: gemm_remote's notes hold
    gemm_remote(a, b, bufs, num_gemm_sms, BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, GROUP_SIZE_M, STAGES,
                cur_wave_sizes=cur_wave_size, wave_offsets=wave_offset, M=m, target_rank=target_rank,
                dst_offsets=dst, atomic_add=True, cum_tiles=m * b.shape[0], **kwargs)


def gemm_splitk(
    a: torch.Tensor,
    b: torch.Tensor,
    c: torch.Tensor,
    world_size: int,
    num_gemm_sms: int,
    BLOCK_SIZE_M: int = 128,
    BLOCK_SIZE_N: int = 256,
    BLOCK_SIZE_K: int = 64,
    GROUP_SIZE_M: int = 8,
    STAGES: int = 3,
    *,
    cur_wave_sizes: TableLike,
    wave_offsets: TableLike,
    signal_ptr: Optional[torch.Tensor] = None,
    signal_offsets: Optional[TableLike] = None,
    cum_tiles: int = 0,
    **kwargs,
) -> None:
    """c += a @ b.T, wave by wave, where a wave is a box [rows, cols, k count] at [row, col, first k]
    of the (M, N, K) iteration space: the call form of the reference's transformed split-K GEMM
    (tests/computation/transform/examples/example_splitk_gemm.py:117-175, called with three-column
    tables at tests/test_all2all_gemm.py:142-160 and tests/test_gemm_all2all_gemm.py:183-196).
    Each (tile, wave) pair is one work item whose partial product is atomically added into `c`,
    which the caller zeroes; a wave with a flag is waited for before its part of A is read."""
    dev = require_cuda(a, b, c)
    sizes3 = as_device_table(cur_wave_sizes, dev, 3)
    offsets3 = as_device_table(wave_offsets, dev, 3)
    num_waves = sizes3.shape[0]
    if offsets3.shape[0] != num_waves:
        raise ValueError("wave size and offset tables disagree on the number of waves")
    # the two-column tables gemm_remote takes, kept with the caller's three-column ones (so that its notes hold too)
    owned = all(isinstance(t, torch.Tensor) and t.is_cuda for t in (cur_wave_sizes, wave_offsets))
    split = recall_note([cur_wave_sizes, wave_offsets], "split-k tables") if owned else None
    if split is None:
        split = (sizes3[:, :2].contiguous(), offsets3[:, :2].contiguous(),
                 torch.zeros(num_waves, dtype=torch.int32, device=dev),
                 torch.stack([offsets3[:, 2], sizes3[:, 2]], dim=1).contiguous())
        if owned:
            remember_note([cur_wave_sizes, wave_offsets], "split-k tables", split)
    sizes2, offsets2, ranks, k_ranges = split
    gemm_remote(a, b, [c], num_gemm_sms, BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, GROUP_SIZE_M, STAGES,
                cur_wave_sizes=sizes2, wave_offsets=offsets2, M=a.shape[0], target_rank=ranks, dst_offsets=offsets2,
                atomic_add=True, k_ranges=k_ranges, signal_ptr=signal_ptr, signal_offsets=signal_offsets,
                cum_tiles=cum_tiles, **kwargs)
