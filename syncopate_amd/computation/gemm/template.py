"""Launchers of the chunk-scheduled GEMM kernels (MI355X HIP, through the C ABI).

Same call surface as the reference's hand-written launchers
(syncopate/computation/gemm/template.py:162-220 `gemm_consumer`, :355-412
`gemm_producer`) and as the launcher its transform pass generates
(`gemm(a, b, c, world_size, num_sms, ..., cur_wave_sizes=, wave_offsets=,
signal_ptr=, signal_offsets=, [counter_ptr=], cum_tiles=)`,
syncopate/computation/transform/transformer.py:1139-1149).

B is stored [N, K] (K contiguous) as in the reference; wave sizes and offsets
are in elements.  Tables may be int32 tensors (GPU or CPU) or nested lists.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ... import _lib
from .._launch import (
    TableLike,
    already_checked,
    as_device_table,
    flag_buffer,
    host_copy,
    host_ptr,
    launches_on_stream,
    acquire_always,
    recall_note,
    remember_checked,
    remember_note,
    require_cuda,
    status_words,
    zeroed_int32,
)

from .tile_policy import choose_xcd_remap

DEFAULT_SPIN_TIMEOUT_US = 2_000_000


@launches_on_stream
def _launch(
    producer: bool,
    a: torch.Tensor,
    b: torch.Tensor,
    c: torch.Tensor,
    signal_buffer: torch.Tensor,
    cur_wave_size: TableLike,
    wave_offset: TableLike,
    signal_offsets: TableLike,
    num_gemm_sms: int,
    BLOCK_SIZE_M: int,
    BLOCK_SIZE_N: int,
    BLOCK_SIZE_K: int,
    GROUP_SIZE_M: int,
    cum_tiles: int,
    counter_buffer: Optional[torch.Tensor],
    visit_log: Optional[torch.Tensor],
    xcd_remap: Optional[bool],
    eight_waves: bool,
    ring_pipe: bool,
    k_stagger: bool,
    two_stage: bool,
    spin_timeout_us: int,
    stream: Optional[torch.cuda.Stream],
    wait_signal_buffer: Optional[torch.Tensor] = None,
    wait_signal_offsets: Optional[TableLike] = None,
    mfma_32x32: bool = False,
) -> None:
    # shape/dtype contract of the reference launchers (template.py:177-185)
    assert a.shape[1] == b.shape[1], "Incompatible dimensions"  # b is [N, K]
    assert a.dtype == b.dtype, "Incompatible dtypes"
    if c.dtype != a.dtype:
        raise TypeError("c must have the element type of a and b")
    dev = require_cuda(a, b, c, signal_buffer)
    if not (a.is_contiguous() and b.is_contiguous() and c.is_contiguous()):
        raise ValueError("a, b and c must be contiguous row-major tensors")
    M, K = a.shape
    N = b.shape[0]
    if tuple(c.shape) != (M, N):
        raise ValueError(f"c must be ({M}, {N}), got {tuple(c.shape)}")
    flags = flag_buffer(signal_buffer)

    sizes = as_device_table(cur_wave_size, dev, 2)
    offsets = as_device_table(wave_offset, dev, 2)
    signals = as_device_table(signal_offsets, dev, None)
    num_waves = signals.numel()
    if sizes.shape[0] != num_waves or offsets.shape[0] != num_waves:
        raise ValueError("wave size, offset and signal tables disagree on the number of waves")

    lib = _lib.load()
    tables = (cur_wave_size, wave_offset, signal_offsets)   # the caller's objects, not our views
    params = (M, N, K, BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, int(cum_tiles), flags.numel())
    caller_owned = all(isinstance(t, torch.Tensor) and t.is_cuda
                       for t in (cur_wave_size, wave_offset, signal_offsets))
    if not (caller_owned and already_checked(tables, params)):
        hs, ho, hg = host_copy(sizes), host_copy(offsets), host_copy(signals)
        _lib.check(
            "syn_gemm_check_waves",
            lib.syn_gemm_check_waves(host_ptr(hs), host_ptr(ho), host_ptr(hg), num_waves, M, N, K,
                                     BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, int(cum_tiles),
                                     flags.numel()),
        )
        if caller_owned:
            remember_checked(tables, params)

    wait_flags = wait_sigs = None
    if (wait_signal_buffer is None) != (wait_signal_offsets is None):
        raise ValueError("the flags to wait for and their per-wave indices come together")
    if wait_signal_buffer is not None:
        if not producer:
            raise ValueError("a consumer waits on its signal buffer: a second flag array is for a producer that also waits")
        wait_flags = flag_buffer(wait_signal_buffer)
        wait_sigs = as_device_table(wait_signal_offsets, dev, None)
        if wait_sigs.numel() != num_waves:
            raise ValueError("one index to wait for per wave (-1: none)")
        # read back once per table object: a device-to-host copy per launch would wait for the stream to drain
        owned = isinstance(wait_signal_offsets, torch.Tensor) and wait_signal_offsets.is_cuda
        note = f"indices to wait for, {wait_flags.numel()} flags"
        if not (owned and recall_note([wait_signal_offsets], note)):
            hw = host_copy(wait_sigs)
            if int(hw.min()) < -1 or int(hw.max()) >= wait_flags.numel():
                raise ValueError("an index to wait for is outside its flag array")
            if owned:
                remember_note([wait_signal_offsets], note, True)

    if producer:
        if counter_buffer is None:
            # equal to the number of waves (template.py:388)
            counter_buffer = zeroed_int32((num_waves,), dev)
        elif counter_buffer.dtype != torch.int32 or counter_buffer.numel() < num_waves:
            raise ValueError("counter buffer must be int32 with one word per wave")

    grid_tiles = lib.syn_gemm_grid(int(cum_tiles), M, N, BLOCK_SIZE_M, BLOCK_SIZE_N, num_gemm_sms)
    if grid_tiles <= 0:
        raise _lib.SyncopateHipError("syn_gemm_grid", grid_tiles)
    if visit_log is not None:
        tiles = (int(cum_tiles) if cum_tiles else M * N) // (BLOCK_SIZE_M * BLOCK_SIZE_N)
        if visit_log.dtype != torch.int32 or visit_log.numel() < 4 * tiles or not visit_log.is_contiguous():
            raise ValueError(f"visit_log must be a contiguous int32 tensor of at least {4 * tiles} words")

    if xcd_remap is None:
        xcd_remap = choose_xcd_remap(BLOCK_SIZE_M, BLOCK_SIZE_N)
    desc = _lib.GemmDesc(
        a=a.data_ptr(),
        b=b.data_ptr(),
        c=c.data_ptr(),
        flags=flags.data_ptr(),
        wave_sizes=sizes.data_ptr(),
        wave_offsets=offsets.data_ptr(),
        signal_offsets=signals.data_ptr(),
        counters=None if counter_buffer is None else counter_buffer.data_ptr(),
        visit_log=None if visit_log is None else visit_log.data_ptr(),
        status=status_words(dev).data_ptr(),
        num_waves=num_waves,
        M=M,
        N=N,
        K=K,
        dtype=_lib.dtype_code(a.dtype),
        block_m=BLOCK_SIZE_M,
        block_n=BLOCK_SIZE_N,
        block_k=BLOCK_SIZE_K,
        group_m=GROUP_SIZE_M,
        num_sms=num_gemm_sms,
        cum_tiles=int(cum_tiles),
        spin_timeout_us=int(spin_timeout_us),
        options=(_lib.SYN_GEMM_XCD_REMAP if xcd_remap else 0) | (_lib.SYN_GEMM_EIGHT_WAVES if eight_waves else 0)
        | (_lib.SYN_GEMM_RING_PIPE if ring_pipe else 0) | (0 if k_stagger else _lib.SYN_GEMM_NO_K_STAGGER)
        | (_lib.SYN_GEMM_TWO_STAGE if two_stage else 0) | (_lib.SYN_GEMM_MFMA_32X32 if mfma_32x32 else 0)
        | (_lib.SYN_GEMM_ACQUIRE_ALWAYS
           if acquire_always(wait_signal_buffer if wait_signal_buffer is not None else signal_buffer) else 0),
    )
    with torch.cuda.device(dev):
        if wait_flags is not None:
            _lib.check("syn_gemm_consumer_producer",
                       lib.syn_gemm_consumer_producer(ctypes.byref(desc), wait_flags.data_ptr(), wait_sigs.data_ptr(),
                                                      _lib.stream_handle(stream)))
            return
        fn = lib.syn_gemm_producer if producer else lib.syn_gemm_consumer
        name = "syn_gemm_producer" if producer else "syn_gemm_consumer"
        _lib.check(name, fn(ctypes.byref(desc), _lib.stream_handle(stream)))


def gemm_consumer(
    a,
    b,
    c,
    signal_buffer,
    cur_wave_size,
    wave_offset,
    signal_offsets,
    world_size,
    num_gemm_sms,
    BLOCK_SIZE_M=128,
    BLOCK_SIZE_N=256,
    BLOCK_SIZE_K=64,
    GROUP_SIZE_M=8,
    STAGES=3,
    *,
    cum_tiles=0,
    visit_log=None,
    xcd_remap=None,
    eight_waves=False,
    ring_pipe=False,
    k_stagger=True,
    two_stage=False,
    mfma_32x32=False,
    spin_timeout_us=DEFAULT_SPIN_TIMEOUT_US,
    stream=None,
):
    """AG+GEMM consumer: c = a @ b.T, tiles of c visited in wave order, each wave
    gated by its flag word (reference: template.py:162-220).

    `STAGES` is accepted for call compatibility; the HIP kernel is double
    buffered.  `visit_log` (int32 [tiles, 4]) receives, per tile id,
    (program id, wave, pid_m, pid_n).
    """
    M = a.shape[0]
    M_per_rank = M // world_size
    assert M_per_rank % BLOCK_SIZE_M == 0
    _launch(False, a, b, c, signal_buffer, cur_wave_size, wave_offset, signal_offsets, num_gemm_sms,
            BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, GROUP_SIZE_M, cum_tiles, None, visit_log,
            xcd_remap, eight_waves, ring_pipe, k_stagger, two_stage, spin_timeout_us, stream, mfma_32x32=mfma_32x32)


def gemm_producer(
    a,
    b,
    c,
    signal_buffer,
    cur_wave_size,
    wave_offset,
    signal_offsets,
    num_gemm_sms,
    BLOCK_SIZE_M=128,
    BLOCK_SIZE_N=256,
    BLOCK_SIZE_K=64,
    GROUP_SIZE_M=8,
    STAGES=3,
    *,
    cum_tiles=0,
    counter_buffer=None,
    visit_log=None,
    xcd_remap=None,
    eight_waves=False,
    ring_pipe=False,
    k_stagger=True,
    two_stage=False,
    mfma_32x32=False,
    stream=None,
):
    """GEMM+RS producer: same GEMM; every finished tile bumps its wave's counter
    and the last tile of a wave sets the wave's flag to 1 (reference:
    template.py:355-412).  Without `counter_buffer` a zeroed one is allocated
    per call, as the reference does.
    """
    _launch(True, a, b, c, signal_buffer, cur_wave_size, wave_offset, signal_offsets, num_gemm_sms,
            BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, GROUP_SIZE_M, cum_tiles, counter_buffer,
            visit_log, xcd_remap, eight_waves, ring_pipe, k_stagger, two_stage, DEFAULT_SPIN_TIMEOUT_US, stream,
            mfma_32x32=mfma_32x32)


def gemm(
    a,
    b,
    c,
    world_size,
    num_gemm_sms,
    BLOCK_SIZE_M=128,
    BLOCK_SIZE_N=256,
    BLOCK_SIZE_K=64,
    GROUP_SIZE_M=8,
    STAGES=3,
    *,
    cur_wave_sizes,
    wave_offsets,
    signal_ptr,
    signal_offsets,
    counter_ptr=None,
    consumer_signal_ptr=None,
    consumer_signal_offsets=None,
    cum_tiles=0,
    visit_log=None,
    xcd_remap=None,
    eight_waves=False,
    ring_pipe=False,
    k_stagger=True,
    two_stage=False,
    mfma_32x32=False,
    spin_timeout_us=DEFAULT_SPIN_TIMEOUT_US,
    stream=None,
):
    """Call form of the launcher the reference's transform pass emits for the
    annotated persistent GEMM (tests/computation/transform/examples/
    example_persistent_gemm.py:125-181; extra arguments transformer.py:1139-1149):
    a consumer when `counter_ptr` is None, a producer otherwise.  A producer given
    `consumer_signal_ptr` and `consumer_signal_offsets` (one index per wave, -1: none) is a
    consumer as well: it waits for those flags wave by wave and sets `signal_ptr`'s - both
    passes of the transform applied to one kernel.
    """
    _launch(counter_ptr is not None, a, b, c, signal_ptr, cur_wave_sizes, wave_offsets, signal_offsets,
            num_gemm_sms, BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, GROUP_SIZE_M, cum_tiles,
            counter_ptr, visit_log, xcd_remap, eight_waves, ring_pipe, k_stagger, two_stage, spin_timeout_us, stream,
            consumer_signal_ptr, consumer_signal_offsets, mfma_32x32=mfma_32x32)
