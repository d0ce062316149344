"""Helpers shared by the kernel launchers: status words, wave-table checks, pointers."""

from __future__ import annotations

import ctypes
import functools
import inspect
import weakref
from typing import Dict, Optional, Sequence, Tuple, Union

import torch

from .. import _lib

TableLike = Union[torch.Tensor, Sequence]

# One int32[SYN_STATUS_WORDS] block per device.  A kernel whose flag wait times
# out records (code, wave, program id, signal offset) here and exits.
_status: Dict[int, torch.Tensor] = {}


def status_words(device: torch.device) -> torch.Tensor:
    idx = device.index if device.index is not None else torch.cuda.current_device()
    buf = _status.get(idx)
    if buf is None:
        buf = torch.zeros(_lib.SYN_STATUS_WORDS, dtype=torch.int32, device=torch.device("cuda", idx))
        _status[idx] = buf
    return buf


class FlagWaitTimeout(RuntimeError):
    """A kernel gave up spinning on a flag word that was never set."""


def check_status(device: Optional[torch.device] = None, *, reset: bool = True) -> None:
    """Synchronise `device` and raise if a kernel reported a flag-wait time-out."""
    devices = list(_status) if device is None else [
        device.index if device.index is not None else torch.cuda.current_device()
    ]
    for idx in devices:
        buf = _status.get(idx)
        if buf is None:
            continue
        torch.cuda.synchronize(idx)
        words = buf.tolist()
        if words[0] != 0:
            if reset:
                buf.zero_()
            if words[0] == _lib.SYN_STATUS_SPIN_TIMEOUT:
                raise FlagWaitTimeout(
                    f"flag wait timed out on cuda:{idx}: wave {words[1]}, program {words[2]}, "
                    f"signal offset {words[3]}"
                )
            raise RuntimeError(f"kernel status {words} on cuda:{idx}")


_ZERO_POOLS: dict = {}
ZERO_POOL_SLICES = 16


def zeroed_int32(shape, device: torch.device) -> torch.Tensor:
    """A zero-filled int32 work area for ONE launch on torch's current stream (locks, counters).

    The areas come out of a pool per (device, stream, shape) that one fill kernel zeroes sixteen launches at a
    time: the fill of a pool is ordered on the stream behind the launches that used its areas and in front of
    the launches that will, so every launch still finds zeros, and fifteen of sixteen launches are not preceded
    by a fill kernel of their own (on a 0.26 ms attention launch that kernel and the gap behind it are 2-3 %).
    While the stream is being captured into a graph every call gets a fresh `torch.zeros`: a replayed graph
    must carry its own fill."""
    shape = tuple(int(x) for x in shape)
    if torch.cuda.is_current_stream_capturing():
        return torch.zeros(shape, dtype=torch.int32, device=device)
    key = (device.index, torch.cuda.current_stream(device).cuda_stream, shape)
    pool = _ZERO_POOLS.get(key)
    if pool is None:
        if len(_ZERO_POOLS) > 64:
            _ZERO_POOLS.clear()       # (the allocator hands a dropped pool's memory on in stream order)
        pool = _ZERO_POOLS[key] = [torch.zeros((ZERO_POOL_SLICES,) + shape, dtype=torch.int32, device=device), 0]
    elif pool[1] >= ZERO_POOL_SLICES:
        pool[0].zero_()
        pool[1] = 0
    area = pool[0][pool[1]]
    pool[1] += 1
    return area


def launches_on_stream(fn):
    """Decorator of a launcher with a `stream` argument: the whole call - wave tables built
    from lists or CPU tensors, zeroed counters, locks, outputs, and the kernel launch - runs
    with `stream` as torch's current stream.  The temporaries' fills are then ordered in front
    of the kernel, and the caching allocator hands their memory on only behind it."""
    sig = inspect.signature(fn)

    @functools.wraps(fn)
    def wrapper(*args, **kwargs):
        bound = sig.bind(*args, **kwargs)
        stream = bound.arguments.get("stream")
        if stream is None:
            return fn(*args, **kwargs)
        with torch.cuda.stream(stream):
            return fn(*args, **kwargs)

    return wrapper


def as_device_table(table: TableLike, device: torch.device, width: Optional[int]) -> torch.Tensor:
    """int32, contiguous, on `device`; `width` = row length (None for 1-D tables)."""
    if isinstance(table, torch.Tensor):
        t = table
        if t.dtype != torch.int32:
            raise TypeError(f"wave tables must be int32, got {t.dtype}")
        if t.device != device:
            t = t.to(device)
    else:
        t = torch.tensor(table, dtype=torch.int32, device=device)
    t = t.contiguous()
    if width is None:
        if t.dim() != 1:
            raise ValueError(f"expected a 1-D table, got shape {tuple(t.shape)}")
    else:
        if t.numel() % width:
            raise ValueError(f"table of {t.numel()} entries is not rows of {width}")
        t = t.view(-1, width)
    return t


def host_copy(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to("cpu", copy=True).contiguous()


# Tables that passed the host-side check are remembered per tensor OBJECT (weak
# reference + in-place version counter), never per address: the caching
# allocator hands the address of a freed table to the next one.  A table given
# as a list or CPU tensor is checked on every call (its host copy is free).
_checked: Dict[Tuple[int, ...], Tuple[Tuple, Tuple[int, ...], Tuple]] = {}


def already_checked(tensors: Sequence[torch.Tensor], params: Tuple) -> bool:
    entry = _checked.get(tuple(id(t) for t in tensors))
    if entry is None:
        return False
    refs, versions, seen_params = entry
    if seen_params != params:
        return False
    for t, ref, ver in zip(tensors, refs, versions):
        if ref() is not t or t._version != ver:
            return False
    return True


def remember_checked(tensors: Sequence[torch.Tensor], params: Tuple) -> None:
    if len(_checked) > 1024:
        _checked.clear()
    _checked[tuple(id(t) for t in tensors)] = (
        tuple(weakref.ref(t) for t in tensors),
        tuple(t._version for t in tensors),
        params,
    )


# What a launcher worked out from a set of tables on the host (a grid size, which kernel form they allow), kept
# the same way: per tensor objects and their versions, one note per (slot, tables).
_notes: Dict[Tuple, Tuple[Tuple, Tuple[int, ...], object]] = {}


def recall_note(tensors: Sequence[torch.Tensor], slot: str):
    entry = _notes.get((slot,) + tuple(id(t) for t in tensors))
    if entry is None:
        return None
    refs, versions, value = entry
    for t, ref, ver in zip(tensors, refs, versions):
        if ref() is not t or t._version != ver:
            return None
    return value


def remember_note(tensors: Sequence[torch.Tensor], slot: str, value) -> None:
    if len(_notes) > 2048:
        _notes.clear()
    _notes[(slot,) + tuple(id(t) for t in tensors)] = (
        tuple(weakref.ref(t) for t in tensors),
        tuple(t._version for t in tensors),
        value,
    )


# Flag arrays whose owner promises what the kernels' fast flag wait needs (include/syncopate_hip.h,
# SYN_GEMM_ACQUIRE_ALWAYS): nothing on the device reads the gathered buffer between the start of a consumer
# kernel and a chunk's flag, and no flag word is raised twice during a launch.  CommContext registers the arrays
# it allocates (its copies are the only writers of its buffers, its flags are reset between iterations); a
# launch on any other flag tensor takes the acquire fence behind every flag wait, like the reference.
_trusted_flags: "weakref.WeakValueDictionary[int, torch.Tensor]" = weakref.WeakValueDictionary()


def trust_flags(*tensors: torch.Tensor) -> None:
    """Declare that the caller upholds the precondition above for these flag arrays (the tensor objects given,
    not views of them made later)."""
    for t in tensors:
        _trusted_flags[id(t)] = t


def acquire_always(signal_buffer: torch.Tensor) -> bool:
    """Whether a launch that waits on `signal_buffer` must fence behind every flag wait."""
    return _trusted_flags.get(id(signal_buffer)) is not signal_buffer


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def host_ptr(t: torch.Tensor) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr())


def require_cuda(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("operands must live in GPU memory (the kernels have no CPU path)")
        if t.device != dev:
            raise ValueError("operands must be on the same device")
    return dev


def flag_buffer(signal_buffer: torch.Tensor) -> torch.Tensor:
    """Flag arrays are 8-byte words (value 1 = set); int64 and uint64 are both accepted."""
    if signal_buffer.element_size() != 8 or signal_buffer.is_floating_point():
        raise TypeError(f"signal buffer must hold 64-bit integer words, got {signal_buffer.dtype}")
    if not signal_buffer.is_contiguous():
        raise ValueError("signal buffer must be contiguous")
    return signal_buffer
