"""Splitting a device's compute units between streams.

Counterpart of the reference's green contexts (comm_runtime/split_green_ctx.py:161-215:
`split_device_green_ctx(dev, num_groups, min_count)` returns `num_groups + 1` streams, the last
one owning the SMs that are left).  On an MI355X a stream can be created with a compute-unit
mask; bit i of the mask names XCD i % 8 and, inside that XCD, compute unit i // 8 counted in turn
over the shader engines.  A group is therefore taken as a run of consecutive bits whose length is
a multiple of 8: every XCD gives up the same number of compute units, spread over its shader
engines, and the kernels on the remaining ones still see eight equal XCDs.
"""

from __future__ import annotations

import atexit
import ctypes
from typing import List, Tuple

import torch

from ... import _lib

XCDS = 8

# Masked streams are handed out for the life of the process (a CommContext keeps using them), and are destroyed
# before the interpreter goes: a process that ended with such streams still alive has crashed inside the HIP
# runtime's own exit handlers.  `atexit` runs this hook while torch and the library are still loaded.
_live_streams: List[Tuple[int, torch.cuda.Stream]] = []
_exit_hook_registered = False


def destroy_masked_streams() -> None:
    """Wait for and destroy every stream `masked_stream` created; they must not be used afterwards."""
    lib = _lib.load()
    while _live_streams:
        handle, stream = _live_streams.pop()
        try:
            stream.synchronize()
        except Exception:       # a device already in an error state: still hand the stream back
            pass
        lib.syn_stream_destroy(ctypes.c_void_p(handle))


def cu_mask_words(first: int, count: int, total: int) -> List[int]:
    """32-bit mask words with bits [first, first + count) set, for a device of `total` compute units."""
    if first < 0 or count <= 0 or first + count > total:
        raise ValueError(f"compute units [{first}, {first + count}) are not inside [0, {total})")
    words = [0] * ((total + 31) // 32)
    for bit in range(first, first + count):
        words[bit // 32] |= 1 << (bit % 32)
    return words


def group_sizes(total: int, num_groups: int, min_count: int) -> List[int]:
    """Sizes of `num_groups` equal groups of at least `min_count` compute units, rounded up to a
    whole number per XCD, and of the group that is left."""
    if num_groups <= 0 or min_count <= 0:
        raise ValueError("num_groups and min_count must be positive")
    each = (min_count + XCDS - 1) // XCDS * XCDS
    if num_groups * each >= total:
        raise RuntimeError(f"{num_groups} groups of {each} compute units leave nothing of {total}")
    return [each] * num_groups + [total - num_groups * each]


def masked_stream(words: List[int], device: torch.device) -> torch.cuda.Stream:
    lib = _lib.load()
    handle = ctypes.c_void_p()
    arr = (ctypes.c_uint32 * len(words))(*words)
    with torch.cuda.device(device):
        _lib.check("syn_stream_create_cu_mask",
                   lib.syn_stream_create_cu_mask(arr, len(words), ctypes.byref(handle)))
    stream = torch.cuda.ExternalStream(handle.value, device=device)
    _live_streams.append((handle.value, stream))
    global _exit_hook_registered
    if not _exit_hook_registered:
        atexit.register(destroy_masked_streams)
        _exit_hook_registered = True
    return stream


def split_device_cu_mask(dev: torch.device, num_groups: int, min_count: int) -> Tuple[List[torch.cuda.Stream], List[int]]:
    """`num_groups + 1` streams on disjoint sets of compute units and the size of each set; the
    last stream owns what the groups leave."""
    total = torch.cuda.get_device_properties(dev).multi_processor_count
    sizes = group_sizes(total, num_groups, min_count)
    streams, first = [], 0
    for size in sizes:
        streams.append(masked_stream(cu_mask_words(first, size, total), dev))
        first += size
    return streams, sizes


def where_workgroups_ran(stream: torch.cuda.Stream, workgroups: int = 4096, dwell: int = 64) -> set:
    """The set of (XCD, shader engine / array / compute unit) a grid launched on `stream` occupied."""
    lib = _lib.load()
    out = torch.zeros(2 * workgroups, dtype=torch.int32, device=stream.device)
    stream.wait_stream(torch.cuda.current_stream(stream.device))
    _lib.check("syn_where_async", lib.syn_where_async(out.data_ptr(), workgroups, dwell, int(stream.cuda_stream)))
    stream.synchronize()
    words = out.cpu().view(-1, 2).tolist()
    return {(xcd & 0xF, (hw >> 8) & 0xFF) for hw, xcd in words}
