"""Side streams that can run beside the compute stream.

A HIP process has a few hardware queues (four by default) and every stream is bound to one of
them; packets of one queue start in order.  A flag wait spinning on a side stream therefore holds
back every later kernel of the streams that share its queue - the compute kernel that would set
the flag included - and a consumer kernel polling for a chunk holds back the copy that carries it.
The reference's stream memory operations (cuStreamWaitValue, communication_context.py:150-160)
have no such coupling, so here the executor has to choose its streams: a candidate shares a queue
with `other` exactly when a bounded wait on the candidate keeps a flag write on `other` from
running, which takes two tiny kernels to find out.
"""

from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ... import _lib

_PROBE_BUDGET_US = 20_000       # a write that is not held back lands within tens of microseconds
_POOL = 32                      # torch hands out its 32 pooled streams per device in turn


def shares_hardware_queue(candidate: torch.cuda.Stream, other: torch.cuda.Stream) -> bool:
    """True if kernels of `other` queue up behind a kernel still running on `candidate`."""
    if candidate.cuda_stream == other.cuda_stream:
        return True
    lib = _lib.load()
    device = candidate.device
    with torch.cuda.device(device):
        flag = torch.zeros(1, dtype=torch.int64, device=device)
        status = torch.zeros(_lib.SYN_STATUS_WORDS, dtype=torch.int32, device=device)
        torch.cuda.synchronize(device)
        _lib.check("syn_flag_wait", lib.syn_flag_wait(flag.data_ptr(), 1, _PROBE_BUDGET_US, status.data_ptr(),
                                                      int(candidate.cuda_stream)))
        _lib.check("syn_flag_set", lib.syn_flag_set(flag.data_ptr(), 1, int(other.cuda_stream)))
        torch.cuda.synchronize(device)
        return int(status[0].item()) != 0


def pick_side_streams(count: int, compute_stream: Optional[torch.cuda.Stream] = None,
                      device: Optional[torch.device] = None,
                      avoid: Sequence[torch.cuda.Stream] = ()) -> List[torch.cuda.Stream]:
    """`count` streams, none on the hardware queue of `compute_stream` (the current stream by
    default) or of a stream in `avoid`, and on queues of their own among themselves as far as the
    queues go round; beyond that the extra streams double up with earlier side streams, never
    with the compute stream."""
    if count <= 0:
        return []
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    compute = torch.cuda.current_stream(device) if compute_stream is None else compute_stream
    apart: List[torch.cuda.Stream] = []          # on queues of their own
    spare: List[torch.cuda.Stream] = []          # clear of the compute stream, doubling up with a side stream
    seen = set()
    for _ in range(_POOL):
        if len(apart) == count:
            break
        cand = torch.cuda.Stream(device=device)
        if cand.cuda_stream in seen:
            break                                # the pool has come round
        seen.add(cand.cuda_stream)
        if any(shares_hardware_queue(cand, s) for s in (compute, *avoid)):
            continue
        if any(shares_hardware_queue(cand, s) for s in apart):
            spare.append(cand)
        else:
            apart.append(cand)
    if not apart:
        raise RuntimeError("no stream on a hardware queue apart from the compute stream's: "
                           "flag waits on a side stream would hold the compute kernel back")
    picked = apart + spare[:max(0, count - len(apart))]
    while len(picked) < count:
        picked.append(apart[len(picked) % len(apart)])
    return picked
