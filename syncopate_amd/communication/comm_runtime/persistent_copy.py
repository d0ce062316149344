"""Copies and accumulations of strided boxes by a persistent grid of workgroups.

Host side of `syn_box_copy_async`.  Same interface and checks as the reference's
`persistent_naive_copy_last_contig` / `persistent_tma_copy_last_contig`
(comm_runtime/non_tma_persistent_copy.py:191-304, tma_persistent_copy.py): same shape and dtype
on both sides, at most five dimensions once leading 1-extents are dropped, last dimension
contiguous, `reduce_op` None (copy) or SUM (dst += src).  There is one kernel here for both names:
gfx950 has no descriptor-driven bulk copy to tell them apart.
"""

from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence, Tuple

import torch

from ... import _lib
from ..descriptor import ReduceOp

MAX_RANK = 5
DEFAULT_BLOCKS = 256            # one workgroup per compute unit

_FLOAT_KINDS = {
    torch.bfloat16: _lib.SYN_ELEM_BF16,
    torch.float16: _lib.SYN_ELEM_FP16,
    torch.float32: _lib.SYN_ELEM_FP32,
}
_SIZE_KINDS = {1: _lib.SYN_ELEM_1B, 2: _lib.SYN_ELEM_2B, 4: _lib.SYN_ELEM_4B, 8: _lib.SYN_ELEM_8B}


def _drop_leading_ones(t: torch.Tensor) -> torch.Tensor:
    while t.dim() > 1 and t.shape[0] == 1:
        t = t[0]
    return t


def merge_box_dims(shape: Sequence[int], src_strides: Sequence[int],
                   dst_strides: Sequence[int]) -> Tuple[List[int], List[int], List[int]]:
    """Drop 1-extents and fold neighbours that are dense in BOTH tensors into one dimension
    (stride[d - 1] == shape[d] * stride[d]); what remains is the shortest description of the box.
    The reference folds only the dense suffix (squeeze_common_dense_suffix); folding everywhere
    moves the same bytes with fewer index divisions."""
    dims = [(n, s, d) for n, s, d in zip(shape, src_strides, dst_strides) if n != 1]
    if not dims:
        return [], [], []
    merged = [dims[0]]
    for n, s, d in dims[1:]:
        pn, ps, pd = merged[-1]
        if ps == n * s and pd == n * d:
            merged[-1] = (pn * n, s, d)
        else:
            merged.append((n, s, d))
    return [m[0] for m in merged], [m[1] for m in merged], [m[2] for m in merged]


def persistent_copy_last_contig(src: torch.Tensor, dst: torch.Tensor, *, num_sms: Optional[int] = None,
                                reduce_op: Optional[ReduceOp] = None,
                                stream: Optional[torch.cuda.Stream] = None,
                                exclusive: bool = False) -> torch.Tensor:
    """dst[...] = src[...] or, with `reduce_op=ReduceOp.SUM`, dst[...] += src[...] on `stream`
    (the current one by default) with at most `num_sms` workgroups of 1024 threads.

    Sums are atomic adds as in the reference, so that several senders may accumulate into one
    destination at a time.  `exclusive=True` (not in the reference) promises that nobody else
    writes the destination box meanwhile: the sum is then a plain read-modify-write, which the
    memory system takes several times faster."""
    src = _drop_leading_ones(src)
    dst = _drop_leading_ones(dst)
    if not (src.is_cuda and dst.is_cuda):
        raise ValueError("device tensors only")
    if src.device != dst.device:
        raise ValueError("src/dst must be on same device")
    if src.shape != dst.shape:
        raise ValueError("src/dst must have same shape")
    if src.dtype != dst.dtype:
        raise ValueError("src/dst must have same dtype")
    if src.dim() > MAX_RANK:
        raise ValueError(f"rank > {MAX_RANK} not supported")
    if src.dim() == 0:
        src, dst = src.reshape(1), dst.reshape(1)
    if src.stride()[-1] != 1 and src.shape[-1] != 1 or dst.stride()[-1] != 1 and dst.shape[-1] != 1:
        raise ValueError(f"require stride[-1]==1. got src {src.stride()} dst {dst.stride()}")
    if reduce_op is not None and reduce_op != ReduceOp.SUM:
        raise ValueError(f"unsupported reduce_op {reduce_op}")
    if reduce_op is not None and src.dtype not in _FLOAT_KINDS:
        raise ValueError(f"sums are for bfloat16, float16 and float32, not {src.dtype}")
    if num_sms is None:
        num_sms = DEFAULT_BLOCKS
    num_sms = int(num_sms)
    if num_sms <= 0:
        raise ValueError("num_sms must be positive")
    if src.numel() == 0:
        return dst
    if any(s < 0 for s in src.stride()) or any(s < 0 for s in dst.stride()):
        raise ValueError("negative strides are not supported")

    shape, sst, dstr = merge_box_dims(src.shape, src.stride(), dst.stride())
    if not shape or sst[-1] != 1 or dstr[-1] != 1:
        # the last extent was 1 and went away: the kernel still wants a contiguous last dimension
        shape.append(1)
        sst.append(1)
        dstr.append(1)

    kind = _FLOAT_KINDS.get(src.dtype) if reduce_op is not None else _SIZE_KINDS.get(src.element_size())
    if kind is None:
        raise ValueError(f"element size {src.element_size()} not supported")
    if reduce_op is None:
        mode = _lib.SYN_BOX_COPY
    else:
        mode = _lib.SYN_BOX_ADD_EXCLUSIVE if exclusive else _lib.SYN_BOX_ADD_ATOMIC
    n = len(shape)
    arr = ctypes.c_int64 * n
    handle = int((torch.cuda.current_stream(src.device) if stream is None else stream).cuda_stream)
    _lib.check("syn_box_copy_async",
               _lib.load().syn_box_copy_async(dst.data_ptr(), src.data_ptr(), n, arr(*shape), arr(*sst),
                                              arr(*dstr), kind, mode, num_sms, handle))
    return dst


# the reference's two names for the operation
persistent_naive_copy_last_contig = persistent_copy_last_contig
persistent_tma_copy_last_contig = persistent_copy_last_contig
