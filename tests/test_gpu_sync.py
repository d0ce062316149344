"""Stream-side plumbing of the single-GPU executor on the GPU: which streams may carry flag waits."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_side_streams_avoid_the_compute_streams_hardware_queue(hip):
    """A process has a handful of hardware queues; a stream that shares one with the compute
    stream would keep a polling kernel and the kernel that answers it in one queue."""
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams, shares_hardware_queue

    compute = torch.cuda.current_stream()
    assert shares_hardware_queue(compute, compute)
    picked = pick_side_streams(2)
    assert len(picked) == 2 and picked[0].cuda_stream != picked[1].cuda_stream
    for s in picked:
        assert not shares_hardware_queue(s, compute)
        assert not shares_hardware_queue(compute, s)
    assert not shares_hardware_queue(picked[0], picked[1])
    # more streams than queues: still none beside the compute stream
    for s in pick_side_streams(6):
        assert not shares_hardware_queue(s, compute)
    # another compute stream, other side streams
    other = picked[0]
    for s in pick_side_streams(2, compute_stream=other):
        assert not shares_hardware_queue(s, other)
