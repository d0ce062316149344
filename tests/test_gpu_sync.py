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


def test_device_split_by_compute_unit_masks(hip):
    """Streams on disjoint sets of compute units (the reference splits the device into green
    contexts, comm_runtime/split_green_ctx.py:161-215): a grid on each stream stays inside its
    set, the sets are disjoint, and every XCD gives the same number of units to the small group."""
    from syncopate_amd.communication.comm_runtime.cu_partition import (
        cu_mask_words,
        group_sizes,
        split_device_cu_mask,
        where_workgroups_ran,
    )

    dev = torch.device("cuda", 0)
    total = torch.cuda.get_device_properties(dev).multi_processor_count
    everywhere = where_workgroups_ran(torch.cuda.current_stream())
    assert len(everywhere) == total
    streams, sizes = split_device_cu_mask(dev, 1, 20)
    assert sizes == [24, total - 24] and len(streams) == 2
    small, rest = (where_workgroups_ran(s) for s in streams)
    assert len(small) == 24 and len(rest) == total - 24
    assert not (small & rest) and (small | rest) == everywhere
    per_xcd = {}
    for xcd, _ in small:
        per_xcd[xcd] = per_xcd.get(xcd, 0) + 1
    assert sorted(per_xcd.values()) == [3] * 8
    # kernels on the two streams run side by side and both finish
    a, b = (torch.zeros(1 << 20, device=dev) for _ in range(2))
    for s, t in zip(streams, (a, b)):
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            t.add_(1.0)
    torch.cuda.synchronize()
    assert a.sum().item() == b.sum().item() == float(1 << 20)
    assert cu_mask_words(8, 24, 64) == [0xFFFFFF00, 0]
    assert group_sizes(256, 2, 9) == [16, 16, 224]


def test_mfma_rate_probe_runs_and_rejects_bad_arguments(hip):
    """The measurement aid of the benchmark: every pattern runs; constant operands give the exact sum."""
    from syncopate_amd import _lib

    sink = torch.zeros(4 * 256, dtype=torch.float32, device="cuda")
    stream = _lib.stream_handle(torch.cuda.current_stream())
    for pattern in (0, 1, 2, 4, 5, 6):
        sink.fill_(-1.0)
        _lib.check("syn_probe_mfma_rate", hip.syn_probe_mfma_rate(sink.data_ptr(), 4, 3, pattern, stream))
        torch.cuda.synchronize()
        assert torch.isfinite(sink).all()
        if pattern in (0, 4):
            assert (sink == 0).all()
        if pattern == 1:
            # 3 rounds x 4 fragment sets x 16 (k) ones per accumulator element, two elements of 16 accumulators summed
            assert (sink == 3 * 4 * 16 * 2 * 16).all()
        if pattern == 5:
            # the 16x16x32 form: 3 rounds x 2 fragment sets x 32 (k), two elements of 64 accumulators summed
            assert (sink == 3 * 2 * 32 * 2 * 64).all()
    for bad in (3, 7, 8, -1):
        assert hip.syn_probe_mfma_rate(sink.data_ptr(), 4, 3, bad, stream) == _lib.SYN_EINVAL
    assert hip.syn_probe_mfma_rate(None, 4, 3, 0, stream) == _lib.SYN_EINVAL
    assert hip.syn_probe_mfma_rate(sink.data_ptr(), 0, 3, 0, stream) == _lib.SYN_EINVAL


def test_read_stream_probe_reads_what_it_says(hip):
    """The benchmark's HBM read probe: eight streams a stride apart, one pass of 1024 groups each.  A marker in
    the first 256 groups of the last stream reaches every lane once and shows up in the sink; the same
    marker just past the stream's end is never read."""
    from syncopate_amd import _lib

    magic, stream_bytes, stride = 0x9E3779B9, 16384, 16384 + 4096
    stream = _lib.stream_handle(torch.cuda.current_stream())
    for beyond in (False, True):
        words = torch.zeros((8 * stride + 16384) // 4, dtype=torch.int32, device="cuda")
        first = (7 * stride + (stream_bytes if beyond else 0)) // 4
        words[first:first + 4 * 256:4] = magic - (1 << 32)
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        _lib.check("syn_probe_read_streams",
                   hip.syn_probe_read_streams(words.data_ptr(), stream_bytes, stride, 8, 1, sink.data_ptr(), stream))
        torch.cuda.synchronize()
        got = [w & 0xFFFFFFFF for w in sink.tolist()]
        assert got == ([0, 0, 0, 0] if beyond else [magic, 0, 0, 0])
    assert hip.syn_probe_read_streams(words.data_ptr(), 16000, stride, 8, 1, sink.data_ptr(), stream) == _lib.SYN_EINVAL
    assert hip.syn_probe_read_streams(words.data_ptr(), stream_bytes, stride, 3, 1, sink.data_ptr(), stream) == _lib.SYN_EINVAL
    assert hip.syn_probe_read_streams(words.data_ptr(), stream_bytes, stride + 8, 8, 1, sink.data_ptr(), stream) == _lib.SYN_EALIGN
    assert hip.syn_probe_read_streams(None, stream_bytes, stride, 8, 1, sink.data_ptr(), stream) == _lib.SYN_EINVAL


def test_flag_write_as_a_stream_memory_operation(hip):
    """syn_flag_write_value: the flag word is written by the stream itself, in stream order."""
    from syncopate_amd import _lib

    flags = torch.zeros(4, dtype=torch.int64, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    _lib.check("syn_delay_us", hip.syn_delay_us(500, _lib.stream_handle(side)))
    _lib.check("syn_flag_write_value", hip.syn_flag_write_value(flags.data_ptr() + 16, 1, _lib.stream_handle(side)))
    side.synchronize()
    assert flags.tolist() == [0, 0, 1, 0]
    assert hip.syn_flag_write_value(None, 1, _lib.stream_handle(side)) == _lib.SYN_EINVAL


def test_attention_slot_probe_runs_every_piece_and_rejects_bad_arguments(hip):
    """syn_probe_attn_slot: every combination of pieces runs to completion on a few workgroups and reports the
    cycles of both halves; the argument checks of the entry point."""
    from syncopate_amd import _lib

    stream = _lib.stream_handle(torch.cuda.current_stream())
    workgroups, iters = 4, 3
    needed = workgroups * 65536 + (32 << 20)
    pool = torch.zeros(needed + 64, dtype=torch.uint8, device="cuda")
    sink = torch.zeros(workgroups * 512, dtype=torch.float32, device="cuda")
    cycles = torch.zeros(2, dtype=torch.int64, device="cuda")

    def run(what, nbytes=needed, wg=workgroups):
        return hip.syn_probe_attn_slot(pool.data_ptr(), nbytes, wg, iters, what, sink.data_ptr(), cycles.data_ptr(), stream)

    for what in (1, 2, 3, 1 | 4, 3 | 4, 3 | 4 | 8, 3 | 4 | 8 | 16, 3 | 4 | 8 | 32, 1 | 4 | 16, 2 | 8, 3 | 4 | 8 | 64,
                 1 | 128, 3 | 4 | 8 | 32 | 128, 3 | 4 | 8 | 16 | 128):
        cycles.zero_()
        _lib.check("syn_probe_attn_slot", run(what))
        torch.cuda.synchronize()
        assert min(cycles.tolist()) > 0, what
        assert torch.isfinite(sink).all()
    assert run(0) == _lib.SYN_EINVAL
    assert run(256) == _lib.SYN_EINVAL
    assert run(128) == _lib.SYN_EINVAL               # the narrow form of products that do not run
    assert run(2 | 128) == _lib.SYN_EINVAL
    assert run(4) == _lib.SYN_EINVAL                 # operands from LDS, but neither half runs
    assert run(1 | 16) == _lib.SYN_EINVAL            # early fragments without LDS reads
    assert run(3, nbytes=needed - 1) == _lib.SYN_EINVAL
    assert run(3, wg=0) == _lib.SYN_EINVAL
    assert hip.syn_probe_attn_slot(None, needed, workgroups, iters, 3, sink.data_ptr(), cycles.data_ptr(), stream) == _lib.SYN_EINVAL
    assert hip.syn_probe_attn_slot(pool.data_ptr() + 8, needed, workgroups, iters, 3, sink.data_ptr(),
                                   cycles.data_ptr(), stream) == _lib.SYN_EALIGN


def test_skewed_read_stream_probe_reads_what_it_says(hip):
    """The skewed form of the read probe (eight blocks of 4 KB per stream and workgroup, stream i one block behind
    stream i - 1): the marker in the first block of the last stream reaches every lane once; past the stream's
    end it is never read."""
    from syncopate_amd import _lib

    magic, stream_bytes, stride = 0x9E3779B9, 32768, 32768 + 4096
    stream = _lib.stream_handle(torch.cuda.current_stream())
    for beyond in (False, True):
        words = torch.zeros((8 * stride + 32768) // 4, dtype=torch.int32, device="cuda")
        first = (7 * stride + (stream_bytes if beyond else 0)) // 4
        words[first:first + 4 * 256:4] = magic - (1 << 32)
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        _lib.check("syn_probe_read_streams_skewed",
                   hip.syn_probe_read_streams_skewed(words.data_ptr(), stream_bytes, stride, 1, sink.data_ptr(), stream))
        torch.cuda.synchronize()
        got = [w & 0xFFFFFFFF for w in sink.tolist()]
        assert got == ([0, 0, 0, 0] if beyond else [magic, 0, 0, 0])
    assert hip.syn_probe_read_streams_skewed(words.data_ptr(), 16384, stride, 1, sink.data_ptr(), stream) == _lib.SYN_EINVAL
    assert hip.syn_probe_read_streams_skewed(words.data_ptr(), stream_bytes, stride + 8, 1, sink.data_ptr(), stream) == _lib.SYN_EALIGN
    assert hip.syn_probe_read_streams_skewed(None, stream_bytes, stride, 1, sink.data_ptr(), stream) == _lib.SYN_EINVAL
