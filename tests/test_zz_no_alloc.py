"""syn_gemm_producer_static — the producer entry point that allocates nothing (its per-wave
counters live in a static device array of the library) — against syn_gemm_producer, through the
C ABI: two calls in a row, the second with a smaller input, results bit for bit."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _desc(_lib, a, b, c, flags, sizes, offsets, signals, counters, status, BM, BN, num_sms):
    M, K = a.shape
    N = b.shape[0]
    return _lib.GemmDesc(
        a=a.data_ptr(), b=b.data_ptr(), c=c.data_ptr(), flags=flags.data_ptr(), wave_sizes=sizes.data_ptr(),
        wave_offsets=offsets.data_ptr(), signal_offsets=signals.data_ptr(),
        counters=None if counters is None else counters.data_ptr(), visit_log=None, status=status.data_ptr(),
        num_waves=signals.numel(), M=M, N=N, K=K, dtype=_lib.dtype_code(a.dtype), block_m=BM, block_n=BN, block_k=64,
        group_m=8, num_sms=num_sms, cum_tiles=M * N, spin_timeout_us=0, options=0)


def _case(M, N, K, world, rank, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    a = (0.02 * torch.randn(M, K, device="cuda", generator=g)).bfloat16()
    b = (0.02 * torch.randn(N, K, device="cuda", generator=g)).bfloat16()
    rows = M // world
    table = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    sizes = table([[rows, N]] * world)
    offsets = table([[((rank + k + 1) % world) * rows, 0] for k in range(world)])
    signals = table(list(range(world)))
    return a, b, sizes, offsets, signals


def test_static_counter_producer_matches_the_allocating_one(hip):
    from syncopate_amd import _lib

    stream = _lib.stream_handle(torch.cuda.current_stream())
    status = torch.zeros(_lib.SYN_STATUS_WORDS, dtype=torch.int32, device="cuda")
    # the second call is smaller in every extent and has fewer waves: counters the first call
    # left behind in the shared array must not leak into it
    for (M, N, K, world, rank, BM, BN, num_sms) in [(4096, 2048, 512, 8, 3, 256, 256, 200),
                                                     (1024, 512, 256, 4, 1, 128, 128, 24)]:
        a, b, sizes, offsets, signals = _case(M, N, K, world, rank, seed=M)
        flags_ref = torch.zeros(world, dtype=torch.int64, device="cuda")
        counters = torch.zeros(world, dtype=torch.int32, device="cuda")
        c_ref = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        d = _desc(_lib, a, b, c_ref, flags_ref, sizes, offsets, signals, counters, status, BM, BN, num_sms)
        _lib.check("syn_gemm_producer", hip.syn_gemm_producer(ctypes.byref(d), stream))

        flags = torch.zeros(world, dtype=torch.int64, device="cuda")
        c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        d = _desc(_lib, a, b, c, flags, sizes, offsets, signals, None, status, BM, BN, num_sms)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info()[0]        # the driver's view: a hipMalloc inside the library would show here
        _lib.check("syn_gemm_producer_static", hip.syn_gemm_producer_static(ctypes.byref(d), stream))
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
        assert status.tolist()[0] == 0
        tiles_per_wave = (M // world // BM) * (N // BN)
        assert counters.tolist() == [tiles_per_wave] * world
        # the library's own array holds this launch's counts (and nothing of the larger launch before it)
        peek = (ctypes.c_int32 * world)()
        _lib.check("syn_gemm_static_counters_peek", hip.syn_gemm_static_counters_peek(peek, world))
        assert list(peek) == [tiles_per_wave] * world
        assert flags.tolist() == [1] * world and flags_ref.tolist() == [1] * world
        assert torch.equal(c, c_ref)                      # same kernel, same tile shape: bit for bit
        ref = a.float() @ b.float().t()
        assert ((c.float() - ref).abs().max() / ref.abs().max()).item() <= 1e-2


def test_static_counter_producer_rejects_what_it_cannot_hold(hip):
    from syncopate_amd import _lib

    stream = _lib.stream_handle(torch.cuda.current_stream())
    status = torch.zeros(_lib.SYN_STATUS_WORDS, dtype=torch.int32, device="cuda")
    a, b, sizes, offsets, signals = _case(512, 256, 128, 2, 0, seed=1)
    flags = torch.zeros(2, dtype=torch.int64, device="cuda")
    c = torch.zeros(512, 256, dtype=torch.bfloat16, device="cuda")
    own = torch.zeros(2, dtype=torch.int32, device="cuda")
    d = _desc(_lib, a, b, c, flags, sizes, offsets, signals, own, status, 128, 128, 8)
    assert hip.syn_gemm_producer_static(ctypes.byref(d), stream) == _lib.SYN_EINVAL      # counters are the library's
    d = _desc(_lib, a, b, c, flags, sizes, offsets, signals, None, status, 128, 128, 8)
    d.num_waves = _lib.SYN_STATIC_MAX_WAVES + 1
    assert hip.syn_gemm_producer_static(ctypes.byref(d), stream) == _lib.SYN_E2BIG
    with pytest.raises(_lib.SyncopateHipError, match="SYN_E2BIG"):
        _lib.check("syn_gemm_producer_static", _lib.SYN_E2BIG)
    torch.cuda.synchronize()
    assert flags.tolist() == [0, 0]


def test_a_rejected_call_leaves_the_static_counters_alone(hip):
    """The counters are cleared behind the checks of the descriptor: a call that is turned away must not zero words
    that an earlier launch on the device may still be counting in."""
    from syncopate_amd import _lib

    stream = _lib.stream_handle(torch.cuda.current_stream())
    status = torch.zeros(_lib.SYN_STATUS_WORDS, dtype=torch.int32, device="cuda")
    a, b, sizes, offsets, signals = _case(512, 256, 128, 2, 0, seed=2)
    flags = torch.zeros(2, dtype=torch.int64, device="cuda")
    c = torch.zeros(512, 256, dtype=torch.bfloat16, device="cuda")
    d = _desc(_lib, a, b, c, flags, sizes, offsets, signals, None, status, 128, 128, 8)
    _lib.check("syn_gemm_producer_static", hip.syn_gemm_producer_static(ctypes.byref(d), stream))
    torch.cuda.synchronize()
    peek = (ctypes.c_int32 * 2)()
    _lib.check("syn_gemm_static_counters_peek", hip.syn_gemm_static_counters_peek(peek, 2))
    assert list(peek) == [4, 4]
    bad = _desc(_lib, a, b, c, flags, sizes, offsets, signals, None, status, 128, 64, 8)      # divides N, but no kernel has this tile shape
    assert hip.syn_gemm_producer_static(ctypes.byref(bad), stream) == _lib.SYN_EINVAL
    bad = _desc(_lib, a, b, c, flags, sizes, offsets, signals, None, status, 128, 128, 8)
    bad.a = a.data_ptr() + 2                                                                   # misaligned operand
    assert hip.syn_gemm_producer_static(ctypes.byref(bad), stream) == _lib.SYN_EALIGN
    torch.cuda.synchronize()
    _lib.check("syn_gemm_static_counters_peek", hip.syn_gemm_static_counters_peek(peek, 2))
    assert list(peek) == [4, 4]
