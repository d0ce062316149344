"""GPU parity of the chunk-scheduled GEMM kernels against the CPU oracle (through the C ABI)."""

import pytest
import torch

from oracle import numerics, visit_order

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2  # max |err| / max |ref| against torch fp32, the bound the path is specified to


def _inputs(M, N, K, dtype, seed=0, scale=0.02):
    g = torch.Generator(device="cpu").manual_seed(seed)
    a = (scale * torch.randn(M, K, generator=g)).to(dtype)
    b = (scale * torch.randn(N, K, generator=g)).to(dtype)
    return a, b


def _row_waves(M, N, world, rank):
    """AG-GEMM wave table of `rank`: chunk (rank+k) % world arrives k-th, flag k-1."""
    rows = M // world
    sizes = [[rows, N] for _ in range(world)]
    offsets = [[((rank + k) % world) * rows, 0] for k in range(world)]
    signals = [-1] + list(range(world - 1))
    return sizes, offsets, signals


def _max_rel_err(out, ref):
    return ((out.float().cpu() - ref).abs().max() / ref.abs().max()).item()


def _check_visits(log, sizes, offsets, signals, M, N, BM, BN, group_m, num_sms, cum_tiles, remap):
    from syncopate_amd.computation._launch import check_status  # noqa: F401

    want = visit_order.gemm_tile_visits(sizes, offsets, signals, M=M, N=N, BM=BM, BN=BN,
                                        group_m=group_m, num_sms=num_sms, cum_tiles=cum_tiles)
    got = log.cpu().view(-1, 4).tolist()
    assert len(got) >= len(want)
    for v in want:
        pid, wave, pm, pn = got[v["tile_id"]]
        assert (pid, wave, pm, pn) == (v["pid"], v["wave"], v["pid_m"], v["pid_n"]), v


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("BM,BN", [(128, 128), (128, 256), (256, 128), (256, 256)])
def test_consumer_resident_matches_fp32_and_visit_order(hip, dtype, BM, BN):
    from syncopate_amd.computation.gemm import gemm_consumer
    from syncopate_amd.computation._launch import check_status

    M, N, K, world, rank = 2048, 1024, 512, 4, 1
    a, b = _inputs(M, N, K, dtype)
    sizes, offsets, signals = _row_waves(M, N, world, rank)
    ref = numerics.gemm_fp32(a, b)
    ad, bd = a.cuda(), b.cuda()
    c = torch.zeros(M, N, dtype=dtype, device="cuda")
    flags = torch.ones(world, dtype=torch.int64, device="cuda")
    tiles = (M // BM) * (N // BN)
    # (programs, XCD remap, 8 wavefronts, four-stage ring instead of the two-stage pipeline)
    variants = [(256, True, False, False), (24, False, False, True), (7, True, False, False)]
    if (BM, BN) != (128, 128):
        variants += [(256, True, True, False), (13, False, True, True)]
    outputs = []
    for num_sms, remap, eight, ring in variants:
        c.zero_()
        log = torch.full((tiles, 4), -1, dtype=torch.int32, device="cuda")
        gemm_consumer(ad, bd, c, flags, sizes, offsets, signals, world, num_sms, BM, BN, 64, 8,
                      cum_tiles=M * N, visit_log=log, xcd_remap=remap, eight_waves=eight, ring_pipe=ring)
        check_status()
        assert _max_rel_err(c, ref) <= REL_TOL
        _check_visits(log, sizes, offsets, signals, M, N, BM, BN, 8, num_sms, M * N, remap)
        outputs.append(c.clone())
    # every variant sums each dot product over k in the same order: results are bitwise equal
    for other in outputs[1:]:
        assert torch.equal(outputs[0], other)
    # without the tile-dependent starting slab every tile sums k from 0: another order, the same product to rounding
    c.zero_()
    gemm_consumer(ad, bd, c, flags, sizes, offsets, signals, world, 24, BM, BN, 64, 8, cum_tiles=M * N, k_stagger=False)
    check_status()
    assert _max_rel_err(c, ref) <= REL_TOL


def test_consumer_k_not_multiple_of_128(hip):
    """Odd slab counts in the two-stage pipeline; a ring request falls back to it."""
    from syncopate_amd.computation.gemm import gemm_consumer
    from syncopate_amd.computation._launch import check_status

    for K in (64, 192, 320):
        M, N = 512, 512
        a, b = _inputs(M, N, K, torch.bfloat16, seed=K)
        sizes, offsets, signals = _row_waves(M, N, 2, 1)
        flags = torch.ones(1, dtype=torch.int64, device="cuda")
        for BM, BN, eight in [(256, 256, False), (128, 256, True), (128, 128, False)]:
            c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
            gemm_consumer(a.cuda(), b.cuda(), c, flags, sizes, offsets, signals, 2, 256, BM, BN,
                          cum_tiles=M * N, eight_waves=eight, ring_pipe=(K == 192))
            check_status()
            assert _max_rel_err(c, numerics.gemm_fp32(a, b)) <= REL_TOL


def test_consumer_group_size_and_column_waves(hip):
    """Waves that split N as well as M, ragged groups (GROUP_SIZE_M does not divide the wave)."""
    from syncopate_amd.computation.gemm import gemm
    from syncopate_amd.computation._launch import check_status

    M, N, K, BM, BN = 1536, 1024, 256, 128, 128
    a, b = _inputs(M, N, K, torch.bfloat16, seed=3)
    ref = numerics.gemm_fp32(a, b)
    sizes = [[640, 512], [896, 512], [640, 512], [896, 512]]
    offsets = [[0, 512], [640, 0], [0, 0], [640, 512]]
    signals = [1, -1, 0, 2]
    cum = sum(s[0] * s[1] for s in sizes)
    assert cum == M * N
    flags = torch.ones(3, dtype=torch.int64, device="cuda")
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    for group_m, num_sms in [(3, 17), (8, 256), (1, 5)]:
        c.zero_()
        log = torch.full((cum // (BM * BN), 4), -1, dtype=torch.int32, device="cuda")
        gemm(a.cuda(), b.cuda(), c, 1, num_sms, BM, BN, 64, group_m, cur_wave_sizes=sizes,
             wave_offsets=offsets, signal_ptr=flags, signal_offsets=signals, cum_tiles=cum,
             visit_log=log)
        check_status()
        assert _max_rel_err(c, ref) <= REL_TOL
        _check_visits(log, sizes, offsets, signals, M, N, BM, BN, group_m, num_sms, cum, True)


def _random_cells(rng, extent, block, max_parts):
    """`extent` cut into 1..max_parts runs of whole blocks: [(first, length)] in elements."""
    blocks = extent // block
    parts = int(rng.integers(1, min(max_parts, blocks) + 1))
    cuts = sorted(rng.choice(range(1, blocks), size=parts - 1, replace=False).tolist()) if parts > 1 else []
    edges = [0] + cuts + [blocks]
    return [(lo * block, (hi - lo) * block) for lo, hi in zip(edges, edges[1:])]


@pytest.mark.parametrize("seed", list(range(8)))
def test_consumer_random_wave_tables(hip, seed):
    """Wave tables drawn at random - the M x N tile space cut into cells of ragged sizes, visited in a random order,
    with a random group size, program count, tile shape and flag assignment: the visit log equals the
    oracle's walk tile by tile and the product is within tolerance."""
    import numpy as np

    from syncopate_amd.computation.gemm import gemm
    from syncopate_amd.computation._launch import check_status

    rng = np.random.default_rng(1000 + seed)
    BM, BN = [(128, 128), (128, 256), (256, 128), (256, 256)][seed % 4]
    M, N, K = 256 * int(rng.integers(2, 7)), 256 * int(rng.integers(1, 5)), 64 * int(rng.integers(2, 7))
    rows, cols = _random_cells(rng, M, BM, 4), _random_cells(rng, N, BN, 3)
    cells = [(r, c) for r in rows for c in cols]
    order = rng.permutation(len(cells)).tolist()
    sizes = [[cells[i][0][1], cells[i][1][1]] for i in order]
    offsets = [[cells[i][0][0], cells[i][1][0]] for i in order]
    num_flags = 3
    signals = [int(rng.integers(-1, num_flags)) for _ in order]
    group_m, num_sms = int(rng.choice([1, 2, 3, 8])), int(rng.integers(1, 48))
    a, b = _inputs(M, N, K, torch.bfloat16, seed=seed)
    ref = numerics.gemm_fp32(a, b)
    flags = torch.ones(num_flags, dtype=torch.int64, device="cuda")
    c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    tiles = (M // BM) * (N // BN)
    log = torch.full((tiles, 4), -1, dtype=torch.int32, device="cuda")
    gemm(a.cuda(), b.cuda(), c, 1, num_sms, BM, BN, 64, group_m, cur_wave_sizes=sizes, wave_offsets=offsets,
         signal_ptr=flags, signal_offsets=signals, cum_tiles=M * N, visit_log=log, xcd_remap=bool(seed & 1))
    check_status()
    assert _max_rel_err(c, ref) <= REL_TOL
    want = visit_order.gemm_tile_visits(sizes, offsets, signals, M=M, N=N, BM=BM, BN=BN, group_m=group_m,
                                        num_sms=num_sms, cum_tiles=M * N)
    got = log.cpu().tolist()
    assert len(want) == tiles
    grid = min(num_sms, tiles)
    for v in want:
        pid, wave, pm, pn = got[v["tile_id"]]
        assert (wave, pm, pn) == (v["wave"], v["pid_m"], v["pid_n"]), v
        if not seed & 1:
            assert pid == v["pid"]
        else:
            assert 0 <= pid < grid      # with the XCD remap the log holds the logical program id
    if seed & 1:
        assert [got[v["tile_id"]][0] for v in want] == [v["pid"] for v in want]


def test_consumer_gated_by_side_stream_producer(hip):
    """Chunks land in the symmetric buffer on a side stream (copy, then flag) while the
    consumer is already running; the result must be bitwise the resident one (the flow of
    tests/test_ag_gemm_hand.py:19-45, 70-130 with the hand-written consumer)."""
    from syncopate_amd import _lib
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams
    from syncopate_amd.computation.gemm import gemm_consumer
    from syncopate_amd.computation._launch import check_status

    M, N, K, world, rank, BM, BN = 4096, 1024, 1024, 8, 3, 128, 256
    a, b = _inputs(M, N, K, torch.bfloat16, seed=5)
    sizes, offsets, signals = _row_waves(M, N, world, rank)
    staged = a.cuda()
    bd = b.cuda()
    flags = torch.ones(world - 1, dtype=torch.int64, device="cuda")
    c_res = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    gemm_consumer(staged, bd, c_res, flags, sizes, offsets, signals, world, 200, BM, BN, cum_tiles=M * N)
    torch.cuda.synchronize()

    rows = M // world
    symm = torch.full((M, K), float("nan"), dtype=torch.bfloat16, device="cuda")   # poison
    symm[rank * rows:(rank + 1) * rows].copy_(staged[rank * rows:(rank + 1) * rows])
    flags.zero_()
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    # a stream on the compute stream's hardware queue would leave the copies stuck behind the polling kernel
    side = pick_side_streams(1)[0]
    torch.cuda.synchronize()
    main = torch.cuda.current_stream()
    side.wait_stream(main)
    # consumer first, with head-room of 56 CUs for the copies
    gemm_consumer(symm, bd, c, flags, sizes, offsets, signals, world, 200, BM, BN, cum_tiles=M * N,
                  spin_timeout_us=3_000_000)
    nbytes = rows * K * 2
    for k in range(1, world):
        chunk = (rank + k) % world
        _lib.check("syn_delay_us", hip.syn_delay_us(200, _lib.stream_handle(side)))
        _lib.check("syn_copy_async", hip.syn_copy_async(symm.data_ptr() + chunk * nbytes,
                                                        staged.data_ptr() + chunk * nbytes, nbytes,
                                                        _lib.stream_handle(side)))
        _lib.check("syn_flag_set", hip.syn_flag_set(flags.data_ptr() + 8 * (k - 1), 1,
                                                    _lib.stream_handle(side)))
    main.wait_stream(side)
    check_status()
    assert flags.tolist() == [1] * (world - 1)
    assert torch.equal(c, c_res)
    assert _max_rel_err(c, numerics.gemm_fp32(a, b)) <= REL_TOL


def test_consumer_flag_never_set_times_out_cleanly(hip):
    from syncopate_amd.computation.gemm import gemm_consumer
    from syncopate_amd.computation._launch import FlagWaitTimeout, check_status

    M, N, K, world = 512, 256, 128, 2
    a, b = _inputs(M, N, K, torch.bfloat16)
    sizes, offsets, signals = _row_waves(M, N, world, 0)
    flags = torch.zeros(1, dtype=torch.int64, device="cuda")
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    gemm_consumer(a.cuda(), b.cuda(), c, flags, sizes, offsets, signals, world, 64, 128, 128,
                  cum_tiles=M * N, spin_timeout_us=20_000)
    with pytest.raises(FlagWaitTimeout):
        check_status()
    check_status()  # status words were reset


def test_bad_tables_are_rejected_before_launch(hip):
    from syncopate_amd import _lib
    from syncopate_amd.computation.gemm import gemm_consumer

    M, N, K = 512, 256, 128
    a, b = _inputs(M, N, K, torch.bfloat16)
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    flags = torch.ones(1, dtype=torch.int64, device="cuda")
    cases = [
        ([[256, 256], [256, 256]], [[0, 0], [512, 0]], [-1, 0]),   # rows beyond M
        ([[256, 256], [256, 256]], [[0, 0], [256, 0]], [-1, 1]),   # flag index beyond the array
        ([[256, 256], [200, 256]], [[0, 0], [256, 0]], [-1, 0]),   # not a multiple of the block
        ([[256, 256]], [[0, 0]], [-1]),                            # covers half of cum_tiles
    ]
    for sizes, offsets, signals in cases:
        with pytest.raises(_lib.SyncopateHipError):
            gemm_consumer(a.cuda(), b.cuda(), c, flags, sizes, offsets, signals, 2, 64, 128, 128,
                          cum_tiles=M * N)


@pytest.mark.parametrize("BM,BN", [(128, 256), (256, 256)])
def test_producer_counters_flags_and_result(hip, BM, BN):
    """GEMM+RS producer: wave order (r+1..r+W-1, r), every counter == tiles of its wave,
    every flag == 1 (reference: tests/computation/gemm/test_gemm_producer.py:34-36)."""
    from syncopate_amd.computation.gemm import gemm_producer

    M, N, K, world, rank = 2048, 1024, 512, 8, 2
    a, b = _inputs(M, N, K, torch.bfloat16, seed=7)
    rows = M // world
    order = [(rank + k + 1) % world for k in range(world)]
    sizes = [[rows, N]] * world
    offsets = [[ch * rows, 0] for ch in order]
    signals = list(range(world))
    flags = torch.zeros(world, dtype=torch.int64, device="cuda")
    counters = torch.zeros(world, dtype=torch.int32, device="cuda")
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    log = torch.full(((M // BM) * (N // BN), 4), -1, dtype=torch.int32, device="cuda")
    gemm_producer(a.cuda(), b.cuda(), c, flags, sizes, offsets, signals, 256, BM, BN,
                  cum_tiles=M * N, counter_buffer=counters, visit_log=log)
    torch.cuda.synchronize()
    per_wave = (rows // BM) * (N // BN)
    assert counters.tolist() == [per_wave] * world
    assert flags.tolist() == [1] * world
    assert _max_rel_err(c, numerics.gemm_fp32(a, b)) <= REL_TOL
    _check_visits(log, sizes, offsets, signals, M, N, BM, BN, 8, 256, M * N, True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_consumer_256x224_tiles(hip, dtype):
    """The 224-wide tile (four wavefronts stacked in M, 2 x 7 MFMA tiles each): N = 3584 is 16 of
    them.  Ragged program counts, odd and even slab counts, both slab pipelines."""
    from syncopate_amd.computation.gemm import gemm_consumer
    from syncopate_amd.computation._launch import check_status

    for M, N, K, world, num_sms, two_stage in [(1024, 448, 256, 2, 7, False), (2048, 896, 512, 4, 61, False),
                                               (2048, 896, 320, 4, 256, True), (1024, 448, 192, 2, 3, False)]:
        a, b = _inputs(M, N, K, dtype, seed=K)
        sizes, offsets, signals = _row_waves(M, N, world, 1)
        flags = torch.ones(world, dtype=torch.int64, device="cuda")
        c = torch.zeros(M, N, dtype=dtype, device="cuda")
        log = torch.full(((M // 256) * (N // 224), 4), -1, dtype=torch.int32, device="cuda")
        gemm_consumer(a.cuda(), b.cuda(), c, flags, sizes, offsets, signals, world, num_sms, 256, 224, 64, 8,
                      cum_tiles=M * N, visit_log=log, two_stage=two_stage, ring_pipe=(K == 512))
        check_status()
        assert _max_rel_err(c, numerics.gemm_fp32(a, b)) <= REL_TOL
        _check_visits(log, sizes, offsets, signals, M, N, 256, 224, 8, num_sms, M * N, True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("BM,BN,eight", [(256, 256, False), (256, 256, True), (256, 224, False), (128, 256, True),
                                         (256, 128, True), (128, 256, False), (256, 128, False), (128, 128, False)])
def test_both_mfma_forms_of_the_k_loop(hip, dtype, BM, BN, eight):
    """The default K loops (two LDS stages with early reads, or three stages) run on 16x16x32 MFMAs and on
    32x32x16 ones on request: both against fp32, the same visit order, and the same bits (K of one,
    two, three and eight slabs; consumer and producer)."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_consumer, gemm_producer

    world, rank = 2, 1
    M, N = 1024, 2 * BN * (2 if BN < 224 else 1)
    for K, num_sms in ((64, 5), (128, 256), (192, 3), (512, 16)):
        a, b = _inputs(M, N, K, dtype, seed=K + BM + BN)
        sizes, offsets, signals = _row_waves(M, N, world, rank)
        ref = numerics.gemm_fp32(a, b)
        ad, bd = a.cuda(), b.cuda()
        flags = torch.ones(world, dtype=torch.int64, device="cuda")
        tiles = (M // BM) * (N // BN)
        results = []
        for wide in (False, True):
            c = torch.zeros(M, N, dtype=dtype, device="cuda")
            log = torch.full((tiles, 4), -1, dtype=torch.int32, device="cuda")
            gemm_consumer(ad, bd, c, flags, sizes, offsets, signals, world, num_sms, BM, BN, 64, 8, cum_tiles=M * N,
                          visit_log=log, eight_waves=eight, mfma_32x32=wide)
            check_status()
            assert _max_rel_err(c, ref) <= REL_TOL, (K, wide)
            _check_visits(log, sizes, offsets, signals, M, N, BM, BN, 8, num_sms, M * N, True)
            results.append(c)
            p_flags = torch.zeros(world, dtype=torch.int64, device="cuda")
            counters = torch.zeros(world, dtype=torch.int32, device="cuda")
            cp = torch.zeros(M, N, dtype=dtype, device="cuda")
            gemm_producer(ad, bd, cp, p_flags, sizes, offsets, [0, 1], num_sms, BM, BN, cum_tiles=M * N,
                          counter_buffer=counters, eight_waves=eight, mfma_32x32=wide)
            check_status()
            assert p_flags.tolist() == [1, 1]
            results.append(cp)
        for other in results[1:]:
            assert torch.equal(results[0], other), K


def test_launch_on_a_stream_that_is_not_current(hip):
    """`stream=` with tables given as lists and no counter buffer: the device tables and the
    zeroed counters the launcher creates must be filled on that stream, ahead of the kernel.
    The stream is kept busy first so that a fill on the wrong stream would overtake nothing."""
    from syncopate_amd import _lib
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_consumer, gemm_producer

    M, N, K, world, rank = 1024, 512, 256, 4, 1
    a, b = _inputs(M, N, K, torch.bfloat16, seed=11)
    ad, bd = a.cuda(), b.cuda()
    ref = numerics.gemm_fp32(a, b)
    rows = M // world
    sizes = [[rows, N]] * world
    offsets = [[((rank + k + 1) % world) * rows, 0] for k in range(world)]
    side = torch.cuda.Stream()
    for trial in range(3):
        flags = torch.zeros(world, dtype=torch.int64, device="cuda")
        c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
        torch.cuda.synchronize()
        _lib.check("syn_delay_us", hip.syn_delay_us(2000, _lib.stream_handle(side)))
        gemm_producer(ad, bd, c, flags, sizes, offsets, list(range(world)), 64, 128, 128, cum_tiles=M * N,
                      stream=side)
        c2 = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
        side.wait_stream(torch.cuda.current_stream())       # c2's fill
        gemm_consumer(ad, bd, c2, flags, sizes, offsets, list(range(world)), world, 64, 128, 128, cum_tiles=M * N,
                      stream=side)
        # churn the allocator on the current stream while the side stream is still busy
        junk = [torch.full((world,), 7, dtype=torch.int32, device="cuda") for _ in range(8)]
        del junk
        side.synchronize()
        check_status()
        assert flags.tolist() == [1] * world
        assert _max_rel_err(c, ref) <= REL_TOL
        assert torch.equal(c, c2)


@pytest.mark.parametrize("producer", [False, True])
def test_more_waves_than_the_kernel_keeps_in_lds(hip, producer):
    """The walk keeps the first 128 rows of the wave tables in LDS and reads the rest from memory: 200 waves of one
    tile row each, in a shuffled order, every wave behind its own flag; visit log against the oracle's walk, product
    against fp32, and (producer) every wave's counter and flag."""
    import numpy as np

    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm, gemm_producer

    waves, BM, BN, K, N = 200, 128, 256, 128, 512
    M = waves * BM
    order = np.random.default_rng(5).permutation(waves).tolist()
    sizes = [[BM, N]] * waves
    offsets = [[o * BM, 0] for o in order]
    signals = list(range(waves))
    a, b = _inputs(M, N, K, torch.bfloat16, seed=9)
    ref = numerics.gemm_fp32(a, b)
    c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    tiles = (M // BM) * (N // BN)
    log = torch.full((tiles, 4), -1, dtype=torch.int32, device="cuda")
    if producer:
        flags = torch.zeros(waves, dtype=torch.int64, device="cuda")
        counters = torch.zeros(waves, dtype=torch.int32, device="cuda")
        gemm_producer(a.cuda(), b.cuda(), c, flags, sizes, offsets, signals, 7, BM, BN, 64, 8, cum_tiles=M * N,
                      counter_buffer=counters, visit_log=log, xcd_remap=False)
        check_status()
        assert flags.tolist() == [1] * waves and counters.tolist() == [N // BN] * waves
    else:
        flags = torch.ones(waves, dtype=torch.int64, device="cuda")
        gemm(a.cuda(), b.cuda(), c, 1, 7, BM, BN, 64, 8, cur_wave_sizes=sizes, wave_offsets=offsets, signal_ptr=flags,
             signal_offsets=signals, cum_tiles=M * N, visit_log=log, xcd_remap=False)
        check_status()
    assert _max_rel_err(c, ref) <= REL_TOL
    want = visit_order.gemm_tile_visits(sizes, offsets, signals, M=M, N=N, BM=BM, BN=BN, group_m=8, num_sms=7,
                                        cum_tiles=M * N)
    got = log.cpu().tolist()
    for v in want:
        assert tuple(got[v["tile_id"]][1:]) == (v["wave"], v["pid_m"], v["pid_n"]), v
