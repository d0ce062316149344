"""The headline configurations at their full sizes, checked through properties that do not need a
CPU pass over the whole problem: the tile-visit log against the oracle (integer work, cheap at
any size), sampled rows against torch's fp32 matmul / attention on the GPU (library routines),
bitwise agreement between launch configurations, counters and flags, invariance of attention
under the arrival order of the kv chunks."""

import pytest
import torch

from oracle import visit_order

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def _rel(out, ref):
    return ((out.float() - ref.float()).abs().max() / ref.float().abs().max()).item()


def _check_visit_log(log, sizes, offsets, signals, M, N, BM, BN, num_sms):
    want = visit_order.gemm_tile_visits(sizes, offsets, signals, M=M, N=N, BM=BM, BN=BN, group_m=8,
                                        num_sms=num_sms, cum_tiles=M * N)
    got = log.cpu().view(-1, 4).tolist()
    assert len(want) == (M // BM) * (N // BN)
    for v in want:
        assert got[v["tile_id"]] == [v["pid"], v["wave"], v["pid_m"], v["pid_n"]], v


def test_ag_gemm_8192x8192x3584(hip):
    """AG+GEMM of rank 0 of 8 (chunks of 1024 rows in swizzled order), every chunk resident."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_consumer

    M, K, N, world, rank = 8192, 8192, 3584, 8, 0
    g = torch.Generator(device="cuda").manual_seed(0)
    a = (0.02 * torch.randn(M, K, device="cuda", generator=g)).bfloat16()
    b = (0.02 * torch.randn(N, K, device="cuda", generator=g)).bfloat16()
    rows = M // world
    sizes = [[rows, N]] * world
    offsets = [[((rank + k) % world) * rows, 0] for k in range(world)]
    signals = [-1] + list(range(world - 1))
    flags = torch.ones(world - 1, dtype=torch.int64, device="cuda")
    sample = torch.arange(5, M, 389, device="cuda")
    ref = a[sample].float() @ b.float().t()

    outputs = []
    # (BM, BN, programs, 8 wavefronts, ring pipeline, 32x32x16 MFMAs in the default pipelines)
    for BM, BN, num_sms, eight, ring, wide in [(256, 256, 224, False, False, False), (256, 256, 256, True, False, False),
                                               (256, 256, 131, True, True, False), (256, 256, 224, False, False, True),
                                               (128, 256, 224, False, False, False), (128, 256, 97, False, False, True)]:
        c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
        log = torch.full(((M // BM) * (N // BN), 4), -1, dtype=torch.int32, device="cuda")
        gemm_consumer(a, b, c, flags, sizes, offsets, signals, world, num_sms, BM, BN, 64, 8,
                      cum_tiles=M * N, visit_log=log, xcd_remap=False, eight_waves=eight, ring_pipe=ring, mfma_32x32=wide)
        check_status()
        assert _rel(c[sample], ref) <= REL_TOL
        _check_visit_log(log, sizes, offsets, signals, M, N, BM, BN, num_sms)
        outputs.append((BM, BN, c))
    # one tile shape -> one order of the fp32 sums, whatever the grid, workgroup shape, pipeline or MFMA form
    for shape in ((256, 256), (128, 256)):
        same_tile = [c for BM, BN, c in outputs if (BM, BN) == shape]
        assert len(same_tile) >= 2
        for other in same_tile[1:]:
            assert torch.equal(same_tile[0], other)
    # other tile shapes rotate the K walk differently: equal to rounding
    assert _rel(outputs[-1][2], outputs[0][2]) <= 2e-2


def test_gemm_rs_producer_8192x8192x3584(hip):
    """GEMM+RS producer of rank 0 of 8: partial C (8192, 8192) written in wave order
    1, 2, ..., 7, 0; counters and flags complete; then the chunked reduce over 8 partials."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_producer
    from syncopate_amd.computation.reduce import ring_reduce

    M, K, N, world, rank, BM, BN = 8192, 3584, 8192, 8, 0, 256, 256
    g = torch.Generator(device="cuda").manual_seed(0)
    a = (0.02 * torch.randn(M, K, device="cuda", generator=g)).bfloat16()
    b = (0.02 * torch.randn(N, K, device="cuda", generator=g)).bfloat16()
    rows = M // world
    order = [(rank + k + 1) % world for k in range(world)]
    sizes = [[rows, N]] * world
    offsets = [[ch * rows, 0] for ch in order]
    signals = list(range(world))
    flags = torch.zeros(world, dtype=torch.int64, device="cuda")
    counters = torch.zeros(world, dtype=torch.int32, device="cuda")
    c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    log = torch.full(((M // BM) * (N // BN), 4), -1, dtype=torch.int32, device="cuda")
    gemm_producer(a, b, c, flags, sizes, offsets, signals, 224, BM, BN, 64, 8, cum_tiles=M * N,
                  counter_buffer=counters, visit_log=log, xcd_remap=False)
    check_status()
    assert counters.tolist() == [(rows // BM) * (N // BN)] * world
    assert flags.tolist() == [1] * world
    assert not torch.isnan(c).any()
    sample = torch.arange(3, M, 411, device="cuda")
    assert _rel(c[sample], a[sample].float() @ b.float().t()) <= REL_TOL
    _check_visit_log(log, sizes, offsets, signals, M, N, BM, BN, 224)

    # the reduce at its full size: own block of the partial plus 7 received partials
    recv = torch.randn(world, rows, N, device="cuda", generator=g).bfloat16()
    out = torch.empty(rows, N, dtype=torch.bfloat16, device="cuda")
    ring_reduce(recv, out, c, rank)
    acc = c[rank * rows:(rank + 1) * rows].clone()
    for i in range(1, world):
        acc = acc + recv[(rank + i) % world]          # torch adds bf16 tensors with one rounding per add
    assert torch.equal(out, acc)


def _attn_tables(B, H, Sq, chunk, order, signals):
    offsets = [[0, 0, 0, o * chunk] for o in order]
    sizes = [[B, H, Sq, chunk]] * len(order)
    cums = [(i + 1) * B * H * Sq for i in range(len(order))]
    return dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_offsets=signals,
                cum_tiles=cums[-1])


def test_allgather_attention_4096x32768_double_ring_order(hip):
    """AG attention of rank 0 of 8: the local 4096 q rows against 32768 kv rows arriving as 8
    chunks in double-ring order; sampled heads against torch's attention in fp32 on the GPU, and
    the same result (to rounding) for a different arrival order."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    B, H, Sq, Skv, D, chunks = 1, 32, 4096, 32768, 128, 8
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(B, H, Sq, D, device="cuda", generator=g).bfloat16()
    k = torch.randn(B, H, Skv, D, device="cuda", generator=g).bfloat16()
    v = torch.randn(B, H, Skv, D, device="cuda", generator=g).bfloat16()
    flags = torch.ones(chunks, dtype=torch.int64, device="cuda")
    scale = D ** -0.5
    ring = _attn_tables(B, H, Sq, Skv // chunks, [0, 1, 7, 6, 4, 5, 3, 2], [-1, 0, 4, 1, 5, 2, 6, 3])
    o, lse = attention_forward(q, k, v, scale, signal_ptr=flags, return_lse=True, **ring)
    check_status()
    for h in (0, 13, 31):
        s = (q[0, h].float() @ k[0, h].float().t()) * scale
        ref = torch.softmax(s, dim=-1) @ v[0, h].float()
        assert _rel(o[0, h], ref) <= REL_TOL
        assert (lse[0, h] - torch.logsumexp(s, dim=-1) / 0.6931471805599453).abs().max().item() <= 2e-2
    plain = _attn_tables(B, H, Sq, Skv // chunks, list(range(chunks)), [-1] + list(range(chunks - 1)))
    o2 = attention_forward(q, k, v, scale, signal_ptr=flags, num_programs=512, **plain)
    check_status()
    # two results that are each within REL_TOL of the fp32 value (the partial O is rounded to bf16 at
    # every merge, as in the reference) are within twice that of each other
    assert _rel(o2, o) <= 2 * REL_TOL
    for h in (5, 22):
        s = (q[0, h].float() @ k[0, h].float().t()) * scale
        assert _rel(o2[0, h], torch.softmax(s, dim=-1) @ v[0, h].float()) <= REL_TOL


def test_all2all_attention_16384_causal(hip):
    """Ulysses-style attention over the whole sequence (S = 16384, 4 local heads), kv in 8 chunks
    of 2048, causal; against torch's causal attention on sampled heads."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    B, H, S, D, chunks = 1, 4, 16384, 128, 8
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(B, H, S, D, device="cuda", generator=g).bfloat16()
    k = torch.randn(B, H, S, D, device="cuda", generator=g).bfloat16()
    v = torch.randn(B, H, S, D, device="cuda", generator=g).bfloat16()
    flags = torch.ones(chunks, dtype=torch.int64, device="cuda")
    scale = D ** -0.5
    tables = _attn_tables(B, H, S, S // chunks, list(range(chunks)), list(range(chunks)))
    for causal in (True, False):
        o = attention_forward(q, k, v, scale, signal_ptr=flags, causal=causal, **tables)
        check_status()
        for h in (0, 3):
            s = (q[0, h].float() @ k[0, h].float().t()) * scale
            if causal:
                s = s.masked_fill(torch.ones(S, S, dtype=torch.bool, device="cuda").triu(1), float("-inf"))
            ref = torch.softmax(s, dim=-1) @ v[0, h].float()
            assert _rel(o[0, h], ref) <= REL_TOL
            del s, ref


def test_all2all_attention_16384_on_the_64_wave_table(hip):
    """The table the benchmark times: 8 arrivals of (Q, K, V) chunks of 2048 rows expanded to 64 waves
    (tests/test_all2all_attn_transform.py:58-117), 4 local heads, causal and not.  The planned launch (one
    program per compute unit, segments of visits to the same q blocks) and the launcher's automatic choice, both
    against torch's attention in fp32 on every head; the visit log of the planned launch against the oracle's
    tile -> work mapping, all 4096 tiles."""
    from oracle import visit_order
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward, plan_attention_work
    from syncopate_amd.communication.code_gen import CommGenerator
    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan_dim
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules
    from syncopate_amd.interface.wave_tables import all2all_attn_tables

    world, H, chunk, D = 8, 4, 2048, 128
    S = world * chunk
    # rank 0's tables from the plan, as the reference's test derives them
    plans = {r: build_all_to_all_plan_dim(shape=(3, 1, H * world, chunk, D), dtype=torch.bfloat16, mesh_size=world,
                                          rank=r, src_buffer="src", dst_buffer="dst", src_split_axis=3,
                                          dst_split_axis=2, transfer_kind="pull", compute_producer=False)
             for r in range(world)}
    gen = CommGenerator(plans)
    gen.plan_signals()
    host = all2all_attn_tables(lower_comm_plan_to_raw_schedules(gen)[0]["dst"], {"batch": 1, "head": 2, "seq": 3})
    offsets, sizes, cums, signals, total = (host.wave_offsets, host.wave_sizes, host.cum_wave_sizes,
                                            host.signal_offsets, host.cum_tiles)
    assert len(cums) == 64 and total // 128 == 4096 and max(signals) + 1 == world
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn(1, H, S, D, device="cuda", generator=g).bfloat16() for _ in range(3))
    flags = torch.ones(world, dtype=torch.int64, device="cuda")
    tables = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_offsets=signals, cum_tiles=total)
    refs = {}
    for causal in (True, False):
        for h in range(H):
            s = (q[0, h].float() @ k[0, h].float().t()) * D ** -0.5
            if causal:
                s = s.masked_fill(torch.ones(S, S, dtype=torch.bool, device="cuda").triu(1), float("-inf"))
            refs[causal, h] = torch.softmax(s, dim=-1) @ v[0, h].float()
            del s
    log = torch.full((total // 128, 8), -1, dtype=torch.int32, device="cuda")
    for causal in (True, False):
        for max_visits in (2, None):
            plan = plan_attention_work(offsets, sizes, cums, causal=causal, num_programs=256, max_visits=max_visits,
                                       list_masked_visits=True)
            log.fill_(-1)
            o = attention_forward(q, k, v, D ** -0.5, signal_ptr=flags, causal=causal, pair_q_blocks=True,
                                  xcd_remap=True, work_plan=plan, visit_log=log, **tables)
            check_status()
            for h in range(H):
                assert _rel(o[0, h], refs[causal, h]) <= REL_TOL, (causal, max_visits, h)
            for t, got in enumerate(log.cpu().tolist()):
                w = visit_order.attn_tile_work(t, offsets, sizes, cums, signals)
                assert got[:7] == [w["wave"], w["z"], w["h"], w["q_block"], w["kv_lo"], w["kv_hi"], w["signal"]], t
        # what attention() and form="auto" pick for these tables
        o = attention_forward(q, k, v, D ** -0.5, signal_ptr=flags, causal=causal, form="auto", **tables)
        check_status()
        for h in range(H):
            assert _rel(o[0, h], refs[causal, h]) <= REL_TOL, (causal, "auto", h)


def test_c1_mesh4_fp16_gathered_4096x512_times_512x1024(hip):
    """The reference's own CPU-runnable case on the HIP consumer: mesh of 4, 1-D swizzle pull,
    per-rank A (1024, 512) fp16 gathered to (4096, 512), B (512, 1024), seed 0; every rank's wave
    tables are the golden schedule the reference's compiler gives for this plan
    (tests/golden/host_compiler.json, case ag_swizzle_pull_c1_gathered).  Result against the
    fp32 matmul of the same fp16 values, visit log against the oracle, every rank, resident and
    with the chunks arriving behind flags on a side stream."""
    import json
    import os

    from oracle import numerics
    from syncopate_amd import _lib
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_consumer

    golden = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "host_compiler.json")))
    schedules = golden["ag_swizzle_pull_c1_gathered"]["schedules"]
    world, rows, K, N = 4, 1024, 512, 1024
    M = world * rows
    torch.manual_seed(0)
    a = torch.cat([torch.randn(rows, K).half() for _ in range(world)])      # generated in rank order
    b = torch.randn(K, N).half()
    ref = numerics.gemm_fp32(a, b.t().contiguous())
    ad, b_nk = a.cuda(), b.t().contiguous().cuda()
    side = pick_side_streams(1)[0]
    for rank in range(world):
        sched = schedules[str(rank)]["a"]
        assert sched["global_shape"] == [M, K]
        offsets = [[o[0], 0] for o in sched["offsets"]]
        sizes = [[s[0], N] for s in sched["shapes"]]
        signals = sched["signals"]
        assert [o[0] for o in offsets] == [((rank + k) % world) * rows for k in range(world)]
        for BM, BN, num_sms in [(128, 128, 256), (256, 256, 48)]:
            flags = torch.ones(world - 1, dtype=torch.int64, device="cuda")
            c = torch.zeros(M, N, dtype=torch.float16, device="cuda")
            log = torch.full(((M // BM) * (N // BN), 4), -1, dtype=torch.int32, device="cuda")
            gemm_consumer(ad, b_nk, c, flags, sizes, offsets, signals, world, num_sms, BM, BN, 64, 8,
                          cum_tiles=M * N, visit_log=log)
            check_status()
            assert _rel(c.cpu(), ref) <= REL_TOL
            _check_visit_log(log, sizes, offsets, signals, M, N, BM, BN, num_sms)
        # gated: the symmetric buffer holds the own shard only (the rest poisoned); peers' chunks
        # arrive on a side stream in schedule order, copy then flag
        symm = torch.full((M, K), float("nan"), dtype=torch.float16, device="cuda")
        symm[rank * rows:(rank + 1) * rows].copy_(ad[rank * rows:(rank + 1) * rows])
        flags = torch.zeros(world - 1, dtype=torch.int64, device="cuda")
        c_gated = torch.zeros(M, N, dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        side.wait_stream(torch.cuda.current_stream())
        gemm_consumer(symm, b_nk, c_gated, flags, sizes, offsets, signals, world, 48, 256, 256, 64, 8,
                      cum_tiles=M * N, spin_timeout_us=3_000_000)
        nbytes = rows * K * 2
        for wave in range(1, world):
            row0 = offsets[wave][0]
            _lib.check("syn_delay_us", hip.syn_delay_us(50, _lib.stream_handle(side)))
            _lib.check("syn_copy_async", hip.syn_copy_async(symm.data_ptr() + row0 * K * 2, ad.data_ptr() + row0 * K * 2,
                                                            nbytes, _lib.stream_handle(side)))
            _lib.check("syn_flag_set", hip.syn_flag_set(flags.data_ptr() + 8 * signals[wave], 1, _lib.stream_handle(side)))
        torch.cuda.current_stream().wait_stream(side)
        check_status()
        assert torch.equal(c_gated, c)          # same tile shape: bitwise the resident result


def test_allgather_attention_full_size_with_chunks_arriving_behind_flags(hip):
    """The all-gather attention configuration at its full size with real gating: only the rank's own
    kv chunk is resident (the rest of the buffer is NaN), the other seven are copied in on a side
    stream in double-ring arrival order - a box copy on 32 compute units, then the chunk's flag -
    while 224 persistent workgroups (two q blocks each) already run.  Sampled heads against torch's
    attention in fp32 on the GPU; the gathered buffer bit for bit."""
    from syncopate_amd import _lib
    from syncopate_amd.communication.comm_runtime.persistent_copy import persistent_copy_last_contig
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    B, H, Sq, Skv, D, chunks = 1, 32, 4096, 32768, 128, 8
    g = torch.Generator(device="cuda").manual_seed(1)
    q = torch.randn(B, H, Sq, D, device="cuda", generator=g).bfloat16()
    kv = torch.randn(2, B, H, Skv, D, device="cuda", generator=g).bfloat16()
    chunk = Skv // chunks
    arrival, signals = [0, 1, 7, 6, 4, 5, 3, 2], [-1, 0, 4, 1, 5, 2, 6, 3]
    tables = _attn_tables(B, H, Sq, chunk, arrival, signals)
    buf = torch.full_like(kv, float("nan"))
    buf[:, :, :, :chunk].copy_(kv[:, :, :, :chunk])
    flags = torch.zeros(chunks, dtype=torch.int64, device="cuda")
    main = torch.cuda.current_stream()
    side = pick_side_streams(1, main, torch.device("cuda", torch.cuda.current_device()))[0]
    torch.cuda.synchronize()
    side.wait_stream(main)
    with torch.cuda.stream(side):
        for wave in range(1, chunks):
            c = arrival[wave]
            _lib.check("syn_delay_us", hip.syn_delay_us(100, _lib.stream_handle(side)))
            persistent_copy_last_contig(kv[:, :, :, c * chunk:(c + 1) * chunk], buf[:, :, :, c * chunk:(c + 1) * chunk],
                                        num_sms=32)
            _lib.check("syn_flag_set", hip.syn_flag_set(flags.data_ptr() + 8 * signals[wave], 1, _lib.stream_handle(side)))
    o = attention_forward(q, buf[0], buf[1], D ** -0.5, signal_ptr=flags, pair_q_blocks=True, num_programs=224,
                          spin_timeout_us=5_000_000, **tables)
    main.wait_stream(side)
    check_status()
    assert flags.tolist()[:7] == [1] * 7
    assert torch.equal(buf, kv)
    assert not torch.isnan(o).any()
    for h in (0, 17, 31):
        s = (q[0, h].float() @ kv[0, 0, h].float().t()) * D ** -0.5
        assert _rel(o[0, h], torch.softmax(s, dim=-1) @ kv[1, 0, h].float()) <= REL_TOL


def test_allgather_attention_full_size_chained(hip):
    """The same configuration in the chained form (512 programs, each walking its two q blocks through the
    eight chunks with the sums in registers): resident, against fp32 on sampled heads, against the form
    that merges after every tile, and the visit log of all 8192 tiles against the oracle; then gated on a
    device split by compute-unit masks - the waiting programs hold their compute units, so the stand-in
    producer's copy kernels get 32 units of their own - with the rest of the buffer NaN until it is copied."""
    from oracle import visit_order
    from syncopate_amd import _lib
    from syncopate_amd.communication.comm_runtime.cu_partition import split_device_cu_mask
    from syncopate_amd.communication.comm_runtime.persistent_copy import persistent_copy_last_contig
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    B, H, Sq, Skv, D, chunks = 1, 32, 4096, 32768, 128, 8
    g = torch.Generator(device="cuda").manual_seed(2)
    q = torch.randn(B, H, Sq, D, device="cuda", generator=g).bfloat16()
    kv = torch.randn(2, B, H, Skv, D, device="cuda", generator=g).bfloat16()
    chunk = Skv // chunks
    arrival, signals = [0, 1, 7, 6, 4, 5, 3, 2], [-1, 0, 4, 1, 5, 2, 6, 3]
    tables = _attn_tables(B, H, Sq, chunk, arrival, signals)
    ones = torch.ones(chunks, dtype=torch.int64, device="cuda")
    tiles = tables["cum_tiles"] // 128
    pairs_per_wave = B * H * Sq // 256
    log = torch.full((tiles, 8), -1, dtype=torch.int32, device="cuda")
    o = attention_forward(q, kv[0], kv[1], D ** -0.5, signal_ptr=ones, pair_q_blocks=True, chain_q_blocks=True,
                          xcd_remap=True, visit_log=log, **tables)
    check_status()
    refs = {}
    for h in (0, 17, 31):
        s = (q[0, h].float() @ kv[0, 0, h].float().t()) * D ** -0.5
        refs[h] = torch.softmax(s, dim=-1) @ kv[1, 0, h].float()
        assert _rel(o[0, h], refs[h]) <= REL_TOL
        del s
    merged = attention_forward(q, kv[0], kv[1], D ** -0.5, signal_ptr=ones, pair_q_blocks=True, num_programs=256,
                               xcd_remap=True, **tables)
    check_status()
    assert _rel(merged, o) <= 2 * REL_TOL
    got = log.cpu().tolist()
    for tile_id in range(0, tiles, 7):
        exp = visit_order.attn_tile_work(tile_id, tables["wave_offsets"], tables["wave_sizes"], tables["cum_wave_sizes"],
                                         signals)
        assert got[tile_id][:7] == [exp["wave"], exp["z"], exp["h"], exp["q_block"], exp["kv_lo"], exp["kv_hi"],
                                    exp["signal"]]
    programs = [rec[7] for rec in got[0::2]]
    assert sorted(programs[:pairs_per_wave]) == list(range(pairs_per_wave))
    assert programs == programs[:pairs_per_wave] * chunks            # a program's pair is the same in every wave

    (comm, rest), sizes = split_device_cu_mask(torch.device("cuda", torch.cuda.current_device()), 1, 32)
    assert sizes == [32, 224]
    buf = torch.full_like(kv, float("nan"))
    buf[:, :, :, :chunk].copy_(kv[:, :, :, :chunk])
    flags = torch.zeros(chunks, dtype=torch.int64, device="cuda")
    out = torch.empty_like(q)
    torch.cuda.synchronize()
    with torch.cuda.stream(comm):
        for wave in range(1, chunks):
            c = arrival[wave]
            _lib.check("syn_delay_us", hip.syn_delay_us(100, _lib.stream_handle(comm)))
            persistent_copy_last_contig(kv[:, :, :, c * chunk:(c + 1) * chunk], buf[:, :, :, c * chunk:(c + 1) * chunk],
                                        num_sms=32, stream=comm)
            _lib.check("syn_flag_set", hip.syn_flag_set(flags.data_ptr() + 8 * signals[wave], 1, _lib.stream_handle(comm)))
    attention_forward(q, buf[0], buf[1], D ** -0.5, signal_ptr=flags, pair_q_blocks=True, chain_q_blocks=True,
                      xcd_remap=True, spin_timeout_us=5_000_000, out=out, stream=rest, **tables)
    torch.cuda.synchronize()
    check_status()
    assert flags.tolist()[:7] == [1] * 7
    assert torch.equal(buf, kv)
    assert not torch.isnan(out).any()
    for h, ref in refs.items():
        assert _rel(out[0, h], ref) <= REL_TOL

