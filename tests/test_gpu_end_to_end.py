"""Fused iterations on one MI355X, from plan builder to kernel: the op list of one rank is
replayed on side streams by CommContext (the other ranks of the mesh are buffers of the same
process) while the chunk-scheduled kernel runs on the compute stream.  The flows follow the
reference's distributed scripts: tests/test_gemm_rs.py:196-233,
tests/test_allgather_attn_transform.py:94-105 and tests/test_all2all_attn_transform.py:118-146.
"""

import numpy as np
import pytest
import torch

from oracle import numerics

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def _rel(out, ref):
    return ((out.float().cpu() - ref.float()).abs().max() / ref.float().abs().max()).item()


def _compile(plans, options=None):
    from syncopate_amd.communication.code_gen import CommGenerator
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules

    gen = CommGenerator(plans)
    gen.plan_signals()
    schedules = lower_comm_plan_to_raw_schedules(gen)
    info = gen.generate_code_for_plan(options) if options is not None else gen.generate_code_for_plan()
    info.local_world_size = info.world_size
    return schedules, info


@pytest.mark.parametrize("rank,shape,copy_units", [(0, (4, 1024, 512, 256, 128, 128, 13), 0),
                                                   (2, (4, 1024, 512, 256, 128, 128, 13), 0),
                                                   (5, (8, 8192, 4096, 512, 256, 256, 224), 0),
                                                   (1, (4, 1024, 512, 256, 128, 128, 13), 8)])
def test_gemm_rs_iteration(hip, rank, shape, copy_units):
    """Producer GEMM -> comm stream waits on each wave's COMPUTE_DONE flag and pushes the chunk
    to its owner -> ring reduce of the received partials.  With `copy_units` the pushes are box
    copies on that many compute units instead of copy-engine ops (CodeGenOptions(copy_engine=False),
    tests/test_gemm_rs_sm.py:92-135)."""
    from syncopate_amd.communication.code_gen import CodeGenOptions
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_producer
    from syncopate_amd.computation.reduce import ring_reduce_tma
    from syncopate_amd.interface.wave_tables import gemm_producer_tables

    world, M, N, K, BM, BN, programs = shape
    rows = M // world
    g = torch.Generator().manual_seed(11 + rank)
    a = (0.1 * torch.randn(M, K, generator=g)).bfloat16()
    b = (0.1 * torch.randn(N, K, generator=g)).bfloat16()
    peer_partials = (0.5 * torch.randn(world, rows, N, generator=g)).bfloat16()

    plans = {r: build_all_to_all_plan(shape=(M, N), dtype=torch.bfloat16, mesh_size=world, rank=r,
                                      src_buffer="src", dst_buffer="dst", transfer_kind="push",
                                      compute_producer=True) for r in range(world)}
    schedules, info = _compile(plans, CodeGenOptions(copy_engine=False) if copy_units else None)
    if copy_units:
        info.num_copy_sms = copy_units
    tables = gemm_producer_tables(schedules[rank]["src"])
    # the chunk a peer owns is computed (and shipped) before the rank's own chunk
    assert [off[0] // rows for off in tables.block_offsets] == [(rank + 1 + i) % world for i in range(world)]

    ctx = CommContext(rank, info)
    src = ctx.comm_buffers["src"][rank]
    dst = ctx.comm_buffers["dst"][rank]
    src.fill_(float("nan"))          # a chunk shipped before its tiles were stored would carry NaNs
    dst.copy_(peer_partials.cuda())  # what the peers pushed (they are not replayed here)
    ad, bd = a.cuda(), b.cuda()
    out = torch.empty(rows, N, dtype=torch.bfloat16, device="cuda")
    comm_stream = torch.cuda.Stream()
    main = torch.cuda.current_stream()

    ctx.reset_signals()
    comm_stream.wait_stream(main)
    gemm_producer(ad, bd, src, ctx.compute_signal_bufs[rank], tables.block_shapes, tables.block_offsets,
                  tables.signal_offsets, programs, BM, BN, 64, 8, cum_tiles=tables.cum_tiles)
    ctx.start_after(comm_stream)
    ctx.execute(neglect_local=True)
    ctx.end_before(comm_stream)
    main.wait_stream(comm_stream)
    ring_reduce_tma(dst, out, src, rank)
    check_status()
    ctx.check_status()

    partial = numerics.gemm_fp32(a, b)
    assert _rel(src, partial) <= REL_TOL
    assert ctx.compute_signal_bufs[rank].tolist() == [1] * world
    for peer in range(world):
        if peer == rank:
            continue
        # the peer's slot `rank` holds the rows it owns of this rank's partial result, bit for bit
        got = ctx.comm_buffers["dst"][peer][rank]
        assert torch.equal(got, src[peer * rows:(peer + 1) * rows])
        peer_flags = ctx.recv_signal_bufs[peer].tolist()
        assert sum(peer_flags) == 1
    # neglect_local drops the local copy only: its flag is still written
    assert ctx.recv_signal_bufs[rank].sum().item() == 1
    assert torch.equal(dst.cpu(), peer_partials)
    want = numerics.ring_reduce(dst.float().cpu().numpy(), src.float().cpu().numpy(), rank, dtype="bf16")
    assert np.array_equal(out.float().cpu().numpy(), want)
    total = partial[rank * rows:(rank + 1) * rows].double()
    for peer in range(world):
        if peer != rank:
            total = total + peer_partials[peer].double()
    assert _rel(out, total) <= 2e-2


@pytest.mark.parametrize("rank", [0, 3])
def test_allgather_gemm_reduce_scatter_in_one_kernel(hip, rank):
    """One GEMM in both roles between two plans: the row chunks of A arrive by all-gather (copy,
    then flag, on side streams), the GEMM waits for a chunk's flag before the wave that reads it,
    and every finished wave's rows of the partial result are pushed to their owner behind the
    wave's COMPUTE_DONE flag.  The waves follow the producer's order (peers' chunks first), so the
    first wave already waits for a remote chunk."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_gather_plan_1d_swizzle, build_all_to_all_plan
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm
    from syncopate_amd.interface.wave_tables import gemm_consumer_tables, gemm_producer_tables

    world, M, N, K, BM, BN, programs = 4, 1024, 512, 256, 128, 128, 13
    rows = M // world
    g = torch.Generator().manual_seed(21 + rank)
    a = (0.1 * torch.randn(M, K, generator=g)).bfloat16()
    b = (0.1 * torch.randn(N, K, generator=g)).bfloat16()

    gather_plans = {r: build_all_gather_plan_1d_swizzle((M, K), torch.bfloat16, 0, world, r, "a", "pull")
                    for r in range(world)}
    gather_schedules, gather_info = _compile(gather_plans)
    scatter_plans = {r: build_all_to_all_plan(shape=(M, N), dtype=torch.bfloat16, mesh_size=world, rank=r,
                                              src_buffer="src", dst_buffer="dst", transfer_kind="push",
                                              compute_producer=True) for r in range(world)}
    scatter_schedules, scatter_info = _compile(scatter_plans)
    arrival = gemm_consumer_tables(gather_schedules[rank]["a"], N)        # which flag announces which row chunk
    flag_of_chunk = {off[0] // rows: sig for off, sig in zip(arrival.block_offsets, arrival.signal_offsets)}
    waves = gemm_producer_tables(scatter_schedules[rank]["src"])           # the kernel's waves, owner by owner
    wait_for = [flag_of_chunk[off[0] // rows] for off in waves.block_offsets]
    assert wait_for.count(-1) == 1 and wait_for[-1] == -1                  # only the rank's own chunk is resident

    gather = CommContext(rank, gather_info)
    scatter = CommContext(rank, scatter_info)
    for r in range(world):                 # every rank's symmetric buffer holds its own shard, NaN elsewhere
        gather.comm_buffers["a"][r].fill_(float("nan"))
        gather.comm_buffers["a"][r][r * rows:(r + 1) * rows].copy_(a[r * rows:(r + 1) * rows])
    src = scatter.comm_buffers["src"][rank]
    src.fill_(float("nan"))
    bd = b.cuda()
    counters = torch.zeros(world, dtype=torch.int32, device="cuda")
    comm_stream = torch.cuda.Stream()
    main = torch.cuda.current_stream()

    gather.reset_signals()
    scatter.reset_signals()
    comm_stream.wait_stream(main)
    gather.start_after(main)
    gather.execute()                       # ahead of the scatter's spinning waits on any queue they share
    gemm(gather.comm_buffers["a"][rank], bd, src, world, programs, BM, BN, 64, 8,
         cur_wave_sizes=waves.block_shapes, wave_offsets=waves.block_offsets,
         signal_ptr=scatter.compute_signal_bufs[rank], signal_offsets=waves.signal_offsets, counter_ptr=counters,
         consumer_signal_ptr=gather.recv_signal_bufs[rank], consumer_signal_offsets=wait_for,
         cum_tiles=waves.cum_tiles)
    scatter.start_after(comm_stream)
    scatter.execute(neglect_local=True)
    scatter.end_before(comm_stream)
    gather.end_before(main)
    main.wait_stream(comm_stream)
    check_status()
    gather.check_status()
    scatter.check_status()

    assert torch.equal(gather.comm_buffers["a"][rank].cpu(), a)
    partial = numerics.gemm_fp32(a, b)
    assert _rel(src, partial) <= REL_TOL
    assert scatter.compute_signal_bufs[rank].tolist() == [1] * world
    assert counters.tolist() == [(rows // BM) * (N // BN)] * world
    for peer in range(world):
        if peer != rank:
            assert torch.equal(scatter.comm_buffers["dst"][peer][rank], src[peer * rows:(peer + 1) * rows])


@pytest.mark.parametrize("rank,layout,form", [(1, "bhsd", {}), (3, "bhsd", {}), (2, "bshd", {}),
                                              (1, "bhsd", dict(pair_q_blocks=True, chain_q_blocks=True)),
                                              (2, "bshd", dict(pair_q_blocks=True, chain_q_blocks=True, xcd_remap=True))],
                         ids=lambda x: "+".join(x) if isinstance(x, dict) else str(x))
def test_allgather_attention_iteration(hip, rank, layout, form):
    """K/V chunks pulled from their owners on a side stream (copy, then flag) while the
    attention kernel walks the waves of the lowered schedule; the local Q attends to the whole
    sequence.  Also in the chained form, where a program goes from one chunk to the next behind its flag
    without writing its q blocks in between."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_gather_plan_1d_swizzle
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.interface.wave_tables import allgather_attn_tables, plan_layout_spec

    world, B, H, SEQ, D = 4, 1, 2, 1024, 128
    per_rank = SEQ // world
    shape, seq_axis, axes = plan_layout_spec(layout, B, H, SEQ, D)
    plans = {r: build_all_gather_plan_1d_swizzle(shape, torch.bfloat16, seq_axis, world, r, "kv", "pull")
             for r in range(world)}
    schedules, info = _compile(plans)
    tables = allgather_attn_tables(schedules[rank]["kv"], per_rank, axes)
    assert [off[3] // per_rank for off in tables.wave_offsets] == [(rank + i) % world for i in range(world)]
    assert tables.signal_offsets == [-1, 0, 1, 2]    # the rank's own chunk needs no flag

    g = torch.Generator().manual_seed(5)
    kv = torch.randn(*shape, generator=g).bfloat16()
    q = torch.randn(B, H, per_rank, D, generator=g).bfloat16()       # [B, H, S, D] whatever the layout
    ctx = CommContext(rank, info, link_delay_us=30)
    for r in range(world):                           # every simulated rank holds its own slice
        own = [slice(None)] * 5
        own[seq_axis] = slice(r * per_rank, (r + 1) * per_rank)
        ctx.comm_buffers["kv"][r][tuple(own)].copy_(kv[tuple(own)])
    buf = ctx.comm_buffers["kv"][rank]
    qd = q.cuda() if layout == "bhsd" else q.permute(0, 2, 1, 3).contiguous().cuda()
    tiles = tables.cum_tiles // 128
    log = torch.full((tiles, 8), -1, dtype=torch.int32, device="cuda")
    main = torch.cuda.current_stream()

    ctx.reset_signals()
    ctx.start_after(main)
    ctx.execute()
    out = attention_forward(qd, buf[0], buf[1], D ** -0.5, wave_offsets=tables.wave_offsets,
                            wave_sizes=tables.wave_sizes, cum_wave_sizes=tables.cum_wave_sizes,
                            signal_ptr=ctx.recv_signal_bufs[rank], signal_offsets=tables.signal_offsets,
                            NUM_WAVES=len(tables.signal_offsets), cum_tiles=tables.cum_tiles, visit_log=log,
                            layout=layout, **form)
    ctx.end_before(main)
    check_status()
    ctx.check_status()

    assert torch.equal(buf.cpu(), kv)                # the gather itself
    to_bhsd = (lambda t: t) if layout == "bhsd" else (lambda t: t.permute(0, 2, 1, 3))
    want = numerics.sdpa_fp32(q, to_bhsd(kv[0]), to_bhsd(kv[1]), D ** -0.5)
    assert _rel(to_bhsd(out), want) <= REL_TOL
    assert (log[:, 0] >= 0).all()                    # every tile of every wave ran


@pytest.mark.parametrize("kind,rank", [("ring", 1), ("double_ring", 2)])
def test_ring_allgather_attention_over_the_mesh(hip, kind, rank):
    """K/V forwarded round a ring, or round two nested rings, instead of pulled from their owners
    (tests/test_ring_allgather_attn_transform.py:160-230, tests/test_double_ring_ag_attn.py:160-230):
    a chunk reaches this rank only after its upstream neighbours have received and forwarded it,
    so every rank's op list is replayed; the attention kernel walks the waves in arrival order."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import (
        build_double_ring_all_gather_plan,
        build_ring_all_gather_plan,
    )
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.interface.wave_tables import allgather_attn_tables, plan_layout_spec

    world, B, H, SEQ, D = 4, 1, 2, 1024, 128
    per_rank = SEQ // world
    shape, seq_axis, axes = plan_layout_spec("bhsd", B, H, SEQ, D)
    if kind == "ring":
        plans = {r: build_ring_all_gather_plan(shape, torch.bfloat16, seq_axis, world, r, "kv") for r in range(world)}
    else:
        plans = {r: build_double_ring_all_gather_plan(shape, torch.bfloat16, seq_axis, world, 2, r, "kv")
                 for r in range(world)}
    schedules, info = _compile(plans)
    tables = allgather_attn_tables(schedules[rank]["kv"], per_rank, axes)
    arrival = [off[3] // per_rank for off in tables.wave_offsets]
    assert sorted(arrival) == list(range(world)) and arrival[0] == rank
    if kind == "ring":
        assert arrival == [(rank - k) % world for k in range(world)]
    assert tables.signal_offsets[0] == -1 and all(sig >= 0 for sig in tables.signal_offsets[1:])

    g = torch.Generator().manual_seed(15)
    kv = torch.randn(*shape, generator=g).bfloat16()
    q = torch.randn(B, H, per_rank, D, generator=g).bfloat16()
    ctx = CommContext(rank, info, link_delay_us=10)
    for r in range(world):
        own = [slice(None)] * 5
        own[seq_axis] = slice(r * per_rank, (r + 1) * per_rank)
        ctx.comm_buffers["kv"][r][tuple(own)].copy_(kv[tuple(own)])
    buf = ctx.comm_buffers["kv"][rank]
    main = torch.cuda.current_stream()

    ctx.reset_signals(whole_mesh=True)
    ctx.start_after(main)
    ctx.execute_mesh()
    out = attention_forward(q.cuda(), buf[0], buf[1], D ** -0.5, wave_offsets=tables.wave_offsets,
                            wave_sizes=tables.wave_sizes, cum_wave_sizes=tables.cum_wave_sizes,
                            signal_ptr=ctx.recv_signal_bufs[rank], signal_offsets=tables.signal_offsets,
                            NUM_WAVES=len(tables.signal_offsets), cum_tiles=tables.cum_tiles)
    ctx.end_before(main)
    check_status()
    ctx.check_status()

    for r in range(world):                           # the gather completed on every simulated rank
        assert torch.equal(ctx.comm_buffers["kv"][r].cpu(), kv), f"rank {r}"
    assert _rel(out, numerics.sdpa_fp32(q, kv[0], kv[1], D ** -0.5)) <= REL_TOL


def test_all2all_attention_iteration_with_graph_replay(hip):
    """Ulysses exchange of stacked Q/K/V captured as a HIP graph (the reference captures the
    comm side, tests/test_all2all_attn_transform.py:278) and replayed several times: every
    replay, with eager work and synchronisation in between, must gather the same bytes and give
    the same attention output as the eager run."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan_dim
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.interface.wave_tables import all2all_attn_tables

    world, rank, B, H, S_local, D = 4, 1, 1, 8, 256, 128
    H_local, SEQ = H // world, world * S_local
    shape = (3, B, H, S_local, D)
    plans = {r: build_all_to_all_plan_dim(shape=shape, dtype=torch.bfloat16, mesh_size=world, rank=r,
                                          src_buffer="src", dst_buffer="dst", src_split_axis=3,
                                          dst_split_axis=2, transfer_kind="pull", compute_producer=False)
             for r in range(world)}
    schedules, info = _compile(plans)
    tables = all2all_attn_tables(schedules[rank]["dst"], {"batch": 1, "head": 2, "seq": 3})
    assert len(tables.signal_offsets) == world * world

    g = torch.Generator().manual_seed(9)
    qkv = [torch.randn(*shape, generator=g).bfloat16() for _ in range(world)]     # per source rank
    # what the exchange must leave on `rank`: its heads, the whole sequence
    gathered = torch.cat([x[:, :, rank * H_local:(rank + 1) * H_local] for x in qkv], dim=3)
    ctx = CommContext(rank, info)
    for r in range(world):
        ctx.comm_buffers["src"][r].copy_(qkv[r])
    dst = ctx.comm_buffers["dst"][rank]
    flags = ctx.recv_signal_bufs[rank]
    main = torch.cuda.current_stream()

    def attend():
        return attention_forward(dst[0], dst[1], dst[2], D ** -0.5, wave_offsets=tables.wave_offsets,
                                 wave_sizes=tables.wave_sizes, cum_wave_sizes=tables.cum_wave_sizes,
                                 signal_ptr=flags, signal_offsets=tables.signal_offsets,
                                 NUM_WAVES=len(tables.signal_offsets), cum_tiles=tables.cum_tiles)

    # eager
    dst.zero_()
    ctx.reset_signals()
    ctx.start_after(main)
    ctx.execute()
    eager = attend()
    ctx.end_before(main)
    check_status()
    ctx.check_status()
    assert torch.equal(dst.cpu(), gathered)
    want = numerics.sdpa_fp32(gathered[0], gathered[1], gathered[2], D ** -0.5)
    assert _rel(eager, want) <= REL_TOL

    # with two flag sets a captured graph would keep writing the set of its capture: refused
    with pytest.raises(RuntimeError, match="flag set"):
        CommContext(rank, info, flag_sets=2).get_graph()
    graph = ctx.get_graph()
    comm_stream = torch.cuda.Stream()
    for replay in range(3):
        dst.zero_()
        ctx.reset_signals()
        torch.cuda.synchronize()
        comm_stream.wait_stream(main)
        with torch.cuda.stream(comm_stream):
            graph.replay()
        out = attend()
        main.wait_stream(comm_stream)
        check_status()
        ctx.check_status()
        assert torch.equal(dst.cpu(), gathered), f"replay {replay}"
        # partial results of one q block merge in the order their workgroups take the lock, so
        # two runs agree to rounding, not bit for bit
        assert _rel(out, want) <= REL_TOL, f"replay {replay}"
        assert flags.tolist() == [1] * world


def test_copy_kernel_producer_matches_copy_engine(hip):
    """The compute-unit copy path of CommContext (copy_blocks > 0) moves the same bytes."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_gather_plan_1d_swizzle

    world, rank, M, K = 4, 3, 512, 384
    plans = {r: build_all_gather_plan_1d_swizzle((M, K), torch.float16, 0, world, r, "a", "pull")
             for r in range(world)}
    _, info = _compile(plans)
    g = torch.Generator().manual_seed(2)
    a = torch.randn(M, K, generator=g).half()
    rows = M // world
    for blocks, fused in ((0, False), (8, False), (8, True), (3, True)):
        ctx = CommContext(rank, info, copy_blocks=blocks, fuse_flags=fused)
        for r in range(world):
            ctx.comm_buffers["a"][r][r * rows:(r + 1) * rows].copy_(a[r * rows:(r + 1) * rows])
        ctx.reset_signals()
        ctx.start_after()
        ctx.execute()
        ctx.end_before()
        ctx.check_status()
        assert torch.equal(ctx.comm_buffers["a"][rank].cpu(), a)
        assert ctx.recv_signal_bufs[rank].tolist() == [1] * (world - 1)
        assert ctx._tickets.tolist() == [0]          # the fused kernel leaves its workgroup counter at zero
    with pytest.raises(ValueError):
        CommContext(rank, info, fuse_flags=True)     # needs the copy kernel


def test_fused_copy_and_flag_gates_the_consumer(hip):
    """The consumer GEMM polls flags that the fused copy + flag kernels of a side stream set: a
    flag seen means the chunk's bytes are there (NaN poison otherwise), over several iterations."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_gather_plan_1d_swizzle
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_consumer
    from syncopate_amd.interface.wave_tables import gemm_consumer_tables

    world, rank, M, N, K, BM, BN = 8, 5, 4096, 1024, 1024, 128, 256
    plans = {r: build_all_gather_plan_1d_swizzle((M, K), torch.bfloat16, 0, world, r, "a", "pull")
             for r in range(world)}
    schedules, info = _compile(plans)
    tables = gemm_consumer_tables(schedules[rank]["a"], N)
    g = torch.Generator().manual_seed(8)
    a = (0.05 * torch.randn(M, K, generator=g)).bfloat16()
    b = (0.05 * torch.randn(N, K, generator=g)).bfloat16().cuda()
    ref = numerics.gemm_fp32(a, b.cpu())
    rows = M // world
    ctx = CommContext(rank, info, copy_blocks=24, fuse_flags=True, flag_sets=2, link_delay_us=30)
    for r in range(world):
        ctx.comm_buffers["a"][r][r * rows:(r + 1) * rows].copy_(a[r * rows:(r + 1) * rows])
    symm = ctx.comm_buffers["a"][rank]
    c = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    first = None
    for it in range(3):
        for r in range(world):
            if r != rank:
                symm[r * rows:(r + 1) * rows].fill_(float("nan"))
        c.zero_()
        ctx.reset_signals()
        ctx.start_after()
        gemm_consumer(symm, b, c, ctx.recv_signal_bufs[rank], tables.block_shapes, tables.block_offsets,
                      tables.signal_offsets, world, 200, BM, BN, cum_tiles=tables.cum_tiles)
        ctx.execute()
        ctx.end_before()
        check_status()
        ctx.check_status()
        assert torch.equal(symm.cpu(), a)
        assert _rel(c, ref) <= REL_TOL
        first = c.clone() if first is None else first
        assert torch.equal(c, first)


def test_copy_kernel_rejects_misaligned(hip):
    buf = torch.zeros(256, dtype=torch.uint8, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    from syncopate_amd import _lib

    assert hip.syn_copy_kernel_async(buf.data_ptr() + 8, buf.data_ptr() + 128, 64, 4, s) == _lib.SYN_EALIGN
    assert hip.syn_copy_kernel_async(buf.data_ptr(), buf.data_ptr() + 128, 60, 4, s) == _lib.SYN_EALIGN
    assert hip.syn_copy_kernel_async(buf.data_ptr(), buf.data_ptr() + 128, 64, 0, s) == _lib.SYN_EINVAL
    words = torch.zeros(4, dtype=torch.int64, device="cuda")
    flag, ticket = words.data_ptr(), words.data_ptr() + 8
    assert hip.syn_copy_flag_async(buf.data_ptr() + 8, buf.data_ptr() + 128, 64, flag, 1, ticket, 4, s) == _lib.SYN_EALIGN
    assert hip.syn_copy_flag_async(buf.data_ptr(), buf.data_ptr() + 128, 64, None, 1, ticket, 4, s) == _lib.SYN_EINVAL
    assert hip.syn_copy_flag_async(buf.data_ptr(), buf.data_ptr() + 128, 0, flag, 1, ticket, 4, s) == _lib.SYN_EINVAL
    assert words.tolist() == [0, 0, 0, 0]
    torch.cuda.synchronize()


@pytest.mark.parametrize("kind", ["ring", "double_ring"])
def test_ring_allgather_gemm_whole_mesh(hip, kind):
    """Ring forms of the all-gather: a rank only receives what its neighbours forward, so the op
    lists of the whole mesh are replayed (on one stream, in an order that honours every flag
    wait) while the consumer GEMM of one rank walks its own schedule."""
    from oracle import visit_order
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import (
        build_double_ring_all_gather_plan,
        build_ring_all_gather_plan,
    )
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm
    from syncopate_amd.interface.wave_tables import gemm_consumer_tables

    world, rank, M, K, N, BM, BN = 4, 2, 1024, 256, 512, 128, 128
    if kind == "ring":
        plans = {r: build_ring_all_gather_plan((M, K), torch.bfloat16, 0, world, r, "a") for r in range(world)}
    else:
        plans = {r: build_double_ring_all_gather_plan((M, K), torch.bfloat16, 0, world, 2, r, "a")
                 for r in range(world)}
    schedules, info = _compile(plans)
    tables = gemm_consumer_tables(schedules[rank]["a"], N)
    rows = M // world
    arrival = [off[0] // rows for off in tables.block_offsets]
    assert sorted(arrival) == list(range(world)) and arrival[0] == rank
    if kind == "ring":
        assert arrival == [(rank - k) % world for k in range(world)]

    g = torch.Generator().manual_seed(21)
    a = (0.05 * torch.randn(M, K, generator=g)).bfloat16()
    b = (0.05 * torch.randn(N, K, generator=g)).bfloat16()
    ctx = CommContext(rank, info, link_delay_us=10)
    for r in range(world):
        ctx.comm_buffers["a"][r][r * rows:(r + 1) * rows].copy_(a[r * rows:(r + 1) * rows])
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    tiles = (M // BM) * (N // BN)
    log = torch.full((tiles, 4), -1, dtype=torch.int32, device="cuda")
    main = torch.cuda.current_stream()

    ctx.reset_signals(whole_mesh=True)
    ctx.start_after(main)
    ctx.execute_mesh()
    gemm(ctx.comm_buffers["a"][rank], b.cuda(), c, world, 24, BM, BN, 64, 8,
         cur_wave_sizes=tables.block_shapes, wave_offsets=tables.block_offsets,
         signal_ptr=ctx.recv_signal_bufs[rank], signal_offsets=tables.signal_offsets,
         cum_tiles=tables.cum_tiles, visit_log=log)
    ctx.end_before(main)
    check_status()
    ctx.check_status()

    for r in range(world):                           # the gather completed on every simulated rank
        assert torch.equal(ctx.comm_buffers["a"][r].cpu(), a), f"rank {r}"
    assert _rel(c, numerics.gemm_fp32(a, b)) <= REL_TOL
    want = visit_order.gemm_tile_visits(tables.block_shapes, tables.block_offsets, tables.signal_offsets,
                                        M=M, N=N, BM=BM, BN=BN, group_m=8, num_sms=24,
                                        cum_tiles=tables.cum_tiles)
    got = log.cpu().tolist()
    for v in want:
        assert got[v["tile_id"]] == [v["pid"], v["wave"], v["pid_m"], v["pid_n"]], v


def test_two_flag_sets_over_iterations(hip):
    """AG+GEMM iterations with two flag sets: every iteration polls the set that the previous
    one left zeroed, new data each time, eagerly and as a replayed graph of two iterations."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_gather_plan_1d_swizzle
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm
    from syncopate_amd.interface.wave_tables import gemm_consumer_tables

    world, rank, M, K, N, BM, BN = 4, 1, 1024, 256, 512, 128, 128
    rows = M // world
    plans = {r: build_all_gather_plan_1d_swizzle((M, K), torch.bfloat16, 0, world, r, "a", "pull")
             for r in range(world)}
    schedules, info = _compile(plans)
    tables = gemm_consumer_tables(schedules[rank]["a"], N)
    ctx = CommContext(rank, info, flag_sets=2)
    sets = [ctx._flag_sets[i][0][rank] for i in range(2)]
    g = torch.Generator().manual_seed(4)
    b = (0.02 * torch.randn(N, K, generator=g)).bfloat16()
    bd = b.cuda()
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    dev_tables = dict(
        cur_wave_sizes=torch.tensor(tables.block_shapes, dtype=torch.int32, device="cuda"),
        wave_offsets=torch.tensor(tables.block_offsets, dtype=torch.int32, device="cuda"),
        signal_offsets=torch.tensor(tables.signal_offsets, dtype=torch.int32, device="cuda"),
        cum_tiles=tables.cum_tiles)

    def load(a):
        for r in range(world):
            ctx.comm_buffers["a"][r][r * rows:(r + 1) * rows].copy_(a[r * rows:(r + 1) * rows])
            if r != rank:       # what this rank holds of a peer's shard is stale until the pull lands
                ctx.comm_buffers["a"][rank][r * rows:(r + 1) * rows].fill_(float("nan"))

    def step():
        cur = torch.cuda.current_stream()
        ctx.reset_signals()
        ctx.start_after(cur)
        ctx.execute()
        gemm(ctx.comm_buffers["a"][rank], bd, c, world, 16, BM, BN, 64, 8,
             signal_ptr=ctx.recv_signal_bufs[rank], **dev_tables)
        ctx.end_before(cur)

    used = []
    for it in range(4):
        a = (0.02 * torch.randn(M, K, generator=g)).bfloat16()
        load(a.cuda())
        step()
        check_status()
        ctx.check_status()
        assert _rel(c, numerics.gemm_fp32(a, b)) <= REL_TOL
        current = ctx.recv_signal_bufs[rank]
        other = sets[1] if current.data_ptr() == sets[0].data_ptr() else sets[0]
        assert current.tolist() == [1] * (world - 1)
        assert other.tolist() == [0] * (world - 1)      # zeroed behind this iteration's copies
        used.append(current.data_ptr())
    assert used[0] == used[2] and used[1] == used[3] and used[0] != used[1]

    # two iterations as one graph (one per flag set), replayed with eager work in between
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
        step()
    for it in range(3):
        a = (0.02 * torch.randn(M, K, generator=g)).bfloat16()
        load(a.cuda())
        c.zero_()
        graph.replay()
        check_status()
        ctx.check_status()
        assert _rel(c, numerics.gemm_fp32(a, b)) <= REL_TOL
        assert sorted(s.sum().item() for s in sets) == [0, world - 1]


@pytest.mark.parametrize("rank,dtype,causal", [(1, torch.float16, False), (3, torch.bfloat16, False),
                                                (0, torch.bfloat16, True)])
def test_attention_to_all2all_iteration(hip, rank, dtype, causal):
    """Attention as the PRODUCER of an all-to-all along the sequence axis
    (tests/test_attn_all2all_transform.py:105-214 of the reference): the kernel writes its output
    into the comm buffer wave by wave (one wave per destination rank), counts finished tiles per
    wave and sets the wave's COMPUTE_DONE flag; the side stream waits for each flag and pushes
    that sequence chunk to its owner."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan_axis
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.interface.wave_tables import attn_producer_tables

    world, B, Hp, D = 4, 2, 2, 128
    SEQ = world * 256
    chunk = SEQ // world
    g = torch.Generator().manual_seed(21 + rank)
    q, k, v = (torch.randn(B, SEQ, Hp, D, generator=g).to(dtype) for _ in range(3))

    plans = {r: build_all_to_all_plan_axis(shape=(B, SEQ, Hp, D), dtype=dtype, mesh_size=world, rank=r,
                                           src_buffer="src", dst_buffer="dst", split_axis=1,
                                           transfer_kind="push", compute_producer=True)
             for r in range(world)}
    schedules, info = _compile(plans)
    tables = attn_producer_tables(schedules[rank]["src"], {"batch": 0, "head": 2, "seq": 1}, SEQ)
    # remote chunks first, in the order of the pushes, the rank's own chunk last
    assert [off[2] // chunk for off in tables.wave_offsets] == [(rank + 1 + i) % world for i in range(world)]
    assert tables.signal_offsets == list(range(world))

    ctx = CommContext(rank, info)
    src = ctx.comm_buffers["src"][rank]
    src.fill_(float("nan"))              # a chunk shipped before its tiles were stored would carry NaNs
    flags = ctx.compute_signal_bufs[rank]
    counters = torch.zeros(flags.numel(), dtype=torch.int32, device="cuda")
    comm_stream = torch.cuda.Stream()
    main = torch.cuda.current_stream()

    ctx.reset_signals()
    comm_stream.wait_stream(main)
    attention_forward(q.cuda(), k.cuda(), v.cuda(), D ** -0.5, layout="bshd", causal=causal,
                      output_buffer=src, counter_ptr=counters, signal_ptr=flags,
                      wave_offsets=tables.wave_offsets, wave_sizes=tables.wave_sizes, cum_wave_sizes=tables.cum_wave_sizes,
                      signal_offsets=tables.signal_offsets, cum_tiles=tables.cum_tiles)
    ctx.start_after(comm_stream)
    ctx.execute()
    ctx.end_before(comm_stream)
    main.wait_stream(comm_stream)
    check_status()
    ctx.check_status()

    ref = torch.nn.functional.scaled_dot_product_attention(
        q.float().transpose(1, 2), k.float().transpose(1, 2), v.float().transpose(1, 2),
        scale=D ** -0.5, is_causal=causal).transpose(1, 2)
    assert _rel(src, ref) <= REL_TOL
    assert flags.tolist() == [1] * world
    assert counters.tolist() == [B * Hp * (chunk // 128)] * world
    for peer in range(world):
        got = ctx.comm_buffers["dst"][peer][:, rank * chunk:(rank + 1) * chunk]
        assert torch.equal(got, src[:, peer * chunk:(peer + 1) * chunk])      # bit for bit, no NaNs
        if peer != rank:
            assert ctx.recv_signal_bufs[peer].sum().item() == 1


@pytest.mark.parametrize("kind,rank,split", [("pull", 1, False), ("pull", 3, False), ("push", 2, False),
                                             ("pull", 0, True)])
def test_gemm_rs_sm_reduce_iteration(hip, kind, rank, split):
    """Reduce-scatter by direct reduction with box copies on compute units
    (tests/test_gemm_rs_sm_reduce.py:95-175): every rank's producer GEMM writes its partial product
    and one COMPUTE_DONE flag per chunk; `pull`: this rank's side stream waits for each peer's
    chunk and adds it into its own result; `push`: it adds its own chunks into the peers' results."""
    from syncopate_amd.communication.code_gen import CodeGenOptions, CommGenerator
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_reduce_scatter_direct_reduce_plan
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_producer
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules
    from syncopate_amd.interface.wave_tables import gemm_producer_tables

    world, M, N, K, BM, BN, programs = 4, 1024, 512, 256, 128, 128, 24
    rows = M // world
    dtype = torch.float16
    plans = {r: build_reduce_scatter_direct_reduce_plan(shape=(M, N), dtype=dtype, axis=0, mesh_size=world,
                                                        rank=r, src_buffer="src", dst_buffer="dst",
                                                        transfer_kind=kind) for r in range(world)}
    gen = CommGenerator(plans)
    gen.plan_signals()
    schedules = lower_comm_plan_to_raw_schedules(gen)
    info = gen.generate_code_for_plan(options=CodeGenOptions(copy_engine=False, use_tma=False))
    info.local_world_size = info.world_size
    if split:
        # the device split in two like the reference's green contexts (tests/test_gemm_rs_collective.py:124-126):
        # 16 compute units for the box copies, the GEMMs on the stream that owns the other 240
        info.num_copy_sms, info.need_green_ctx, programs = 10, True, 240
        ctx = CommContext(rank, info)
        assert ctx.cu_split == [16, 240]
    else:
        ctx = CommContext(rank, info)
        with pytest.raises(ValueError):
            ctx.execute()                     # box copies need compute units: num_copy_sms is still 0
        torch.cuda.synchronize()
        info.num_copy_sms = 10
    compute = ctx.compute_stream

    g = torch.Generator().manual_seed(23)
    a = [(0.1 * torch.randn(M, K, generator=g)).to(dtype) for _ in range(world)]
    b = [(0.1 * torch.randn(N, K, generator=g)).to(dtype) for _ in range(world)]
    start = (0.25 * torch.randn(world, rows, N, generator=g)).to(dtype)
    for r in range(world):
        ctx.comm_buffers["src"][r].fill_(float("nan"))     # a chunk added before it was stored shows
        ctx.comm_buffers["dst"][r].copy_(start[r].cuda())
    ctx.reset_signals(whole_mesh=True)
    operands = {r: (a[r].cuda(), b[r].cuda()) for r in range(world)}
    compute.wait_stream(torch.cuda.current_stream())
    ctx.start_after()
    ctx.execute()                                          # the side stream waits for the flags
    runs = range(world) if kind == "pull" else [rank]
    with torch.cuda.stream(compute):
        for r in runs:
            tables = gemm_producer_tables(schedules[r]["src"])
            gemm_producer(*operands[r], ctx.comm_buffers["src"][r], ctx.compute_signal_bufs[r],
                          tables.block_shapes, tables.block_offsets, tables.signal_offsets, programs, BM, BN, 64, 8,
                          cum_tiles=tables.cum_tiles)
    torch.cuda.current_stream().wait_stream(compute)
    ctx.end_before()
    check_status()
    ctx.check_status()

    partial = {r: ctx.comm_buffers["src"][r].cpu() for r in runs}
    for r in runs:
        assert _rel(partial[r], numerics.gemm_fp32(a[r], b[r])) <= REL_TOL
    tiny = torch.finfo(dtype).tiny

    def add_once(acc, term, fragile):
        """One addition in the element type; `fragile` collects the elements where an operand or
        the sum is subnormal (atomic units may flush those), which are compared by tolerance."""
        out = (acc.float() + term.float()).to(dtype)
        for t in (acc, term, out):
            fragile |= (t.abs() < tiny) & (t != 0)
        return out

    def same(got, want, fragile):
        assert torch.equal(got[~fragile], want[~fragile])
        assert fragile.float().mean().item() < 0.01
        torch.testing.assert_close(got[fragile].float(), want[fragile].float(), atol=1e-3, rtol=0)

    if kind == "pull":
        # additions in the op list's order, one rounding each
        order = [op.src_rank for ops in info.operations[rank] for op in ops if hasattr(op, "src_slice")]
        assert sorted(order) == list(range(world)) and order[-1] == rank
        want = start[rank].clone()
        fragile = torch.zeros(rows, N, dtype=torch.bool)
        for r in order:
            want = add_once(want, partial[r][rank * rows:(rank + 1) * rows], fragile)
        same(ctx.comm_buffers["dst"][rank].cpu(), want, fragile)
        assert ctx.recv_signal_bufs[rank].tolist() == [1] * world
        total = start[rank].double() + sum(numerics.gemm_fp32(a[r], b[r])[rank * rows:(rank + 1) * rows].double()
                                           for r in range(world))
        # the reference's bound for this path (tests/test_gemm_rs_sm_reduce.py:175)
        torch.testing.assert_close(ctx.comm_buffers["dst"][rank].cpu().double(), total, atol=1e-2, rtol=1e-2)
    else:
        for peer in range(world):
            fragile = torch.zeros(rows, N, dtype=torch.bool)
            want = add_once(start[peer], partial[rank][peer * rows:(peer + 1) * rows], fragile)
            same(ctx.comm_buffers["dst"][peer].cpu(), want, fragile)
            assert ctx.recv_signal_bufs[peer].tolist() == [1 if i == rank else 0 for i in range(world)]


@pytest.mark.parametrize("form", ["reduce_scatter", "all_reduce", "all_reduce_two_buffers"])
def test_gemm_then_library_collective_whole_mesh(hip, form):
    """Producer GEMM -> per slab: wait for its COMPUTE_DONE flag, one collective of the mesh, one
    RECEIVE flag (tests/test_gemm_rs_collective.py:90-165, tests/test_gemm_ar_collective.py,
    tests/test_gemm_ar_collective_nvsharp.py; the second GEMM of tests/test_domino_alike_mlp_collective.py:121-200
    and tests/test_domino_alike_mlp_collective_nvsharp.py is this flow on an MLP's shapes).  The
    other ranks' partial products are computed beforehand; this rank's kernel runs beside the
    replay of the mesh, which carries each collective out over the ranks' buffers."""
    from syncopate_amd.communication.code_gen import CommGenerator
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import (
        build_all_reduce_nvsharp_plan,
        build_all_reduce_plan,
        build_reduce_scatter_collective_plan,
    )
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_producer
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules
    from syncopate_amd.interface.wave_tables import gemm_producer_tables

    world, rank, M, N, K, BM, BN, programs, slabs = 4, 2, 1024, 512, 256, 128, 128, 24, 2
    dtype = torch.bfloat16
    if form == "reduce_scatter":
        build = lambda r: build_reduce_scatter_collective_plan(
            shape=(M, N), dtype=dtype, axis=0, split_axis=1, mesh_size=world, rank=r, src_buffer="src",
            dst_buffer="dst", num_reduce_scatters=slabs, compute_producer=True)
        produced, result = "src", "dst"
    elif form == "all_reduce":
        build = lambda r: build_all_reduce_plan(
            shape=(M, N), dtype=dtype, mesh_size=world, rank=r, buffer_name="c", num_all_reduces=slabs,
            split_axis=0, compute_producer=True)
        produced, result = "c", "c"
    else:
        build = lambda r: build_all_reduce_nvsharp_plan(
            shape=(M, N), dtype=dtype, mesh_size=world, rank=r, src_name="src", dst_name="dst",
            num_all_reduces=slabs, split_axis=1, compute_producer=True)
        produced, result = "src", "dst"
    gen = CommGenerator({r: build(r) for r in range(world)})
    gen.plan_signals()
    schedules = lower_comm_plan_to_raw_schedules(gen)
    info = gen.generate_code_for_plan()
    info.local_world_size = info.world_size
    ctx = CommContext(rank, info)
    with pytest.raises(NotImplementedError):
        ctx.execute()                       # one rank's list alone cannot carry out a collective

    g = torch.Generator().manual_seed(31)
    a = [(0.1 * torch.randn(M, K, generator=g)).to(dtype) for _ in range(world)]
    b = [(0.1 * torch.randn(N, K, generator=g)).to(dtype) for _ in range(world)]
    for r in range(world):
        ctx.comm_buffers[produced][r].fill_(float("nan"))
    ctx.reset_signals(whole_mesh=True)

    def produce(r):
        tables = gemm_producer_tables(schedules[r][produced])
        shapes, offsets, signals = tables.block_shapes, tables.block_offsets, tables.signal_offsets
        if form == "all_reduce":
            # source and result in one buffer: the lowering puts the resident whole tensor in front
            # as a wave without a flag, and the caller drops it (tests/test_gemm_ar_collective.py:120-122)
            assert shapes[0] == [M, N] and signals[0] == -1
            shapes, offsets, signals = shapes[1:], offsets[1:], signals[1:]
        assert len(shapes) == slabs and sorted(signals) == list(range(slabs))
        gemm_producer(a[r].cuda(), b[r].cuda(), ctx.comm_buffers[produced][r], ctx.compute_signal_bufs[r],
                      shapes, offsets, signals, programs, BM, BN, 64, 8,
                      cum_tiles=sum(h * w for h, w in shapes))

    for r in range(world):
        if r != rank:
            produce(r)
    ctx.start_after()
    ctx.execute_mesh()
    produce(rank)
    ctx.end_before()
    check_status()
    ctx.check_status()

    partial = [numerics.gemm_fp32(a[r], b[r]) for r in range(world)]
    total = sum(p.double() for p in partial)
    rows = M // world
    for r in range(world):
        got = ctx.comm_buffers[result][r].cpu()
        want = total[r * rows:(r + 1) * rows] if form == "reduce_scatter" else total
        assert got.shape == want.shape
        # W roundings to 16 bits on top of the GEMMs'; the reference bounds the path by 1e-2 too
        torch.testing.assert_close(got.double(), want, atol=2e-2, rtol=2e-2)
        assert ctx.recv_signal_bufs[r].tolist() == [1] * slabs
    if form != "all_reduce":
        # the partial products were only read
        assert _rel(ctx.comm_buffers["src"][rank], partial[rank]) <= REL_TOL


@pytest.mark.parametrize("rank", [1, 2])
def test_gemm_all2all_gemm_chain(hip, rank):
    """An MLP with its hidden layer sharded by columns and its output by rows
    (tests/test_gemm_all2all_gemm.py:126-200, 257-318): producer GEMM x @ w1_shard^T with a flag per
    row block -> all-to-all by box copies on compute units (every rank sends each owner its rows)
    -> split-K consumer GEMM over the gathered columns, which starts on a source rank's columns
    as soon as that rank's block has arrived.  The other ranks' first GEMMs are computed
    beforehand; the whole mesh's op lists are replayed beside this rank's two kernels."""
    from syncopate_amd.communication.code_gen import CodeGenOptions, CommGenerator
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan_dim
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_producer, gemm_splitk
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules
    from syncopate_amd.interface.wave_tables import gemm_producer_tables

    world, seq, hidden, ffn, BM, BN = 4, 1024, 256, 1024, 128, 128
    seq_local, ffn_local = seq // world, ffn // world
    dtype = torch.float16
    gen = CommGenerator({r: build_all_to_all_plan_dim(
        shape=(seq, ffn_local), dtype=dtype, mesh_size=world, rank=r, src_buffer="src", dst_buffer="dst",
        src_split_axis=1, dst_split_axis=0, transfer_kind="push", compute_producer=True) for r in range(world)})
    gen.plan_signals()
    schedules = lower_comm_plan_to_raw_schedules(gen)
    info = gen.generate_code_for_plan(CodeGenOptions(copy_engine=False))
    info.local_world_size = info.world_size
    info.num_copy_sms = 12
    ctx = CommContext(rank, info)

    g = torch.Generator().manual_seed(41)
    x = (0.1 * torch.randn(seq, hidden, generator=g)).to(dtype)
    w1 = [(0.1 * torch.randn(ffn_local, hidden, generator=g)).to(dtype) for _ in range(world)]
    w2 = (0.1 * torch.randn(hidden, ffn, generator=g)).to(dtype)
    xd, w2d = x.cuda(), w2.cuda()

    def first_gemm(r):
        tables = gemm_producer_tables(schedules[r]["src"])
        gemm_producer(xd, w1[r].cuda(), ctx.comm_buffers["src"][r], ctx.compute_signal_bufs[r], tables.block_shapes,
                      tables.block_offsets, tables.signal_offsets, 24, BM, BN, 64, 8, cum_tiles=tables.cum_tiles)

    # the consumer's tables: a wave per source rank, [rows, hidden, that rank's columns] at [0, 0, first column]
    dst = schedules[rank]["dst"]
    shapes = [[rows, hidden, cols] for rows, cols in dst.gen_block_shape_lists()]
    offsets = [[r0, 0, c0] for r0, c0 in dst.gen_block_offset_lists()]
    signals = dst.gen_signal_lists()
    assert sorted(c0 for _, _, c0 in offsets) == [q * ffn_local for q in range(world)] and sorted(signals) == [0, 1, 2, 3]

    out = torch.zeros(seq_local, hidden, dtype=dtype, device="cuda")
    ctx.comm_buffers["dst"][rank].fill_(float("nan"))       # columns read before their flag would show
    ctx.reset_signals(whole_mesh=True)
    for r in range(world):
        if r != rank:
            first_gemm(r)
    ctx.start_after()
    ctx.execute_mesh()
    first_gemm(rank)
    gemm_splitk(ctx.comm_buffers["dst"][rank], w2d, out, world, 24, BM, BN, 64, 8, cur_wave_sizes=shapes,
                wave_offsets=offsets, signal_ptr=ctx.recv_signal_bufs[rank], signal_offsets=signals,
                cum_tiles=sum(s[0] * s[1] for s in shapes))
    ctx.end_before()
    check_status()
    ctx.check_status()

    hidden_act = torch.cat([numerics.gemm_fp32(x, w1[r]) for r in range(world)], dim=1)       # [seq, ffn]
    mine = hidden_act[rank * seq_local:(rank + 1) * seq_local]
    gathered = ctx.comm_buffers["dst"][rank].float().cpu()
    assert _rel(gathered, mine) <= REL_TOL
    for q in range(world):
        # what rank q sent is bit for bit what its GEMM produced
        sent = ctx.comm_buffers["src"][q][rank * seq_local:(rank + 1) * seq_local]
        assert torch.equal(ctx.comm_buffers["dst"][rank][:, q * ffn_local:(q + 1) * ffn_local], sent)
    want = mine.to(dtype).float() @ w2.float().t()
    # four partial products rounded to fp16 and added; the reference bounds the chain by 5e-1
    assert _rel(out, want) <= 4 * REL_TOL
    assert ctx.recv_signal_bufs[rank].tolist() == [1] * world


@pytest.mark.parametrize("slices", [0, 2])
def test_all2all_then_split_k_gemm(hip, slices):
    """Attention output [B, S, H/W, D] per rank -> all-to-all (heads gathered, sequence scattered,
    4-D boxes copied on compute units) -> output projection over the gathered heads, a source
    rank's heads at a time (tests/test_all2all_gemm.py:80-160, 222-275).  With `slices` every
    shard is pulled in that many slices of the sequence, each a wave of its own
    (build_all_to_all_plan_dim_waves, tests/test_all2all_gemm_split_collective.py:212-240)."""
    from syncopate_amd.communication.code_gen import CodeGenOptions, CommGenerator
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan_dim, build_all_to_all_plan_dim_waves
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_splitk
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules

    world, rank, S, H, D, BM, BN = 4, 3, 1024 if slices else 512, 8, 128, 128, 256
    B = 1 if slices else 2            # a slice of the sequence is one run of GEMM rows only for a single batch
    s_local, h_local, hidden = S // world, H // world, H * D
    dtype = torch.float16
    common = dict(shape=(B, S, h_local, D), dtype=dtype, mesh_size=world, src_buffer="src", dst_buffer="dst",
                  src_split_axis=2, dst_split_axis=1)
    if slices:
        gen = CommGenerator({r: build_all_to_all_plan_dim_waves(rank=r, transfer_kind="pull", num_waves=slices, **common)
                             for r in range(world)})
    else:
        gen = CommGenerator({r: build_all_to_all_plan_dim(rank=r, transfer_kind="push", **common)
                             for r in range(world)})
    gen.plan_signals()
    schedules = lower_comm_plan_to_raw_schedules(gen)
    info = gen.generate_code_for_plan(CodeGenOptions(copy_engine=False))
    info.local_world_size = info.world_size
    info.num_copy_sms = 12
    ctx = CommContext(rank, info)
    assert tuple(ctx.comm_buffers["dst"][rank].shape) == (B, s_local, H, D)

    g = torch.Generator().manual_seed(43)
    attn_out = [(0.1 * torch.randn(B, S, h_local, D, generator=g)).to(dtype) for _ in range(world)]
    w = (0.1 * torch.randn(hidden, hidden, generator=g)).to(dtype)
    for r in range(world):
        ctx.comm_buffers["src"][r].copy_(attn_out[r].cuda())
    ctx.comm_buffers["dst"][rank].fill_(float("nan"))

    dst = schedules[rank]["dst"]
    shapes = [[b * s, hidden, h * d] for b, s, h, d in dst.gen_block_shape_lists()]
    offsets = [[ob * s_local + os_, 0, oh * D + od] for ob, os_, oh, od in dst.gen_block_offset_lists()]
    signals = dst.gen_signal_lists()
    assert sorted(o[2] for o in offsets) == sorted(q * h_local * D for q in range(world) for _ in range(max(slices, 1)))
    assert len(shapes) == world * max(slices, 1)
    if slices:
        assert sorted({o[0] for o in offsets}) == [i * (s_local // slices) for i in range(slices)]

    gemm_input = ctx.comm_buffers["dst"][rank].reshape(-1, hidden)          # [B * S/W, H * D]
    out = torch.zeros(gemm_input.shape[0], hidden, dtype=dtype, device="cuda")
    ctx.reset_signals(whole_mesh=True)
    ctx.start_after()
    ctx.execute_mesh()
    gemm_splitk(gemm_input, w.cuda(), out, world, 40, BM, BN, 64, 8, cur_wave_sizes=shapes, wave_offsets=offsets,
                signal_ptr=ctx.recv_signal_bufs[rank], signal_offsets=signals,
                cum_tiles=sum(s[0] * s[1] for s in shapes))
    ctx.end_before()
    check_status()
    ctx.check_status()

    # the exchange, restated: rank r keeps its sequence slice of every rank's heads
    want_in = torch.cat([attn_out[q][:, rank * s_local:(rank + 1) * s_local] for q in range(world)], dim=2)
    assert torch.equal(ctx.comm_buffers["dst"][rank].cpu(), want_in)
    want = want_in.reshape(-1, hidden).float() @ w.float().t()
    assert _rel(out, want) <= 4 * REL_TOL
    assert ctx.recv_signal_bufs[rank].tolist() == [1] * len(shapes)


@pytest.mark.parametrize("lead_on_compute_stream,lead_copy_blocks,list_blocks",
                         [(False, 0, 0), (True, 0, 0), (True, 64, 0), (False, 64, 0), (False, 0, 8), (True, 64, 8)])
def test_leading_ops_ahead_of_the_consumer(hip, lead_on_compute_stream, lead_copy_blocks, list_blocks):
    """execute(lead_ops=4): the first two chunk copies and their flags are in place before the
    consumer is launched - through an event the compute stream waits for, or enqueued on the
    compute stream itself (lead_on), as two kernels each or as one copy-and-flag kernel each
    (lead_copy_blocks), or the whole op list as one kernel that walks it (list_blocks; two kernels
    with leading ops).  Every form must gather the same bytes and give the resident result."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_gather_plan_1d_swizzle
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm
    from syncopate_amd.interface.wave_tables import gemm_consumer_tables

    world, rank, M, K, N, BM, BN = 4, 2, 2048, 512, 512, 128, 128
    rows = M // world
    plans = {r: build_all_gather_plan_1d_swizzle((M, K), torch.bfloat16, 0, world, r, "a", "pull")
             for r in range(world)}
    schedules, info = _compile(plans)
    tables = gemm_consumer_tables(schedules[rank]["a"], N)
    ctx = CommContext(rank, info, lead_copy_blocks=lead_copy_blocks, list_blocks=list_blocks)
    g = torch.Generator().manual_seed(21)
    a = (0.02 * torch.randn(M, K, generator=g)).bfloat16()
    b = (0.02 * torch.randn(N, K, generator=g)).bfloat16()
    ad, bd = a.cuda(), b.cuda()
    for r in range(world):
        ctx.comm_buffers["a"][r][r * rows:(r + 1) * rows].copy_(ad[r * rows:(r + 1) * rows])
        if r != rank:
            ctx.comm_buffers["a"][rank][r * rows:(r + 1) * rows].fill_(float("nan"))
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    cur = torch.cuda.current_stream()
    for it in range(2):
        ctx.reset_signals()
        ctx.start_after(cur)
        ctx.execute(lead_ops=4, lead_on=cur if lead_on_compute_stream else None)
        ctx.wait_lead(cur)
        gemm(ctx.comm_buffers["a"][rank], bd, c, world, 24, BM, BN, 64, 8, cur_wave_sizes=tables.block_shapes,
             wave_offsets=tables.block_offsets, signal_ptr=ctx.recv_signal_bufs[rank],
             signal_offsets=tables.signal_offsets, cum_tiles=tables.cum_tiles)
        ctx.end_before(cur)
        check_status()
        ctx.check_status()
        assert torch.equal(ctx.comm_buffers["a"][rank], ad)
        assert ctx.recv_signal_bufs[rank].tolist() == [1] * (world - 1)
        assert _rel(c, numerics.gemm_fp32(a, b)) <= REL_TOL
        if list_blocks:
            assert ctx._list_tickets[0].tolist() == [0] * (world - 1)      # every ticket word left zero again
        # the peers' rows are stale again for the next iteration
        for r in range(world):
            if r != rank:
                ctx.comm_buffers["a"][rank][r * rows:(r + 1) * rows].fill_(float("nan"))
