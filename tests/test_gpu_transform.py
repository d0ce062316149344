"""Annotated kernels bound to the HIP templates and launched through the binding (GPU, C ABI).

The reference transforms an annotated Triton kernel and calls the result with the wave tables as
keywords (tests/test_ag_gemm_gen.py:44-77, tests/test_gemm_rs_transform.py,
tests/test_allgather_attn_transform.py:60-105, tests/test_gemm_rs_direct_reduce.py:166-189); the
calls below use the same keywords on the binding.
"""

import json
import os

import pytest
import torch

from oracle import numerics

pytestmark = pytest.mark.gpu

SNIPPETS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "annotation_cases.json")))["snippets"]
REL_TOL = 1e-2


def _rel(out, ref):
    return ((out.float().cpu() - ref.float()).abs().max() / ref.float().abs().max()).item()


def _table(rows, device="cuda"):
    return torch.tensor(rows, dtype=torch.int32, device=device)


def test_gemm_bindings_consumer_producer_and_one_tile_per_program(hip):
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_consumer
    from syncopate_amd.computation.transform import AnnotationTransformer

    M, N, K, BM, BN, world = 1024, 512, 256, 128, 128, 4
    g = torch.Generator().manual_seed(3)
    a = (0.05 * torch.randn(M, K, generator=g)).bfloat16().cuda()
    b = (0.05 * torch.randn(N, K, generator=g)).bfloat16().cuda()
    rows = M // world
    sizes = [[rows, N]] * world
    offsets = [[((1 + i) % world) * rows, 0] for i in range(world)]
    signals = [-1, 0, 1, 2]
    ref = numerics.gemm_fp32(a.cpu(), b.cpu())
    plain = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    ones = torch.ones(world, dtype=torch.int64, device="cuda")
    gemm_consumer(a, b, plain, ones, sizes, offsets, signals, world, 40, BM, BN, cum_tiles=M * N)

    consumer = AnnotationTransformer(enable_consumer=True).transform(SNIPPETS["gemm_persistent_with_epilogue"])
    c1 = torch.zeros_like(plain)
    consumer.launch(a, b, c1, world, 40, BM, BN, 64, 8, cur_wave_sizes=_table(sizes), wave_offsets=_table(offsets),
                    signal_ptr=ones, signal_offsets=_table(signals), cum_tiles=M * N)
    check_status()
    assert torch.equal(c1, plain) and _rel(c1, ref) <= REL_TOL

    producer = AnnotationTransformer(enable_producer=True).transform(SNIPPETS["gemm_persistent_with_epilogue"])
    flags = torch.zeros(world, dtype=torch.int64, device="cuda")
    counters = torch.zeros(world, dtype=torch.int32, device="cuda")
    c2 = torch.zeros_like(plain)
    producer.launch(a, b, c2, world, 40, BM, BN, 64, 8, cur_wave_sizes=_table(sizes), wave_offsets=_table(offsets),
                    signal_ptr=flags, signal_offsets=_table([0, 1, 2, 3]), counter_ptr=counters, cum_tiles=M * N)
    check_status()
    assert torch.equal(c2, plain)
    assert flags.tolist() == [1] * world and counters.tolist() == [(rows // BM) * (N // BN)] * world

    # the form with one tile per program names its tables wave_sizes / cum_wave_sizes / NUM_WAVES
    single = AnnotationTransformer(enable_consumer=True).transform(SNIPPETS["gemm_one_tile_per_program"])
    c3 = torch.zeros_like(plain)
    cums = [(i + 1) * rows * N for i in range(world)]
    single.launch(a, b, c3, world, 40, BM, BN, 64, 8, wave_sizes=_table(sizes), wave_offsets=_table(offsets),
                  cum_wave_sizes=_table(cums), signal_ptr=ones, signal_offsets=_table(signals), cum_tiles=M * N,
                  NUM_WAVES=world)
    check_status()
    assert torch.equal(c3, plain)


def test_gemm_in_both_roles_waits_on_one_flag_array_and_reports_into_another(hip):
    """Consumer and producer annotations on one kernel (both transform passes applied): the GEMM
    waits for a wave's consumer flag before it reads that wave's rows of A and counts finished tiles
    into the producer's flags.  The last two row chunks of A arrive late, on a side stream."""
    from syncopate_amd import _lib
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm
    from syncopate_amd.computation.transform import AnnotationTransformer

    M, N, K, BM, BN, world = 1024, 512, 256, 128, 128, 4
    g = torch.Generator().manual_seed(13)
    a_full = (0.05 * torch.randn(M, K, generator=g)).bfloat16().cuda()
    b = (0.05 * torch.randn(N, K, generator=g)).bfloat16().cuda()
    rows = M // world
    sizes = [[rows, N]] * world
    offsets = [[i * rows, 0] for i in range(world)]
    a = a_full.clone()
    a[2 * rows:].fill_(float("nan"))          # chunks 2 and 3 are not there yet
    wait_flags = torch.zeros(2, dtype=torch.int64, device="cuda")
    done_flags = torch.zeros(world, dtype=torch.int64, device="cuda")
    counters = torch.zeros(world, dtype=torch.int32, device="cuda")
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    side = pick_side_streams(1)[0]
    main = torch.cuda.current_stream()
    side.wait_stream(main)
    both = AnnotationTransformer(enable_consumer=True, enable_producer=True) \
        .transform(SNIPPETS["gemm_persistent_with_epilogue"])
    assert both.template == "gemm" and both.consumer and both.producer
    both.launch(a, b, c, world, 40, BM, BN, 64, 8, cur_wave_sizes=_table(sizes), wave_offsets=_table(offsets),
                producer_signal_ptr=done_flags, producer_signal_offsets=_table([0, 1, 2, 3]),
                producer_counter_ptr=counters, consumer_signal_ptr=wait_flags,
                consumer_signal_offsets=_table([-1, -1, 0, 1]), cum_tiles=M * N, spin_timeout_us=3_000_000)
    lib = _lib.load()
    for i in range(2):
        _lib.check("syn_delay_us", lib.syn_delay_us(300, _lib.stream_handle(side)))
        with torch.cuda.stream(side):
            a[(2 + i) * rows:(3 + i) * rows].copy_(a_full[(2 + i) * rows:(3 + i) * rows])
        _lib.check("syn_flag_set", lib.syn_flag_set(wait_flags.data_ptr() + 8 * i, 1, _lib.stream_handle(side)))
    main.wait_stream(side)
    check_status()
    assert _rel(c, numerics.gemm_fp32(a_full.cpu(), b.cpu())) <= REL_TOL
    assert done_flags.tolist() == [1] * world and counters.tolist() == [(rows // BM) * (N // BN)] * world

    # the second flag pair: both or neither, with counters only, indices inside the array
    kw = dict(cur_wave_sizes=_table(sizes), wave_offsets=_table(offsets), signal_ptr=done_flags,
              signal_offsets=_table([0, 1, 2, 3]), cum_tiles=M * N)
    with pytest.raises(ValueError):
        gemm(a_full, b, c, world, 40, BM, BN, 64, 8, consumer_signal_ptr=wait_flags,
             consumer_signal_offsets=_table([-1, -1, 0, 1]), **kw)                             # no counters
    with pytest.raises(ValueError):
        gemm(a_full, b, c, world, 40, BM, BN, 64, 8, counter_ptr=counters, consumer_signal_ptr=wait_flags, **kw)
    with pytest.raises(ValueError):
        gemm(a_full, b, c, world, 40, BM, BN, 64, 8, counter_ptr=counters, consumer_signal_ptr=wait_flags,
             consumer_signal_offsets=_table([-1, -1, 0, 2]), **kw)                             # beyond the array


def test_gemm_binding_with_a_peer_bound_result(hip):
    """Reduce-scatter by direct reduction inside the kernel (tests/test_gemm_rs_direct_reduce.py:102-192):
    the schedule of the push plan makes `c_desc` a producer-side, reducing descriptor, so every
    wave is atomically added into its owner's result."""
    from syncopate_amd.communication.code_gen import CommGenerator
    from syncopate_amd.communication.common_descriptors import build_reduce_scatter_direct_reduce_plan
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.transform import AnnotationTransformer, RemoteBinding
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules

    world, M, N, K, BM, BN = 4, 1024, 512, 256, 128, 256
    rows = M // world
    dtype = torch.float16
    gen = CommGenerator({r: build_reduce_scatter_direct_reduce_plan(
        shape=(M, N), dtype=dtype, axis=0, mesh_size=world, rank=r, src_buffer="src", dst_buffer="dst",
        transfer_kind="push") for r in range(world)})
    gen.plan_signals()
    schedules = lower_comm_plan_to_raw_schedules(gen)
    g = torch.Generator().manual_seed(17)
    a = [(0.05 * torch.randn(M, K, generator=g)).to(dtype) for _ in range(world)]
    b = [(0.05 * torch.randn(N, K, generator=g)).to(dtype) for _ in range(world)]
    results = [torch.zeros(rows, N, dtype=dtype, device="cuda") for _ in range(world)]
    for rank in range(world):
        schedule = schedules[rank]["src"]
        binding = AnnotationTransformer(remote_descriptors={"c_desc": RemoteBinding("c_ptr", schedule)}) \
            .transform(SNIPPETS["gemm_persistent_with_epilogue"])
        assert binding.remote["c_desc"].is_reduce and binding.remote["c_desc"].role == "producer"
        shapes = schedule.gen_block_shape_lists()
        # the resident block has no peer (-1): folded to the rank itself, as the reference's caller does
        ranks = [r if r >= 0 else rank for r in schedule.gen_target_rank_list()]
        binding.launch(a[rank].cuda(), b[rank].cuda(), results, world, 48 + rank, BM, BN, 64, 8,
                       cur_wave_sizes=_table(shapes), wave_offsets=_table(schedule.gen_block_offset_lists()),
                       target_rank=_table(ranks), dst_offsets=_table(schedule.gen_dst_offset_lists()),
                       cum_tiles=sum(h * w for h, w in shapes), M=M)
    check_status()
    total = sum(numerics.gemm_fp32(a[r], b[r]) for r in range(world))
    torch.testing.assert_close(torch.cat(results).float().cpu(), total, atol=1e-2, rtol=1e-2)


def test_attention_binding_matches_the_template_call(hip):
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation.transform import AnnotationTransformer

    B, H, Sq, Skv, D, chunks = 1, 2, 256, 1024, 128, 4
    g = torch.Generator().manual_seed(5)
    q, k, v = ((torch.randn(B, H, s, D, generator=g)).half().cuda() for s in (Sq, Skv, Skv))
    chunk = Skv // chunks
    cums = [(i + 1) * B * H * Sq for i in range(chunks)]
    tables = dict(wave_offsets=_table([[0, 0, 0, o * chunk] for o in (1, 2, 3, 0)]),
                  wave_sizes=_table([[B, H, Sq, chunk]] * chunks), cum_wave_sizes=_table(cums),
                  signal_ptr=torch.ones(chunks, dtype=torch.int64, device="cuda"),
                  signal_offsets=_table([-1, 0, 1, 2]), cum_tiles=cums[-1])
    want = attention_forward(q, k, v, D ** -0.5, **tables)
    binding = AnnotationTransformer(enable_consumer=True).transform(SNIPPETS["attention_with_kv_range"])
    got = binding.launch(q, k, v, D ** -0.5, NUM_WAVES=chunks, **tables)
    check_status()
    # partial results of one q block are merged in the order the kv chunks finish: two launches
    # agree to rounding, not bit for bit
    torch.testing.assert_close(got.float(), want.float(), atol=2e-3, rtol=2e-3)
    assert _rel(got, numerics.sdpa_fp32(q.cpu(), k.cpu(), v.cpu(), D ** -0.5)) <= 2e-2


def test_split_k_binding(hip):
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.transform import AnnotationTransformer

    M, N, K, BM, BN = 256, 512, 384, 128, 256
    g = torch.Generator().manual_seed(13)
    a = (0.05 * torch.randn(M, K, generator=g)).bfloat16()
    b = (0.05 * torch.randn(N, K, generator=g)).bfloat16()
    binding = AnnotationTransformer(enable_consumer=True).transform(SNIPPETS["gemm_split_k_persistent"])
    assert binding.template == "gemm_splitk"
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    flags = torch.ones(3, dtype=torch.int64, device="cuda")
    binding.launch(a.cuda(), b.cuda(), c, 1, 20, BM, BN, 64, 8,
                   cur_wave_sizes=_table([[M, N, 128]] * 3), wave_offsets=_table([[0, 0, 256], [0, 0, 0], [0, 0, 128]]),
                   signal_ptr=flags, signal_offsets=_table([0, 1, 2]), cum_tiles=3 * M * N)
    check_status()
    assert _rel(c, numerics.gemm_fp32(a, b)) <= 3 * REL_TOL
