"""Chunks and flags that arrive in an order other than the schedule's.

The wave order is the order in which the plan EXPECTS the chunks (syncopate/computation/gemm/template.py:92-97,
121-128: a program waits for the flag of the wave its next tile is in).  A peer that is late, or links of
different speed, deliver them in another order.  Nothing may depend on the expected order but speed: every
chunk has its own flag, a program that waits for a late chunk holds only its own compute unit, and the
result is bit for bit the resident one.  No wait may time out - every kernel ends normally.
"""

import pytest
import torch

from oracle import numerics

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


@pytest.mark.parametrize("order", ["reversed", "interleaved"])
def test_gemm_consumer_with_chunks_delivered_out_of_schedule_order(hip, order):
    from syncopate_amd import _lib
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_consumer

    M, N, K, world, rank, BM, BN = 2048, 512, 512, 8, 2, 128, 128
    g = torch.Generator().manual_seed(17)
    a = (0.02 * torch.randn(M, K, generator=g)).bfloat16()
    b = (0.02 * torch.randn(N, K, generator=g)).bfloat16()
    rows = M // world
    # the schedule of a 1-D swizzle pull: wave k = chunk (rank + k) % world behind flag k - 1
    sizes = [[rows, N]] * world
    offsets = [[((rank + k) % world) * rows, 0] for k in range(world)]
    signals = [-1] + list(range(world - 1))
    staged, bd = a.cuda(), b.cuda()
    ones = torch.ones(world - 1, dtype=torch.int64, device="cuda")
    c_res = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    gemm_consumer(staged, bd, c_res, ones, sizes, offsets, signals, world, 96, BM, BN, cum_tiles=M * N)
    torch.cuda.synchronize()

    symm = torch.full((M, K), float("nan"), dtype=torch.bfloat16, device="cuda")      # poison: nothing is read early
    symm[rank * rows:(rank + 1) * rows].copy_(staged[rank * rows:(rank + 1) * rows])
    flags = torch.zeros(world - 1, dtype=torch.int64, device="cuda")
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    side = pick_side_streams(1)[0]
    torch.cuda.synchronize()
    main = torch.cuda.current_stream()
    side.wait_stream(main)
    # 96 programs: the first waves' programs wait while the copies of the LAST waves land first
    gemm_consumer(symm, bd, c, flags, sizes, offsets, signals, world, 96, BM, BN, cum_tiles=M * N,
                  spin_timeout_us=5_000_000)
    waves = list(range(1, world))
    delivery = waves[::-1] if order == "reversed" else waves[1::2] + waves[0::2]
    nbytes = rows * K * 2
    for k in delivery:
        chunk = (rank + k) % world
        _lib.check("syn_delay_us", hip.syn_delay_us(150, _lib.stream_handle(side)))
        _lib.check("syn_copy_async", hip.syn_copy_async(symm.data_ptr() + chunk * nbytes, staged.data_ptr() + chunk * nbytes,
                                                        nbytes, _lib.stream_handle(side)))
        _lib.check("syn_flag_set", hip.syn_flag_set(flags.data_ptr() + 8 * (k - 1), 1, _lib.stream_handle(side)))
    main.wait_stream(side)
    check_status()                                   # raises if any wait gave up
    assert flags.tolist() == [1] * (world - 1)
    assert torch.equal(c, c_res)
    assert ((c.float().cpu() - numerics.gemm_fp32(a, b)).abs().max() / numerics.gemm_fp32(a, b).abs().max()).item() <= REL_TOL


@pytest.mark.parametrize("form", ["one_tile_per_program", "pairs_chained", "planned_causal"])
def test_attention_with_kv_chunks_delivered_out_of_schedule_order(hip, form):
    from syncopate_amd import _lib
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward, plan_attention_work

    H, Sq, chunk, chunks = 2, 512, 256, 4
    Skv = chunk * chunks
    causal = form == "planned_causal"
    if causal:
        Sq = Skv
    g = torch.Generator().manual_seed(23)
    q = torch.randn(1, H, Sq, 128, generator=g).bfloat16()
    k = torch.randn(1, H, Skv, 128, generator=g).bfloat16()
    v = torch.randn(1, H, Skv, 128, generator=g).bfloat16()
    arrival = [2, 0, 3, 1]                                  # the schedule: wave i = kv chunk arrival[i] behind flag i - 1
    offsets = [[0, 0, 0, cidx * chunk] for cidx in arrival]
    sizes = [[1, H, Sq, chunk]] * chunks
    cums = [(i + 1) * H * Sq for i in range(chunks)]
    signals = [-1, 0, 1, 2]
    kw = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_offsets=signals, cum_tiles=cums[-1],
              causal=causal)
    if form == "pairs_chained":
        kw.update(pair_q_blocks=True, chain_q_blocks=True)
    elif form == "planned_causal":
        kw.update(pair_q_blocks=True, work_plan=plan_attention_work(offsets, sizes, cums, causal=True, num_programs=6,
                                                                    max_visits=2))
    else:
        kw.update(num_programs=12)
    kd, vd = k.cuda(), v.cuda()
    ones = torch.ones(chunks - 1, dtype=torch.int64, device="cuda")
    resident = attention_forward(q.cuda(), kd, vd, 128 ** -0.5, signal_ptr=ones, **kw)
    torch.cuda.synchronize()

    kbuf = torch.full_like(kd, float("nan"))
    vbuf = torch.full_like(vd, float("nan"))
    own = arrival[0]
    kbuf[:, :, own * chunk:(own + 1) * chunk].copy_(kd[:, :, own * chunk:(own + 1) * chunk])
    vbuf[:, :, own * chunk:(own + 1) * chunk].copy_(vd[:, :, own * chunk:(own + 1) * chunk])
    flags = torch.zeros(chunks - 1, dtype=torch.int64, device="cuda")
    side = pick_side_streams(1)[0]
    torch.cuda.synchronize()
    main = torch.cuda.current_stream()
    side.wait_stream(main)
    gated = attention_forward(q.cuda(), kbuf, vbuf, 128 ** -0.5, signal_ptr=flags, spin_timeout_us=5_000_000, **kw)
    with torch.cuda.stream(side):
        for wave in (3, 2, 1):                              # reversed
            cidx = arrival[wave]
            _lib.check("syn_delay_us", hip.syn_delay_us(150, _lib.stream_handle(side)))
            kbuf[:, :, cidx * chunk:(cidx + 1) * chunk].copy_(kd[:, :, cidx * chunk:(cidx + 1) * chunk])
            vbuf[:, :, cidx * chunk:(cidx + 1) * chunk].copy_(vd[:, :, cidx * chunk:(cidx + 1) * chunk])
            _lib.check("syn_flag_set", hip.syn_flag_set(flags.data_ptr() + 8 * (wave - 1), 1, _lib.stream_handle(side)))
    main.wait_stream(side)
    check_status()
    assert flags.tolist() == [1] * (chunks - 1)
    ref = numerics.sdpa_fp32(q, k, v, 128 ** -0.5, causal=causal)
    assert ((gated.float().cpu() - ref).abs().max() / ref.abs().max()).item() <= REL_TOL
    if form == "pairs_chained":
        # one program per pair of q blocks, sums in registers, fixed order of the kv chunks: the same bits
        assert torch.equal(gated, resident)
    else:
        # partial results are merged in the order the programs finish: equal to rounding
        assert ((gated.float() - resident.float()).abs().max() / resident.float().abs().max()).item() <= REL_TOL
