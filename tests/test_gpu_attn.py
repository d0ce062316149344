"""GPU parity of the chunked-KV flash attention against the CPU oracle (through the C ABI)."""

import pytest
import torch

from oracle import numerics, visit_order

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def _qkv(Z, H, Sq, Skv, dtype, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(Z, H, Sq, 128, generator=g).to(dtype)
    k = torch.randn(Z, H, Skv, 128, generator=g).to(dtype)
    v = torch.randn(Z, H, Skv, 128, generator=g).to(dtype)
    return q, k, v


def _kv_waves(Z, H, Sq, chunks, signals):
    """One wave per kv chunk (element units), all of q against it."""
    offsets, sizes, cums, total = [], [], [], 0
    for lo, hi in chunks:
        offsets.append([0, 0, 0, lo])
        sizes.append([Z, H, Sq, hi - lo])
        total += Z * H * Sq
        cums.append(total)
    return offsets, sizes, cums, list(signals), total


def _attention_snippet():
    """The annotated attention kernel of the annotation fixture (a producer needs an epilogue mark on top)."""
    import json
    import os

    path = os.path.join(os.path.dirname(__file__), "golden", "annotation_cases.json")
    return json.load(open(path))["snippets"]["attention_with_kv_range"]


def _rel(out, ref):
    return ((out.float().cpu() - ref).abs().max() / ref.abs().max()).item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("num_programs", [0, 5])
def test_chunked_kv_matches_sdpa_and_oracle(hip, dtype, num_programs):
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    Z, H, Sq, Skv = 1, 3, 256, 1024
    q, k, v = _qkv(Z, H, Sq, Skv, dtype)
    chunks = [(512, 768), (0, 256), (768, 1024), (256, 512)]          # arrival order
    offsets, sizes, cums, signals, total = _kv_waves(Z, H, Sq, chunks, [-1, 0, 1, 2])
    flags = torch.ones(3, dtype=torch.int64, device="cuda")
    sm_scale = 128 ** -0.5
    log = torch.full((total // 128, 8), -1, dtype=torch.int32, device="cuda")
    o, lse = attention_forward(q.cuda(), k.cuda(), v.cuda(), sm_scale, wave_offsets=offsets,
                               wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags,
                               signal_offsets=signals, NUM_WAVES=4, cum_tiles=total,
                               num_programs=num_programs, return_lse=True, visit_log=log)
    check_status()
    ref = numerics.sdpa_fp32(q, k, v, sm_scale)
    assert _rel(o, ref) <= REL_TOL
    want_o, want_lse = numerics.chunked_attention(q, k, v, sm_scale, chunks)
    assert _rel(o, want_o.float()) <= REL_TOL
    assert (lse.cpu() - want_lse).abs().max().item() <= 2e-2
    # lse2 is the base-2 log-sum-exp of the scaled scores
    s = (q.float() @ k.float().transpose(-1, -2)) * sm_scale
    assert (lse.cpu() - torch.logsumexp(s, dim=-1) / 0.6931471805599453).abs().max().item() <= 2e-2
    rows = log.cpu().tolist()
    for t, got in enumerate(rows):
        w = visit_order.attn_tile_work(t, offsets, sizes, cums, signals)
        assert got[:7] == [w["wave"], w["z"], w["h"], w["q_block"], w["kv_lo"], w["kv_hi"], w["signal"]]


def test_causal_extension_matches_sdpa(hip):
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    Z, H, S = 2, 2, 512
    q, k, v = _qkv(Z, H, S, S, torch.bfloat16, seed=4)
    chunks = [(0, 128), (128, 384), (384, 512)]
    offsets, sizes, cums, signals, total = _kv_waves(Z, H, S, chunks, [-1, -1, -1])
    flags = torch.ones(1, dtype=torch.int64, device="cuda")
    for scale in (128 ** -0.5, 1.0):
        o = attention_forward(q.cuda(), k.cuda(), v.cuda(), scale, wave_offsets=offsets, wave_sizes=sizes,
                              cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals,
                              cum_tiles=total, causal=True)
        check_status()
        ref = numerics.sdpa_fp32(q, k, v, scale, causal=True)
        assert _rel(o, ref) <= REL_TOL


def test_hand_template_form_resident(hip):
    """attention(q, k, v, sm_scale, wave_dicts) with the everything-resident table
    (reference: syncopate/computation/attn/template.py:442-497, kv_divide waves; the hand-written
    kernel is driven the same way in tests/test_allgather_attn.py:20-40, 70-120)."""
    from syncopate_amd.computation.attn import attention, build_waves_and_signals_divisible
    from syncopate_amd.computation._launch import check_status

    Z, H, N_CTX = 2, 2, 768
    g = torch.Generator(device="cpu").manual_seed(20)
    q = (0.5 * torch.randn(Z, H, N_CTX, 128, generator=g)).half()
    k = (0.5 * torch.randn(Z, H, N_CTX, 128, generator=g)).half()
    v = (0.5 * torch.randn(Z, H, N_CTX, 128, generator=g)).half()
    wave_dicts = build_waves_and_signals_divisible(Z, H, N_CTX, N_CTX, w=3)
    assert wave_dicts["CUM_CHUNK_BLOCK"] == 4
    o = attention(q.cuda(), k.cuda(), v.cuda(), 0.5, wave_dicts)
    check_status()
    p = torch.softmax((q.float() @ k.float().transpose(2, 3)) * 0.5, dim=-1)
    ref = p @ v.float()
    torch.testing.assert_close(o.float().cpu(), ref, atol=5e-2, rtol=0)   # the reference's bound (:486)
    assert _rel(o, ref) <= REL_TOL


@pytest.mark.parametrize("causal", [False, True])
def test_bshd_layout_and_strided_views(hip, causal):
    """The reference's second layout, q/k/v as [Z, S, H, D] (example_attn_bshd.py), and views of
    a stacked comm buffer whose batch/head/row strides are not those of a contiguous tensor."""
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    Z, H, S = 2, 3, 512
    q, k, v = _qkv(Z, H, S, S, torch.bfloat16, seed=4)
    sm_scale = 128 ** -0.5
    ref = numerics.sdpa_fp32(q, k, v, sm_scale, causal=causal)
    chunks = [(0, 256), (256, 512)]
    offsets, sizes, cums, signals, total = _kv_waves(Z, H, S, chunks, [-1, 0])
    flags = torch.ones(1, dtype=torch.int64, device="cuda")
    tables = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags,
                  signal_offsets=signals, cum_tiles=total, causal=causal)

    # [Z, S, H, D] tensors
    qs, ks, vs = (t.permute(0, 2, 1, 3).contiguous().cuda() for t in (q, k, v))
    o = attention_forward(qs, ks, vs, sm_scale, layout="bshd", **tables)
    check_status()
    assert o.shape == qs.shape
    assert _rel(o.permute(0, 2, 1, 3), ref) <= REL_TOL

    # k and v as slices of one stacked [2, Z, H, S + 128, D] buffer, q a slice of a wider tensor
    kv = torch.zeros(2, Z, H, S + 128, 128, dtype=torch.bfloat16, device="cuda")
    kv[0, :, :, 64:64 + S].copy_(k)
    kv[1, :, :, 64:64 + S].copy_(v)
    wide = torch.zeros(Z, H + 1, S, 128, dtype=torch.bfloat16, device="cuda")
    wide[:, 1:].copy_(q)
    o2 = attention_forward(wide[:, 1:], kv[0, :, :, 64:64 + S], kv[1, :, :, 64:64 + S], sm_scale, **tables)
    check_status()
    assert _rel(o2, ref) <= REL_TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("num_programs,xcd_remap", [(0, False), (3, False), (0, True), (16, True)])
def test_paired_q_blocks_match_sdpa_and_oracle(hip, dtype, num_programs, xcd_remap):
    """Two q blocks per workgroup in opposite phases (an extension: one program per tile in the
    reference): same tiles, same merge under the q blocks' locks, results to the same tolerance."""
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    Z, H, Sq, Skv = 2, 3, 512, 1024
    q, k, v = _qkv(Z, H, Sq, Skv, dtype, seed=4)
    chunks = [(512, 768), (0, 256), (768, 1024), (256, 512)]          # arrival order
    offsets, sizes, cums, signals, total = _kv_waves(Z, H, Sq, chunks, [-1, 0, 1, 2])
    flags = torch.ones(3, dtype=torch.int64, device="cuda")
    sm_scale = 128 ** -0.5
    tiles = total // 128
    log = torch.full((tiles, 8), -1, dtype=torch.int32, device="cuda")
    o, lse = attention_forward(q.cuda(), k.cuda(), v.cuda(), sm_scale, wave_offsets=offsets,
                               wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags,
                               signal_offsets=signals, NUM_WAVES=4, cum_tiles=total,
                               num_programs=num_programs, return_lse=True, visit_log=log,
                               pair_q_blocks=True, xcd_remap=xcd_remap)
    check_status()
    assert _rel(o, numerics.sdpa_fp32(q, k, v, sm_scale)) <= REL_TOL
    want_o, want_lse = numerics.chunked_attention(q, k, v, sm_scale, chunks)
    assert _rel(o, want_o.float()) <= REL_TOL
    assert (lse.cpu() - want_lse).abs().max().item() <= 2e-2

    # every tile was visited once, with the kv range and flag of its wave; tiles 2i and 2i + 1 by one program
    got = log.cpu().tolist()
    grid = min(num_programs, tiles // 2) if num_programs else tiles // 2
    for tile_id, rec in enumerate(got):
        exp = visit_order.attn_tile_work(tile_id, offsets, sizes, cums, signals)
        assert rec[:7] == [exp["wave"], exp["z"], exp["h"], exp["q_block"], exp["kv_lo"], exp["kv_hi"], exp["signal"]]
        assert 0 <= rec[7] < grid
        assert rec[7] == got[tile_id ^ 1][7]
    if not xcd_remap:
        assert [rec[7] for rec in got[0::2]] == [pair % grid for pair in range(tiles // 2)]
    else:
        # a bijection between workgroups and first pairs: every program took its share
        first = {}
        for pair in range(tiles // 2):
            first.setdefault(got[2 * pair][7], pair)
        assert sorted(first) == list(range(grid)) and sorted(first.values()) == list(range(grid))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("num_programs,xcd_remap", [(0, False), (12, False), (0, True)])
def test_chained_q_blocks_match_sdpa_and_oracle(hip, dtype, num_programs, xcd_remap):
    """Waves that differ in the kv range only, as many programs as a wave has pairs of q blocks: a program
    walks from one wave's kv range into the next with the sums in registers and writes its q blocks
    once.  Same tiles on the same programs as the persistent launch of that size (an extension: the
    reference merges under the q block's lock after every tile)."""
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    Z, H, Sq, Skv = 2, 3, 512, 1024
    q, k, v = _qkv(Z, H, Sq, Skv, dtype, seed=6)
    chunks = [(512, 640), (0, 384), (768, 1024), (384, 512), (640, 768)]     # arrival order, ragged
    offsets, sizes, cums, signals, total = _kv_waves(Z, H, Sq, chunks, [-1, 0, 1, 2, 1])
    flags = torch.ones(3, dtype=torch.int64, device="cuda")
    sm_scale = 128 ** -0.5
    tiles = total // 128
    pairs_per_wave = Z * H * Sq // 256
    log = torch.full((tiles, 8), -1, dtype=torch.int32, device="cuda")
    o = torch.full((Z, H, Sq, 128), float("nan"), dtype=dtype, device="cuda")
    _, lse = attention_forward(q.cuda(), k.cuda(), v.cuda(), sm_scale, wave_offsets=offsets,
                               wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags,
                               signal_offsets=signals, NUM_WAVES=len(chunks), cum_tiles=total,
                               num_programs=num_programs, return_lse=True, visit_log=log, out=o,
                               pair_q_blocks=True, chain_q_blocks=True, xcd_remap=xcd_remap)
    check_status()
    assert _rel(o, numerics.sdpa_fp32(q, k, v, sm_scale)) <= REL_TOL
    want_o, want_lse = numerics.chunked_attention(q, k, v, sm_scale, chunks)
    assert _rel(o, want_o.float()) <= REL_TOL
    assert (lse.cpu() - want_lse).abs().max().item() <= 2e-2

    got = log.cpu().tolist()
    for tile_id, rec in enumerate(got):
        exp = visit_order.attn_tile_work(tile_id, offsets, sizes, cums, signals)
        assert rec[:7] == [exp["wave"], exp["z"], exp["h"], exp["q_block"], exp["kv_lo"], exp["kv_hi"], exp["signal"]]
        assert rec[7] == got[tile_id ^ 1][7]
    programs = [rec[7] for rec in got[0::2]]
    if not xcd_remap:
        # tile t of a persistent launch of that many programs runs on program t % programs
        assert programs == [pair % pairs_per_wave for pair in range(tiles // 2)]
    else:
        assert sorted(programs[:pairs_per_wave]) == list(range(pairs_per_wave))
        assert programs == programs[:pairs_per_wave] * len(chunks)


def test_chained_q_blocks_argument_errors_and_timeout(hip):
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import FlagWaitTimeout, check_status

    Z, H, Sq, Skv = 1, 2, 256, 512
    q, k, v = (t.cuda() for t in _qkv(Z, H, Sq, Skv, torch.bfloat16))
    flags = torch.ones(2, dtype=torch.int64, device="cuda")
    offsets, sizes, cums, signals, total = _kv_waves(Z, H, Sq, [(0, 256), (256, 512)], [-1, 0])
    kw = dict(wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals, cum_tiles=total)
    with pytest.raises(ValueError, match="pair_q_blocks"):
        attention_forward(q, k, v, 0.1, wave_offsets=offsets, chain_q_blocks=True, **kw)
    with pytest.raises(ValueError, match="num_programs = 2"):
        attention_forward(q, k, v, 0.1, wave_offsets=offsets, pair_q_blocks=True, chain_q_blocks=True, num_programs=1, **kw)
    # a wave over other heads than wave 0's
    shifted = [offsets[0], [0, 1, 0, 256]]
    narrow = [[Z, 1, Sq, 256], [Z, 1, Sq, 256]]
    with pytest.raises(ValueError, match="same"):
        attention_forward(q, k, v, 0.1, wave_offsets=shifted, wave_sizes=narrow, cum_wave_sizes=[Sq, 2 * Sq],
                          signal_ptr=flags, signal_offsets=signals, cum_tiles=2 * Sq, pair_q_blocks=True,
                          chain_q_blocks=True)

    # the second wave's flag never comes: every wavefront leaves at that fetch, and the launch says so
    flags.zero_()
    attention_forward(q, k, v, 0.1, wave_offsets=offsets, pair_q_blocks=True, chain_q_blocks=True,
                      spin_timeout_us=20_000, **kw)
    with pytest.raises(FlagWaitTimeout):
        check_status()
    check_status()


@pytest.mark.parametrize("seed", list(range(6)))
def test_random_wave_tables(hip, seed):
    """Tables drawn at random: heads, q rows and kv rows cut into ragged ranges, every (head range, q range, kv
    range) one wave, in a random order, with a random program count; odd seeds with two q blocks per
    workgroup.  The visit log equals the oracle's tile by tile, the result the chunked oracle's."""
    import numpy as np

    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    rng = np.random.default_rng(2000 + seed)
    pair = bool(seed & 1)
    Z, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    Sq, Skv = 256 * int(rng.integers(1, 4)), 128 * int(rng.integers(2, 9))

    def cut(extent, block, max_parts):
        blocks = extent // block
        parts = int(rng.integers(1, min(max_parts, blocks) + 1))
        cuts = sorted(rng.choice(range(1, blocks), size=parts - 1, replace=False).tolist()) if parts > 1 else []
        edges = [0] + cuts + [blocks]
        return [(lo * block, (hi - lo) * block) for lo, hi in zip(edges, edges[1:])]

    heads, qs, kvs = cut(H, 1, 2), cut(Sq, 256 if pair else 128, 2), cut(Skv, 128, 4)
    cells = [(h, q_, kv) for h in heads for q_ in qs for kv in kvs]
    order = rng.permutation(len(cells)).tolist()
    offsets = [[0, cells[i][0][0], cells[i][1][0], cells[i][2][0]] for i in order]
    sizes = [[Z, cells[i][0][1], cells[i][1][1], cells[i][2][1]] for i in order]
    cums, total = [], 0
    for sz in sizes:
        total += sz[0] * sz[1] * sz[2]
        cums.append(total)
    signals = [int(rng.integers(-1, 2)) for _ in order]
    tiles = total // 128
    num_programs = int(rng.choice([0, 1, 3, 7]))
    q, k, v = _qkv(Z, H, Sq, Skv, torch.bfloat16, seed=seed)
    flags = torch.ones(2, dtype=torch.int64, device="cuda")
    log = torch.full((tiles, 8), -1, dtype=torch.int32, device="cuda")
    sm_scale = 128 ** -0.5
    o = attention_forward(q.cuda(), k.cuda(), v.cuda(), sm_scale, wave_offsets=offsets, wave_sizes=sizes,
                          cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals, NUM_WAVES=len(order),
                          cum_tiles=total, num_programs=num_programs, visit_log=log, pair_q_blocks=pair)
    check_status()
    assert _rel(o, numerics.sdpa_fp32(q, k, v, sm_scale)) <= REL_TOL
    got = log.cpu().tolist()
    units = tiles // 2 if pair else tiles
    grid = min(num_programs, units) if num_programs else units
    for tile_id, rec in enumerate(got):
        exp = visit_order.attn_tile_work(tile_id, offsets, sizes, cums, signals)
        assert rec[:7] == [exp["wave"], exp["z"], exp["h"], exp["q_block"], exp["kv_lo"], exp["kv_hi"], exp["signal"]]
        assert rec[7] == ((tile_id // 2) if pair else tile_id) % grid


@pytest.mark.parametrize("pair", [False, True])
def test_more_waves_than_a_wavefront_has_lanes(hip, pair):
    """Eighty waves of one kv block each, padded with zero rows to 128: the wave of a tile id is looked up sixty-four
    prefix sums at a time, so the table spans two looks and ends in padding."""
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    Z, H, Sq, waves = 1, 1, 256, 80
    Skv = waves * 128
    q, k, v = _qkv(Z, H, Sq, Skv, torch.bfloat16, seed=50)
    order = torch.randperm(waves, generator=torch.Generator().manual_seed(3)).tolist()
    chunks = [(o * 128, (o + 1) * 128) for o in order]
    offsets, sizes, cums, signals, total = _kv_waves(Z, H, Sq, chunks, [-1] * waves)
    pad = 128 - waves
    offsets += [[0, 0, 0, 0]] * pad
    sizes += [[0, 0, 0, 0]] * pad
    cums += [0] * pad
    signals += [0] * pad
    flags = torch.ones(1, dtype=torch.int64, device="cuda")
    tiles = total // 128
    log = torch.full((tiles, 8), -1, dtype=torch.int32, device="cuda")
    sm_scale = 128 ** -0.5
    o = attention_forward(q.cuda(), k.cuda(), v.cuda(), sm_scale, wave_offsets=offsets, wave_sizes=sizes,
                          cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals, NUM_WAVES=128, cum_tiles=total,
                          visit_log=log, pair_q_blocks=pair, num_programs=3)
    check_status()
    # eighty partial results merged with a rounding to bf16 each (a random walk of 80 steps of up to 2^-9, in the order in
    # which the programs happen to take the locks: 0.016 to 0.021 from run to run): three times the usual bound
    assert _rel(o, numerics.sdpa_fp32(q, k, v, sm_scale)) <= 3 * REL_TOL
    for tile_id, rec in enumerate(log.cpu().tolist()):
        exp = visit_order.attn_tile_work(tile_id, offsets, sizes, cums, signals)
        assert rec[:7] == [exp["wave"], exp["z"], exp["h"], exp["q_block"], exp["kv_lo"], exp["kv_hi"], exp["signal"]]


def test_chained_form_replayed_as_a_graph(hip):
    """The chained launch (scratch words zeroed by a fill kernel, the kernel itself) captured as a HIP graph and
    replayed three times on new inputs, with eager work and synchronisation between the replays: every replay
    gives what the eager launch gives on the same inputs."""
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    Z, H, Sq, Skv = 1, 2, 512, 768
    sm_scale = 128 ** -0.5
    chunks = [(256, 512), (0, 256), (512, 768)]
    offsets, sizes, cums, signals, total = _kv_waves(Z, H, Sq, chunks, [-1, 0, 1])
    dev = lambda rows: torch.tensor(rows, dtype=torch.int32, device="cuda")
    tables = dict(wave_offsets=dev(offsets), wave_sizes=dev(sizes), cum_wave_sizes=dev(cums), signal_offsets=dev(signals),
                  cum_tiles=total, NUM_WAVES=len(chunks))
    flags = torch.ones(2, dtype=torch.int64, device="cuda")
    q, k, v = (t.cuda() for t in _qkv(Z, H, Sq, Skv, torch.bfloat16, seed=30))
    out = torch.zeros_like(q)
    kw = dict(signal_ptr=flags, pair_q_blocks=True, chain_q_blocks=True, out=out, **tables)
    attention_forward(q, k, v, sm_scale, **kw)          # warm-up: tables checked, program count noted
    check_status()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph):
            attention_forward(q, k, v, sm_scale, **kw)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        nq, nk, nv = _qkv(Z, H, Sq, Skv, torch.bfloat16, seed=40 + replay)
        q.copy_(nq.cuda()); k.copy_(nk.cuda()); v.copy_(nv.cuda())
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        check_status()
        got = out.clone()
        assert _rel(got, numerics.sdpa_fp32(nq, nk, nv, sm_scale)) <= REL_TOL, f"replay {replay}"
        eager = attention_forward(q, k, v, sm_scale, **{**kw, "out": torch.empty_like(q)})
        check_status()
        assert torch.equal(got, eager), f"replay {replay}"


def test_auto_form_takes_what_the_tables_allow(hip):
    """form="auto" (what attention() passes): chained where every wave lists the same (z, h, q) ranges, two q blocks
    per workgroup where the waves hold even numbers of q blocks, one program per tile otherwise; the same result
    to rounding every time, and the choice is remembered per table objects."""
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status, recall_note

    Z, H, Skv = 1, 2, 512
    sm_scale = 128 ** -0.5
    flags = torch.ones(2, dtype=torch.int64, device="cuda")

    def tables_for(Sq, q_cuts):
        offsets, sizes, cums, total = [], [], [], 0
        for q_lo, q_len in q_cuts:
            for kv_lo in (256, 0):
                offsets.append([0, 0, q_lo, kv_lo])
                sizes.append([Z, H, q_len, 256])
                total += Z * H * q_len
                cums.append(total)
        dev = lambda rows: torch.tensor(rows, dtype=torch.int32, device="cuda")
        return dict(wave_offsets=dev(offsets), wave_sizes=dev(sizes), cum_wave_sizes=dev(cums),
                    signal_offsets=dev([-1, 0, 1, 0][:len(cums)]), cum_tiles=total)

    cases = [(512, [(0, 512)], (True, Z * H * 512 // 256)),            # same q range in both waves: chained
             (512, [(0, 256), (256, 256)], (True, 0)),                # two q ranges: pairs, merged under locks
             (384, [(0, 384)], (False, 0))]                           # three q blocks per wave: one program per tile
    for Sq, q_cuts, want in cases:
        q, k, v = _qkv(Z, H, Sq, Skv, torch.bfloat16, seed=Sq)
        t = tables_for(Sq, q_cuts)
        o = attention_forward(q.cuda(), k.cuda(), v.cuda(), sm_scale, signal_ptr=flags, form="auto", **t)
        check_status()
        assert _rel(o, numerics.sdpa_fp32(q, k, v, sm_scale)) <= REL_TOL
        key = (t["wave_offsets"], t["wave_sizes"], t["cum_wave_sizes"], t["signal_offsets"])
        assert recall_note(key, "attention form") == want
        o2 = attention_forward(q.cuda(), k.cuda(), v.cuda(), sm_scale, signal_ptr=flags, form="auto", **t)   # from the note
        check_status()
        assert torch.equal(o, o2) or _rel(o2, o.float().cpu()) <= REL_TOL
        t["wave_sizes"][0, 3] = 256                                   # an in-place write: the note no longer holds
        assert recall_note(key, "attention form") is None
    with pytest.raises(ValueError, match="form"):
        attention_forward(q.cuda(), k.cuda(), v.cuda(), sm_scale, signal_ptr=flags, form="fastest", **t)


def test_paired_q_blocks_argument_errors(hip):
    from syncopate_amd.computation.attn import attention_forward

    q, k, v = (t.cuda() for t in _qkv(1, 1, 384, 256, torch.bfloat16))
    offsets, sizes, cums, signals, total = _kv_waves(1, 1, 384, [(0, 256)], [-1])
    flags = torch.ones(1, dtype=torch.int64, device="cuda")
    kw = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals,
              cum_tiles=total)
    with pytest.raises(ValueError, match="even number of q blocks"):
        attention_forward(q, k, v, 0.1, pair_q_blocks=True, **kw)            # three q blocks
    q2, k2, v2 = (t.cuda() for t in _qkv(1, 1, 256, 256, torch.bfloat16))
    offsets, sizes, cums, signals, total = _kv_waves(1, 1, 256, [(0, 256)], [-1])
    kw = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals,
              cum_tiles=total)
    with pytest.raises(ValueError, match="chain_q_blocks does not go with causal"):
        attention_forward(q2, k2, v2, 0.1, pair_q_blocks=True, chain_q_blocks=True, causal=True, **kw)
    with pytest.raises(ValueError):
        attention_forward(q2, k2, v2, 0.1, pair_q_blocks=True,
                          counter_ptr=torch.zeros(1, dtype=torch.int32, device="cuda"), **kw)
    # under a causal mask the pairs' kv ranges have to begin at even blocks
    q3, k3, v3 = (t.cuda() for t in _qkv(1, 1, 512, 512, torch.bfloat16))
    offsets, sizes, cums, signals, total = _kv_waves(1, 1, 512, [(0, 128), (128, 512)], [-1, -1])
    kw = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals,
              cum_tiles=total)
    with pytest.raises(ValueError, match="even blocks"):
        attention_forward(q3, k3, v3, 0.1, pair_q_blocks=True, causal=True, **kw)


def test_producer_form_that_also_waits(hip):
    """Both roles at once (tests/test_all2all_attn_all2all.py:192-245: consumer_signal_* beside the
    producer's): the kernel waits for a wave's consumer flag before it reads that wave's K and V,
    and counts finished tiles into the producer's flags."""
    from syncopate_amd import _lib
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.transform import AnnotationTransformer

    Z, H, Sq, Skv = 1, 2, 256, 1024
    q, k, v = _qkv(Z, H, Sq, Skv, torch.float16, seed=9)
    chunks = [(0, 256), (256, 512), (512, 768), (768, 1024)]
    offsets, sizes, cums, _, total = _kv_waves(Z, H, Sq, chunks, [0, 1, 2, 3])
    sm_scale = 128 ** -0.5
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    staged_k, staged_v = kd.clone(), vd.clone()
    kd[:, :, 512:].fill_(float("nan"))        # the last two chunks arrive late
    vd[:, :, 512:].fill_(float("nan"))
    wait_flags = torch.zeros(2, dtype=torch.int64, device="cuda")
    done_flags = torch.zeros(4, dtype=torch.int64, device="cuda")
    counters = torch.zeros(4, dtype=torch.int32, device="cuda")
    side = pick_side_streams(1)[0]
    main = torch.cuda.current_stream()
    side.wait_stream(main)
    binding = AnnotationTransformer(enable_consumer=True, enable_producer=True, consumer_descriptors=("desc_q",)) \
        .transform(_attention_snippet().replace("    attend(", "    # @sy.producer_epilogue\n    attend("))
    assert binding.template == "attention"
    out = binding.launch(qd, kd, vd, sm_scale, wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums,
                         NUM_WAVES=4, cum_tiles=total, producer_signal_ptr=done_flags,
                         producer_signal_offsets=[0, 1, 2, 3], producer_counter_ptr=counters,
                         consumer_signal_ptr=wait_flags, consumer_signal_offsets=[-1, -1, 0, 1],
                         spin_timeout_us=3_000_000)
    lib = _lib.load()
    for i, (lo, hi) in enumerate(chunks[2:]):
        _lib.check("syn_delay_us", lib.syn_delay_us(300, _lib.stream_handle(side)))
        with torch.cuda.stream(side):
            kd[:, :, lo:hi].copy_(staged_k[:, :, lo:hi])
            vd[:, :, lo:hi].copy_(staged_v[:, :, lo:hi])
        _lib.check("syn_flag_set", lib.syn_flag_set(wait_flags.data_ptr() + 8 * i, 1, _lib.stream_handle(side)))
    main.wait_stream(side)
    check_status()
    assert _rel(out, numerics.sdpa_fp32(q, k, v, sm_scale)) <= REL_TOL
    assert done_flags.tolist() == [1, 1, 1, 1] and counters.tolist() == [Z * H * Sq // 128] * 4
    # argument errors of the second flag pair
    with pytest.raises(ValueError):
        attention_forward(qd, kd, vd, sm_scale, wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums,
                          signal_ptr=done_flags, signal_offsets=[0, 1, 2, 3], cum_tiles=total,
                          consumer_signal_ptr=wait_flags, consumer_signal_offsets=[-1, -1, 0, 1])     # no counters
    with pytest.raises(ValueError):
        attention_forward(qd, kd, vd, sm_scale, wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums,
                          signal_ptr=done_flags, signal_offsets=[0, 1, 2, 3], cum_tiles=total, counter_ptr=counters,
                          consumer_signal_ptr=wait_flags, consumer_signal_offsets=[-1, -1, 0, 2])     # beyond the array


def test_causal_producer_counts_tiles_above_the_diagonal(hip):
    """Producer form under the causal mask: a (q block, kv chunk) tile that lies wholly above the
    diagonal computes nothing, but it is one of its wave's tiles - every counter must reach the
    wave's tile count and every flag must be published (a consumer of the flags would hang
    otherwise).  Also on a stream that is not the current one, with the launcher's own
    temporaries (tables from lists, locks, lse)."""
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    Z, H, S = 1, 2, 512
    q, k, v = _qkv(Z, H, S, S, torch.bfloat16, seed=12)
    chunks = [(0, 128), (128, 384), (384, 512)]
    offsets, sizes, cums, _, total = _kv_waves(Z, H, S, chunks, [0, 1, 2])
    scale = 128 ** -0.5
    ref = numerics.sdpa_fp32(q, k, v, scale, causal=True)
    side = torch.cuda.Stream()
    for stream in (None, side):
        flags = torch.zeros(3, dtype=torch.int64, device="cuda")
        counters = torch.zeros(3, dtype=torch.int32, device="cuda")
        qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
        torch.cuda.synchronize()
        o = attention_forward(qd, kd, vd, scale, wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums,
                              signal_ptr=flags, signal_offsets=[0, 1, 2], cum_tiles=total, causal=True,
                              counter_ptr=counters, spin_timeout_us=200_000, stream=stream)
        if stream is not None:
            stream.synchronize()
        check_status()
        assert counters.tolist() == [Z * H * S // 128] * 3
        assert flags.tolist() == [1, 1, 1]
        assert _rel(o, ref) <= REL_TOL


def test_lock_areas_come_zeroed_across_many_launches(hip):
    """The launcher's lock words come out of a pool that is zero-filled sixteen launches at a time: forty merging
    launches in a row (the pool wraps twice), on the current stream and on another one, each against the fp32
    reference - a launch that found a used lock word would skip or double a merge."""
    from syncopate_amd.computation.attn import attention_forward
    from syncopate_amd.computation._launch import check_status

    Z, H, Sq, Skv = 1, 2, 512, 1024
    q, k, v = _qkv(Z, H, Sq, Skv, torch.bfloat16, seed=77)
    chunks = [(256, 512), (0, 256), (768, 1024), (512, 768)]
    offsets, sizes, cums, signals, total = _kv_waves(Z, H, Sq, chunks, [-1] * 4)
    flags = torch.ones(1, dtype=torch.int64, device="cuda")
    sm_scale = 128 ** -0.5
    ref = numerics.sdpa_fp32(q, k, v, sm_scale)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    for stream in (None, side):
        outs = [attention_forward(qd, kd, vd, sm_scale, wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums,
                                  signal_ptr=flags, signal_offsets=signals, NUM_WAVES=4, cum_tiles=total, num_programs=3,
                                  pair_q_blocks=True, stream=stream) for _ in range(40)]
        check_status()
        for o in outs:
            assert _rel(o, ref) <= REL_TOL
