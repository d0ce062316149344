"""Pins of the CPU oracle itself: reference-held vectors, closed forms, library routines,
brute force.  Nothing here touches the GPU."""

import itertools
import math

import numpy as np
import pytest
import torch

from oracle import numerics, visit_order


# ---------------------------------------------------------------- tile visit order

def _dispatch(tile_id, wave_offsets, wave_sizes, cum_wave_sizes, group_m):
    wave = next(i for i, c in enumerate(cum_wave_sizes) if tile_id < c)
    prev = 0 if wave == 0 else cum_wave_sizes[wave - 1]
    pm, pn = visit_order.get_pid_mn(tile_id - prev, wave_sizes[wave][0], wave_sizes[wave][1], group_m)
    return pm + wave_offsets[wave][0], pn + wave_offsets[wave][1]


# literal tile orders of the reference's transform-pass test
# (tests/computation/transform/test_transform_pass.py:253-291)
REFERENCE_ORDERS = [
    (8, [(0, 0)], [(4, 2)], [8],
     [(0, 0), (1, 0), (2, 0), (3, 0), (0, 1), (1, 1), (2, 1), (3, 1)]),
    (8, [(0, 0), (2, 0)], [(2, 2), (2, 2)], [4, 8],
     [(0, 0), (1, 0), (0, 1), (1, 1), (2, 0), (3, 0), (2, 1), (3, 1)]),
]


@pytest.mark.parametrize("group_m,offsets,sizes,cums,expected", REFERENCE_ORDERS)
def test_wave_dispatch_reproduces_reference_orders(group_m, offsets, sizes, cums, expected):
    assert [_dispatch(t, offsets, sizes, cums, group_m) for t in range(cums[-1])] == expected


@pytest.mark.parametrize("num_m,num_n,group_m", [(5, 7, 4), (3, 2, 2), (8, 14, 8), (7, 1, 4), (1, 9, 3)])
def test_get_pid_mn_is_a_bijection_with_grouped_columns(num_m, num_n, group_m):
    seen = [visit_order.get_pid_mn(t, num_m, num_n, group_m) for t in range(num_m * num_n)]
    assert sorted(seen) == sorted(itertools.product(range(num_m), range(num_n)))
    # full groups: m runs fastest inside a group, groups advance after group_m * num_n tiles
    for t, (pm, pn) in enumerate(seen):
        g = t // (group_m * num_n)
        assert g * group_m <= pm < min(num_m, (g + 1) * group_m)
        if (g + 1) * group_m <= num_m:
            assert (pm, pn) == (g * group_m + t % group_m, (t % (group_m * num_n)) // group_m)


def test_worked_example_of_the_headline_configuration():
    """AG-GEMM 8192x3584, rank 0 of 8, 128x256 tiles, 256 programs: wave k = tiles [112k, 112k+112),
    tile t of a wave -> (8k + t % 8, t // 8); program 200 visits tiles 200, 456, 712."""
    sizes = [[1024, 3584]] * 8
    offsets = [[1024 * k, 0] for k in range(8)]
    signals = [-1, 0, 1, 2, 3, 4, 5, 6]
    visits = visit_order.gemm_tile_visits(sizes, offsets, signals, M=8192, N=3584, BM=128, BN=256,
                                          group_m=8, num_sms=256, cum_tiles=8192 * 3584)
    assert len(visits) == 896
    for v in visits:
        k, t = divmod(v["tile_id"], 112)
        assert (v["wave"], v["pid_m"], v["pid_n"]) == (k, 8 * k + t % 8, t // 8)
        assert (v["pid"], v["iter"]) == (v["tile_id"] % 256, v["tile_id"] // 256)
    mine = [v for v in visits if v["pid"] == 200]
    assert [(v["tile_id"], v["wave"], v["pid_m"], v["pid_n"], v["waited_signal"]) for v in mine] == [
        (200, 1, 8, 11, 0), (456, 4, 32, 1, 3), (712, 6, 48, 5, 5)]
    assert sum(1 for v in visits if v["pid"] == 127) == 4 and sum(1 for v in visits if v["pid"] == 128) == 3


def test_random_wave_tables_cover_every_tile_once():
    rng = np.random.default_rng(0)
    for _ in range(50):
        BM, BN = int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4]))
        tiles_m, tiles_n = int(rng.integers(1, 7)), int(rng.integers(1, 7))
        cuts = sorted(set(rng.integers(1, tiles_m + 1, size=2).tolist()) | {tiles_m})
        sizes, offsets, lo = [], [], 0
        for hi in cuts:
            sizes.append([(hi - lo) * BM, tiles_n * BN])
            offsets.append([lo * BM, 0])
            lo = hi
        order = rng.permutation(len(sizes))
        sizes, offsets = [sizes[i] for i in order], [offsets[i] for i in order]
        signals = [-1] + list(range(len(sizes) - 1))
        M, N = tiles_m * BM, tiles_n * BN
        visits = visit_order.gemm_tile_visits(sizes, offsets, signals, M=M, N=N, BM=BM, BN=BN,
                                              group_m=int(rng.integers(1, 5)), num_sms=int(rng.integers(1, 12)),
                                              cum_tiles=M * N)
        assert sorted((v["pid_m"], v["pid_n"]) for v in visits) == sorted(
            itertools.product(range(tiles_m), range(tiles_n)))
        waves = [v["wave"] for v in visits]
        assert waves == sorted(waves)                      # waves are contiguous in tile-id order
        for v in visits:
            w = v["wave"]
            assert offsets[w][0] // BM <= v["pid_m"] < (offsets[w][0] + sizes[w][0]) // BM


def test_attention_tile_work_covers_every_q_kv_pair_once():
    # all-to-all style table: 3 chunks, all (q chunk, kv chunk) pairs in arrival order
    Z, H, chunk, bm = 2, 3, 256, 128
    offsets, sizes, cums, sigs, total = [], [], [], [], 0
    pairs = [(0, 0), (1, 1), (0, 1), (1, 0), (2, 2), (0, 2), (2, 0), (1, 2), (2, 1)]
    for qc, kc in pairs:
        offsets.append([0, 0, qc * chunk, kc * chunk])
        sizes.append([Z, H, chunk, chunk])
        total += Z * H * chunk
        cums.append(total)
        sigs.append(max(qc, kc) - 1)
    seen = []
    for t in range(total // bm):
        w = visit_order.attn_tile_work(t, offsets, sizes, cums, sigs)
        assert w["signal"] == sigs[w["wave"]]
        for kv in range(w["kv_lo"], w["kv_hi"]):
            seen.append((w["z"], w["h"], w["q_block"], kv))
    blocks = 3 * chunk // bm
    assert sorted(seen) == sorted(itertools.product(range(Z), range(H), range(blocks), range(blocks)))
    with pytest.raises(IndexError):
        visit_order.attn_tile_work(total // bm, offsets, sizes, cums, sigs)


def test_attention_in_wave_order_matches_the_reference_generated_dispatch():
    """The golden tuples come from the reference's own generated dispatch text evaluated tile by
    tile (tests/golden/make_attn_dispatch_fixtures.py): q fastest, then h, then z inside a wave
    (attn/template.py:39-44), wave offsets added afterwards (transformer.py:561-676)."""
    import json
    import os

    golden = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "attn_dispatch_cases.json")))
    bm, bn = golden["block_m"], golden["block_n"]
    assert set(golden["cases"]) >= {"one_wave_z2_h3_q2", "ragged_offsets", "double_ring_w8_small"}
    for name, case in golden["cases"].items():
        assert len(case["tiles"]) == case["cum_wave_sizes"][-1] // bm
        for tile_id, expect in enumerate(case["tiles"]):
            w = visit_order.attn_tile_work(tile_id, case["wave_offsets"], case["wave_sizes"],
                                           case["cum_wave_sizes"], case["signal_offsets"], block_m=bm, block_n=bn)
            got = [w["wave"], w["z"], w["h"], w["q_block"], w["kv_lo"], w["kv_hi"], w["signal"]]
            assert got == expect, (name, tile_id, got, expect)


def test_attention_in_wave_order_hand_evaluated_literal():
    """get_pid_range (attn/template.py:39-44) by hand for Z=2, H=3, two q blocks:
    tile t -> q = t % 2, h = (t // 2) % 3, z = t // 6.  Swapping any two of z, h, q fails it."""
    expect_zhq = [(0, 0, 0), (0, 0, 1), (0, 1, 0), (0, 1, 1), (0, 2, 0), (0, 2, 1),
                  (1, 0, 0), (1, 0, 1), (1, 1, 0), (1, 1, 1), (1, 2, 0), (1, 2, 1)]
    offsets, sizes, cums, sigs = [[0, 0, 0, 0]], [[2, 3, 256, 384]], [2 * 3 * 256], [-1]
    for t, (z, h, q) in enumerate(expect_zhq):
        w = visit_order.attn_tile_work(t, offsets, sizes, cums, sigs)
        assert (w["z"], w["h"], w["q_block"], w["kv_lo"], w["kv_hi"]) == (z, h, q, 0, 3)
    # a second wave at offsets (z 1, h 2, q block 1, kv block 2) of shape 1 x 2 x 2 q blocks x 1 kv block
    offsets, sizes, cums, sigs = [[0, 0, 0, 0], [1, 2, 128, 256]], [[1, 1, 128, 128], [1, 2, 256, 128]], [128, 128 + 512], [-1, 3]
    got = [visit_order.attn_tile_work(t, offsets, sizes, cums, sigs) for t in range(5)]
    assert [(g["wave"], g["z"], g["h"], g["q_block"], g["kv_lo"], g["kv_hi"], g["signal"]) for g in got] == [
        (0, 0, 0, 0, 0, 1, -1), (1, 1, 2, 1, 2, 3, 3), (1, 1, 2, 2, 2, 3, 3), (1, 1, 3, 1, 2, 3, 3), (1, 1, 3, 2, 2, 3, 3)]


# ---------------------------------------------------------------- rounding and ring reduce

def test_bf16_rounding_is_round_to_nearest_even():
    # bf16 has 8 significand bits: ulp(1.0) = 2^-7
    x = np.array([1.0, 1 + 2.0 ** -8, 1 + 2.0 ** -7 + 2.0 ** -8, 1 + 2.0 ** -7 + 2.0 ** -9,
                  1 + 2.0 ** -7 + 2.0 ** -8 + 2.0 ** -12], dtype=np.float32)
    #             exact  tie -> even (down)  tie -> even (up)          below the tie
    #             above the tie
    want = np.array([1.0, 1.0, 1 + 2.0 ** -6, 1 + 2.0 ** -7, 1 + 2.0 ** -6], dtype=np.float32)
    assert np.array_equal(numerics.round_to(x, "bf16"), want)
    rng = np.random.default_rng(1)
    r = (rng.standard_normal(200000) * np.exp(rng.uniform(-20, 20, 200000))).astype(np.float32)
    assert np.array_equal(numerics.round_to(r, "bf16"), torch.from_numpy(r).bfloat16().float().numpy())
    assert np.array_equal(numerics.round_to(r, "fp16")[np.abs(r) < 6e4],
                          torch.from_numpy(r).half().float().numpy()[np.abs(r) < 6e4])


@pytest.mark.parametrize("dtype,tdtype", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_ring_reduce_equals_sequential_adds_in_the_tensor_dtype(dtype, tdtype):
    """acc += data on 16-bit tensors: torch's own bf16/fp16 addition is the library routine."""
    g = torch.Generator().manual_seed(3)
    world, rows, n, rank = 5, 7, 24, 3
    recv = torch.randn(world, rows, n, generator=g).to(tdtype)
    local = torch.randn(world * rows, n, generator=g).to(tdtype)
    acc = local[rank * rows:(rank + 1) * rows].clone()
    for i in range(1, world):
        acc = acc + recv[(rank + i) % world]
    got = numerics.ring_reduce(recv.float().numpy(), local.float().numpy(), rank, dtype=dtype)
    assert np.array_equal(got, acc.float().numpy())
    once = numerics.ring_reduce(recv.float().numpy(), local.float().numpy(), rank, dtype=dtype,
                                round_each_add=False)
    tot = local[rank * rows:(rank + 1) * rows].float()
    for i in range(1, world):
        tot = tot + recv[(rank + i) % world].float()
    assert np.array_equal(once, tot.to(tdtype).float().numpy())


def test_ring_reduce_order_matters_and_is_the_ring_order():
    """1 + 2^-8 + 2^-8 in bf16: (1 + 2^-8) rounds to 1 twice, but 2^-8 + 2^-8 first gives 1 + 2^-7."""
    tiny = 2.0 ** -8
    recv = np.zeros((3, 1, 8), dtype=np.float32)
    local = np.zeros((3, 8), dtype=np.float32)
    local[0], recv[1], recv[2] = 1.0, tiny, tiny          # rank 0: 1, then rank 1, then rank 2
    assert numerics.ring_reduce(recv, local, 0)[0, 0] == 1.0
    local[:] = 0
    recv[:] = 0
    local[1], recv[2], recv[0] = tiny, tiny, 1.0          # rank 1: tiny + tiny, then rank 0's 1.0
    assert numerics.ring_reduce(recv, local, 1)[0, 0] == 1.0 + 2.0 ** -7


# ---------------------------------------------------------------- attention

@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("order", [[0, 1, 2, 3], [2, 0, 3, 1]])
def test_chunked_attention_reduces_to_sdpa(causal, order):
    g = torch.Generator().manual_seed(7)
    Z, H, S, D = 1, 2, 512, 128
    q = torch.randn(Z, H, S, D, generator=g).bfloat16()
    k = torch.randn(Z, H, S, D, generator=g).bfloat16()
    v = torch.randn(Z, H, S, D, generator=g).bfloat16()
    chunks = [(128 * c, 128 * (c + 1)) for c in order]
    scale = D ** -0.5
    o, lse2 = numerics.chunked_attention(q, k, v, scale, chunks, causal=causal)
    ref = numerics.sdpa_fp32(q, k, v, scale, causal=causal)
    assert (o.float() - ref).abs().max() / ref.abs().max() <= 1e-2
    s = (q.float() @ k.float().transpose(-1, -2)) * scale
    if causal:
        s = s.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), 1), float("-inf"))
    assert (lse2 - torch.logsumexp(s, -1) / math.log(2)).abs().max() <= 1e-2
    exact, _ = numerics.chunked_attention(q, k, v, scale, chunks, causal=causal, round_merges=False)
    assert (exact.float() - ref).abs().max() <= (o.float() - ref).abs().max() + 1e-3


def test_lse_merge_identity():
    """max + log2(1 + 2^-|d|) == log2(2^a + 2^b) (syncopate/computation/attn/template.py:339-346)."""
    a = torch.tensor([3.0, -2.0, 10.0, 0.0])
    b = torch.tensor([1.0, 5.0, 10.0, -40.0])
    merged = torch.maximum(a, b) + torch.log2(1 + torch.exp2(-(a - b).abs()))
    assert torch.allclose(merged, torch.log2(torch.exp2(a) + torch.exp2(b)), atol=1e-6)
