"""GPU parity of the GEMM forms that bind A or C to a peer's buffer per wave (through the C ABI).

Counterparts in the reference: tests/test_ag_gemm_direct_read.py:150-205 (A read from the owner's
shard), tests/test_gemm_rs_persistent.py and tests/test_gemm_rs_direct_reduce.py:100-192 (C tiles
atomically added into the owner's result; `assert_close(..., atol=1e-2, rtol=1e-2)`).  On one GPU
the peers are tensors of this process and every rank's kernel runs in turn on one stream.
"""

import pytest
import torch

from oracle import numerics, visit_order

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2  # max |err| / max |ref| against torch fp32


def _max_rel_err(out, ref):
    return ((out.float().cpu() - ref).abs().max() / ref.abs().max()).item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("BM,BN,eight", [(128, 256, False), (256, 256, False), (256, 128, True)])
def test_ag_direct_read_matches_gathered_gemm(hip, dtype, BM, BN, eight):
    from syncopate_amd.computation.gemm import gemm_ag_direct_read, gemm_consumer
    from syncopate_amd.computation._launch import check_status

    world, rank, rows, K, N = 4, 2, 512, 384, 768
    M = world * rows
    g = torch.Generator().manual_seed(5)
    shards = [(0.02 * torch.randn(rows, K, generator=g)).to(dtype) for _ in range(world)]
    b = (0.02 * torch.randn(N, K, generator=g)).to(dtype)
    ref = numerics.gemm_fp32(torch.cat(shards), b)

    order = [(rank + k) % world for k in range(world)]
    sizes = [[rows, N]] * world
    offsets = [[r * rows, 0] for r in order]
    dshards = [s.cuda() for s in shards]
    c = torch.zeros(M, N, dtype=dtype, device="cuda")
    log = torch.full(((M // BM) * (N // BN), 4), -1, dtype=torch.int32, device="cuda")
    gemm_ag_direct_read(dshards, b.cuda(), c, sizes, offsets, order, world, world, 61, True, BM, BN, 64, 8,
                        visit_log=log, eight_waves=eight)
    check_status()
    assert _max_rel_err(c, ref) <= REL_TOL

    # same tiles, same K order: bitwise equal to the consumer over the gathered buffer
    c2 = torch.zeros_like(c)
    flags = torch.ones(1, dtype=torch.int64, device="cuda")
    gemm_consumer(torch.cat(dshards), b.cuda(), c2, flags, sizes, offsets, [-1] * world, world, 61, BM, BN,
                  cum_tiles=M * N, eight_waves=eight)
    check_status()
    assert torch.equal(c, c2)

    want = visit_order.gemm_tile_visits(sizes, offsets, [-1] * world, M=M, N=N, BM=BM, BN=BN, group_m=8,
                                        num_sms=61, cum_tiles=M * N)
    got = log.cpu().view(-1, 4).tolist()
    for v in want:
        assert tuple(got[v["tile_id"]]) == (v["pid"], v["wave"], v["pid_m"], v["pid_n"])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rs_persistent_atomic_add_over_all_ranks(hip, dtype):
    """Every rank's partial product lands in the owners' [M / W, N] buffers by packed atomics."""
    from syncopate_amd.computation.gemm import gemm_rs_producer_persistent
    from syncopate_amd.computation._launch import check_status

    world, M, N, K_local, BM, BN = 4, 1024, 512, 256, 128, 256
    rows = M // world
    g = torch.Generator().manual_seed(9)
    a = [(0.02 * torch.randn(M, K_local, generator=g)).to(dtype) for _ in range(world)]
    b = [(0.02 * torch.randn(N, K_local, generator=g)).to(dtype) for _ in range(world)]
    ref = sum(numerics.gemm_fp32(a[r], b[r]) for r in range(world))

    outs = [torch.zeros(rows, N, dtype=dtype, device="cuda") for _ in range(world)]
    for r in range(world):
        # remote rows first, own rows last (template_rs.py:363)
        order = [(r + k + 1) % world for k in range(world)]
        sizes = [[rows, N]] * world
        offsets = [[t * rows, 0] for t in order]
        gemm_rs_producer_persistent(a[r].cuda(), b[r].cuda(), outs, sizes, offsets, order, world, world,
                                    64 + r, BM, BN, 64, 8)
    check_status()
    got = torch.cat(outs).float().cpu()
    # the reference's own bound for this path (tests/test_gemm_rs_direct_reduce.py:192)
    torch.testing.assert_close(got, ref, atol=1e-2, rtol=1e-2)
    assert _max_rel_err(torch.cat(outs), ref) <= 2 * REL_TOL   # W-1 roundings to 16 bits on top of the GEMM's


def test_generated_form_store_with_dst_offsets_and_flags(hip):
    """`gemm_remote` as the transform pass emits it: target_rank / dst_offsets per wave, plain
    stores, waves that split N, a flag per wave."""
    from syncopate_amd.computation.gemm import gemm_remote
    from syncopate_amd.computation._launch import check_status

    M, N, K, BM, BN = 512, 1024, 192, 128, 128
    g = torch.Generator().manual_seed(11)
    a = (0.02 * torch.randn(M, K, generator=g)).bfloat16()
    b = (0.02 * torch.randn(N, K, generator=g)).bfloat16()
    ref = numerics.gemm_fp32(a, b)
    # four waves = quadrants; quadrant q goes to peer q % 2 at a shifted position of a wider buffer
    sizes = [[256, 512]] * 4
    offsets = [[0, 0], [256, 512], [0, 512], [256, 0]]
    targets = [0, 1, 1, 0]
    dst = [[128, 256], [0, 0], [256, 768], [384, 1024]]
    ldc, peer_rows = 1536, 640
    peers = [torch.full((peer_rows, ldc), 7.0, dtype=torch.bfloat16, device="cuda") for _ in range(2)]
    flags = torch.ones(4, dtype=torch.int64, device="cuda")
    gemm_remote(a.cuda(), b.cuda(), peers, 32, BM, BN, 64, 2, cur_wave_sizes=sizes, wave_offsets=offsets, M=M,
                target_rank=targets, dst_offsets=dst, signal_ptr=flags, signal_offsets=[0, 1, 2, 3],
                cum_tiles=M * N)
    check_status()
    touched = [torch.zeros(peer_rows, ldc, dtype=torch.bool) for _ in range(2)]
    for (sm, sn), (om, on), t, (dm, dn) in zip(sizes, offsets, targets, dst):
        block = peers[t][dm:dm + sm, dn:dn + sn]
        want = ref[om:om + sm, on:on + sn]
        assert ((block.float().cpu() - want).abs().max() / ref.abs().max()).item() <= REL_TOL
        touched[t][dm:dm + sm, dn:dn + sn] = True
    for t in range(2):
        # nothing outside the waves' regions was written
        assert torch.all(peers[t].cpu()[~touched[t]] == 7.0)


def test_remote_argument_errors(hip):
    from syncopate_amd.computation.gemm import gemm_remote

    a = torch.zeros(256, 64, dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(256, 64, dtype=torch.bfloat16, device="cuda")
    c = torch.zeros(256, 256, dtype=torch.bfloat16, device="cuda")
    kw = dict(cur_wave_sizes=[[256, 256]], wave_offsets=[[0, 0]], M=256, cum_tiles=256 * 256)
    with pytest.raises(ValueError):
        gemm_remote(a, b, c, 8, 128, 128, **kw)                       # nothing bound to a peer
    with pytest.raises(ValueError):
        gemm_remote(a, b, [c], 8, 128, 128, target_rank=[1], dst_offsets=[[0, 0]], **kw)   # rank out of range
    with pytest.raises(ValueError):
        gemm_remote(a, b, [c], 8, 128, 128, target_rank=[0], dst_offsets=[[128, 0]], **kw)  # does not fit
    with pytest.raises(ValueError):
        gemm_remote([a[:128]], b, c, 8, 128, 128, a_target_rank=[0], **kw)   # wave taller than the shard


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("BM,BN,chunks", [(128, 256, [(256, 128), (0, 64), (64, 192), (384, 128)]),
                                          (256, 256, [(0, 256), (256, 256)]),
                                          (128, 128, [(448, 64), (0, 448)])])
def test_split_k_waves_add_up_to_the_product(hip, dtype, BM, BN, chunks):
    """Waves that each contract over part of K (first k, count) and add their partial product into
    C: the transformed split-K GEMM of the reference (tests/computation/transform/examples/
    example_splitk_gemm.py:36-112), whose K chunks arrive one by one (tests/test_all2all_gemm.py:
    94-103 builds the three-column tables)."""
    from syncopate_amd.computation.gemm import gemm_splitk
    from syncopate_amd.computation._launch import check_status

    M, N, K = 512, 512, 512
    g = torch.Generator().manual_seed(21)
    a = (0.05 * torch.randn(M, K, generator=g)).to(dtype)
    b = (0.05 * torch.randn(N, K, generator=g)).to(dtype)
    ref = numerics.gemm_fp32(a, b)
    sizes = [[M, N, count] for _, count in chunks]
    offsets = [[0, 0, first] for first, _ in chunks]
    flags = torch.ones(len(chunks), dtype=torch.int64, device="cuda")
    c = torch.zeros(M, N, dtype=dtype, device="cuda")
    gemm_splitk(a.cuda(), b.cuda(), c, 1, 37, BM, BN, 64, 8, cur_wave_sizes=sizes, wave_offsets=offsets,
                signal_ptr=flags, signal_offsets=list(range(len(chunks))), cum_tiles=len(chunks) * M * N)
    check_status()
    # one rounding to 16 bits per chunk on top of the product's
    assert _max_rel_err(c, ref) <= len(chunks) * REL_TOL
    torch.testing.assert_close(c.float().cpu(), ref, atol=2e-2, rtol=2e-2)
    # each chunk alone is the product over its columns
    for (first, count), size, off in zip(chunks, sizes, offsets):
        part = torch.zeros(M, N, dtype=dtype, device="cuda")
        gemm_splitk(a.cuda(), b.cuda(), part, 1, 16, BM, BN, 64, 8, cur_wave_sizes=[size], wave_offsets=[off],
                    cum_tiles=M * N)
        want = numerics.gemm_fp32(a[:, first:first + count], b[:, first:first + count])
        assert ((part.float().cpu() - want).abs().max() / ref.abs().max()).item() <= REL_TOL
    check_status()


def test_split_k_argument_errors(hip):
    from syncopate_amd.computation.gemm import gemm_remote, gemm_splitk

    a = torch.zeros(256, 256, dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(256, 256, dtype=torch.bfloat16, device="cuda")
    c = torch.zeros(256, 256, dtype=torch.bfloat16, device="cuda")
    kw = dict(cum_tiles=256 * 256)
    with pytest.raises(ValueError, match="multiples of 64"):
        gemm_splitk(a, b, c, 1, 8, 128, 128, cur_wave_sizes=[[256, 256, 96]], wave_offsets=[[0, 0, 0]], **kw)
    with pytest.raises(ValueError, match="past K"):
        gemm_splitk(a, b, c, 1, 8, 128, 128, cur_wave_sizes=[[256, 256, 128]], wave_offsets=[[0, 0, 192]], **kw)
    with pytest.raises(ValueError, match="added into"):
        gemm_remote(a, b, [c], 8, 128, 128, cur_wave_sizes=[[256, 256]], wave_offsets=[[0, 0]], M=256,
                    target_rank=[0], dst_offsets=[[0, 0]], k_ranges=[[0, 128]], **kw)      # plain stores
