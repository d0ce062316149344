"""GPU parity of the chunked ring reduce against the CPU oracle: bit-exact."""

import numpy as np
import pytest
import torch

from oracle import numerics

pytestmark = pytest.mark.gpu


def _case(world, rows, N, dtype, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    recv = torch.randn(world, rows, N, generator=g).to(dtype)
    local = torch.randn(world * rows, N, generator=g).to(dtype)
    return recv, local


@pytest.mark.parametrize("dtype,name", [(torch.bfloat16, "bf16"), (torch.float16, "fp16")])
@pytest.mark.parametrize("world,rows,N", [(8, 128, 512), (4, 64, 256), (2, 8, 8), (3, 40, 72),
                                           (16, 16, 128), (1, 16, 64)])
@pytest.mark.parametrize("acc_mode", ["dtype", "fp32"])
def test_ring_reduce_bit_exact(hip, dtype, name, world, rows, N, acc_mode):
    from syncopate_amd.computation.reduce import ring_reduce

    for rank in sorted({0, world - 1, world // 2}):
        recv, local = _case(world, rows, N, dtype, seed=world * 100 + rank)
        want = numerics.ring_reduce(recv.float().numpy(), local.float().numpy(), rank, dtype=name,
                                    round_each_add=(acc_mode == "dtype"))
        recv_d = recv.cuda()
        # the slot of the rank itself is never read: poison it
        recv_d[rank].fill_(float("nan"))
        out = torch.empty(rows, N, dtype=dtype, device="cuda")
        ring_reduce(recv_d, out, local.cuda(), rank, acc_mode=acc_mode)
        got = out.float().cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("world,rows,N", [(8, 128, 512), (3, 40, 72), (1, 16, 64)])
def test_ring_reduce_over_blocks_that_lie_apart(hip, world, rows, N):
    """The received blocks as a [W, rows, N] view of a padded buffer (blocks 4 KiB further apart than
    their size, the gaps poisoned): the same bits as from the contiguous layout."""
    from syncopate_amd.computation.reduce import padded_receive_buffer, ring_reduce

    rank = world // 2
    recv, local = _case(world, rows, N, torch.bfloat16, seed=7 * world)
    want = numerics.ring_reduce(recv.float().numpy(), local.float().numpy(), rank, dtype="bf16", round_each_add=True)
    padded = padded_receive_buffer(world, rows, N, torch.bfloat16, "cuda")
    assert padded.shape == recv.shape and (world == 1 or padded.stride(0) == rows * N + 2048)
    torch.as_strided(padded, (world * (rows * N + 2048),), (1,)).fill_(float("nan"))
    padded.copy_(recv)
    padded[rank].fill_(float("nan"))
    out = torch.empty(rows, N, dtype=torch.bfloat16, device="cuda")
    ring_reduce(padded, out, local.cuda(), rank)
    assert np.array_equal(out.float().cpu().numpy().view(np.uint32), want.view(np.uint32))
    # blocks that are not whole 16-byte groups apart, or that overlap, are refused
    flat = torch.zeros(world * (rows * N + 4) + 8, dtype=torch.bfloat16, device="cuda")
    if world > 1:
        from syncopate_amd import _lib
        with pytest.raises(_lib.SyncopateHipError):
            ring_reduce(torch.as_strided(flat, (world, rows, N), (rows * N + 4, N, 1)), out, local.cuda(), rank)
        with pytest.raises(ValueError):
            ring_reduce(torch.as_strided(flat, (world, rows, N), (rows * N - 8, N, 1)), out, local.cuda(), rank)


def test_ring_reduce_full_size_properties(hip):
    """Benchmark size (8 x (1024, 8192) bf16): integer-valued inputs make every partial sum
    exact, so the result must equal the integer sum whatever the order or rounding."""
    from syncopate_amd.computation.reduce import ring_reduce

    world, rows, N, rank = 8, 1024, 8192, 5
    g = torch.Generator(device="cpu").manual_seed(11)
    recv = torch.randint(-8, 9, (world, rows, N), generator=g).to(torch.bfloat16)
    local = torch.randint(-8, 9, (world * rows, N), generator=g).to(torch.bfloat16)
    want = local[rank * rows:(rank + 1) * rows].float()
    for i in range(1, world):
        want = want + recv[(rank + i) % world].float()
    out = torch.empty(rows, N, dtype=torch.bfloat16, device="cuda")
    for mode in ("dtype", "fp32"):
        ring_reduce(recv.cuda(), out, local.cuda(), rank, acc_mode=mode)
        assert torch.equal(out.float().cpu(), want)


def test_ring_reduce_rejects_bad_arguments(hip):
    from syncopate_amd import _lib
    from syncopate_amd.computation.reduce import ring_reduce

    recv = torch.zeros(4, 3, 5, dtype=torch.bfloat16, device="cuda")     # 15 elements: not 8-divisible
    local = torch.zeros(12, 5, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(3, 5, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_lib.SyncopateHipError):
        ring_reduce(recv, out, local, 0)
    recv = torch.zeros(4, 8, 8, dtype=torch.bfloat16, device="cuda")
    local = torch.zeros(32, 8, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(8, 8, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_lib.SyncopateHipError):
        ring_reduce(recv, out, local, 4)                                  # rank out of range


def test_every_world_size_makes_one_pass_over_its_chunk(hip):
    """World sizes without a kernel of their own (3, 5, 6, 7, 9 ... 16) share a general kernel; like the others it
    reads every received block once.  A launch that walked its chunk once per workgroup gave the same bits a
    thousand times slower - so the bound here is generous: within 20 x of the time of world 8 on the same chunk."""
    from syncopate_amd.computation.reduce import ring_reduce

    rows, n = 512, 8192

    def launch_ms(world):
        g = torch.Generator(device="cuda").manual_seed(world)
        recv = torch.randn(world, rows, n, device="cuda", generator=g).bfloat16()
        local = torch.randn(world * rows, n, device="cuda", generator=g).bfloat16()
        out = torch.empty(rows, n, dtype=torch.bfloat16, device="cuda")
        for _ in range(3):
            ring_reduce(recv, out, local, 1)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(10):
            ring_reduce(recv, out, local, 1)
        stop.record()
        torch.cuda.synchronize()
        acc = local[rows:2 * rows].clone()
        for i in range(1, world):
            acc = acc + recv[(1 + i) % world]
        assert torch.equal(out, acc)
        return start.elapsed_time(stop) / 10

    eight = launch_ms(8)
    for world in (3, 7, 13):
        assert launch_ms(world) < 20 * eight * max(1.0, world / 8), world


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("world", [2, 4, 8])
def test_skewed_walk_of_large_chunks_is_bit_exact(hip, world, dtype):
    """Chunks of at least 16 MiB per block are walked skewed (stream i one 4 KB block behind stream i - 1), plus a
    ragged tail in the plain walk: the sums are those of the ring order, bit for bit, in both accumulation modes'
    default; blocks a multiple of 64 KiB apart but not adjacent take the same path."""
    from syncopate_amd.computation.reduce import ring_reduce

    rows, n, rank = 1024 + 3, 8192, world - 1               # 16 MiB + three rows per block
    g = torch.Generator(device="cuda").manual_seed(7 * world)
    recv = torch.randn(world, rows, n, device="cuda", generator=g).to(dtype)
    local = torch.randn(world * rows, n, device="cuda", generator=g).to(dtype)
    out = torch.full((rows, n), float("nan"), dtype=dtype, device="cuda")
    ring_reduce(recv, out, local, rank)
    acc = local[rank * rows:(rank + 1) * rows].clone()
    for i in range(1, world):
        acc = acc + recv[(rank + i) % world]
    assert torch.equal(out, acc)
    # the same blocks inside a buffer whose blocks are 64 KiB further apart
    apart = rows * n + 32768
    wide = torch.zeros(world * apart, dtype=dtype, device="cuda")
    view = torch.as_strided(wide, (world, rows, n), (apart, n, 1))
    view.copy_(recv)
    out.fill_(float("nan"))
    ring_reduce(view, out, local, rank)
    assert torch.equal(out, acc)
