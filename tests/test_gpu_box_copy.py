"""GPU parity of the box copy / accumulate kernel behind SMCopyOp (through the C ABI).

Counterpart in the reference: persistent_naive_copy_last_contig / persistent_tma_copy_last_contig
(comm_runtime/non_tma_persistent_copy.py:191-304), used by tests/test_gemm_rs_sm_reduce.py:105-175.
Copies are bit-exact against slicing on the CPU; sums are checked against one addition in the
element type (the reference bounds the same path by atol = rtol = 1e-2).
"""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _fill(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype.is_floating_point:
        return torch.randn(shape, generator=g).to(dtype)
    info = torch.iinfo(dtype)
    return torch.randint(max(info.min, -2 ** 40), min(info.max, 2 ** 40), shape, generator=g, dtype=dtype)


BOXES = [
    # (source shape, source box, destination shape, destination box)
    ((64, 256), ((8, 40), (0, 256)), (32, 256), ((0, 32), (0, 256))),             # whole rows: one dense run
    ((64, 256), ((8, 40), (64, 192)), (48, 512), ((16, 48), (256, 384))),         # 16-byte aligned columns
    ((33, 77), ((1, 30), (3, 70)), (40, 90), ((5, 34), (11, 78))),                # nothing aligned
    ((4, 6, 50, 24), ((1, 3), (2, 5), (10, 45), (8, 24)), (2, 8, 64, 16), ((0, 2), (4, 7), (20, 55), (0, 16))),
    ((2, 3, 4, 5, 64), ((0, 2), (1, 3), (0, 4), (2, 5), (16, 48)),
     (2, 2, 4, 3, 32), ((0, 2), (0, 2), (0, 4), (0, 3), (0, 32))),                # five dimensions
    ((1, 1, 128), ((0, 1), (0, 1), (5, 99)), (200,), ((101, 195),)),              # leading 1-extents dropped
    ((300000,), ((7, 299999),), (300000,), ((1, 299993),)),                       # long row, many rounds per lane
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.uint8, torch.int64])
@pytest.mark.parametrize("case", range(len(BOXES)))
@pytest.mark.parametrize("blocks", [3, 64])
def test_copy_is_bit_exact_and_stays_in_the_box(hip, dtype, case, blocks):
    from syncopate_amd.communication.comm_runtime.persistent_copy import persistent_naive_copy_last_contig

    sshape, sbox, dshape, dbox = BOXES[case]
    src = _fill(sshape, dtype, 3 + case)
    dst = _fill(dshape, dtype, 50 + case)
    ssl = tuple(slice(a, b) for a, b in sbox)
    dsl = tuple(slice(a, b) for a, b in dbox)
    want = dst.clone()
    want[dsl] = src[ssl].reshape(want[dsl].shape)
    ddev, sdev = dst.cuda(), src.cuda()
    s_view, d_view = sdev[ssl], ddev[dsl]
    if s_view.dim() != d_view.dim():
        d_view = d_view.reshape((1,) * (s_view.dim() - d_view.dim()) + tuple(d_view.shape))
    got = persistent_naive_copy_last_contig(s_view, d_view, num_sms=blocks)
    assert got.data_ptr() == d_view.data_ptr()
    torch.cuda.synchronize()
    assert torch.equal(ddev.cpu().view(torch.uint8), want.view(torch.uint8))
    assert torch.equal(sdev.cpu().view(torch.uint8), src.view(torch.uint8))


def _signed(shape, dtype, seed, low, high):
    """Random signs, magnitudes in [low, high): sums of a [0.5, 2) and a [4, 8) operand stay normal
    numbers, so flushing of subnormals (which the atomic units may do) cannot show."""
    g = torch.Generator().manual_seed(seed)
    mag = low + (high - low) * torch.rand(shape, generator=g)
    sign = torch.randint(0, 2, shape, generator=g).float() * 2 - 1
    return (mag * sign).to(dtype)


def _ulps(a, b, dtype):
    bits = torch.int16 if dtype != torch.float32 else torch.int32
    return (a.contiguous().view(bits).long() - b.contiguous().view(bits).long()).abs().max().item()


@pytest.mark.parametrize("exclusive", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("case", range(len(BOXES)))
def test_sum_adds_once_in_the_element_type(hip, dtype, case, exclusive):
    from syncopate_amd.communication.comm_runtime.persistent_copy import persistent_tma_copy_last_contig
    from syncopate_amd.communication.descriptor import ReduceOp

    sshape, sbox, dshape, dbox = BOXES[case]
    src = _signed(sshape, dtype, 7 + case, 0.5, 2.0)
    dst = _signed(dshape, dtype, 90 + case, 4.0, 8.0)
    ssl = tuple(slice(a, b) for a, b in sbox)
    dsl = tuple(slice(a, b) for a, b in dbox)
    want = dst.clone()
    want[dsl] = (dst[dsl].float() + src[ssl].reshape(dst[dsl].shape).float()).to(dtype)
    ddev, sdev = dst.cuda(), src.cuda()
    s_view, d_view = sdev[ssl], ddev[dsl]
    if s_view.dim() != d_view.dim():
        d_view = d_view.reshape((1,) * (s_view.dim() - d_view.dim()) + tuple(d_view.shape))
    persistent_tma_copy_last_contig(s_view, d_view, num_sms=16, reduce_op=ReduceOp.SUM, exclusive=exclusive)
    torch.cuda.synchronize()
    got = ddev.cpu()
    outside = torch.ones(dshape, dtype=torch.bool)
    outside[dsl] = False
    assert torch.equal(got[outside].view(torch.uint8), dst[outside].view(torch.uint8))
    # normal numbers in, normal numbers out: the atomic units round like an add in the type,
    # and so does the plain read-modify-write of the exclusive form
    assert _ulps(got[dsl], want[dsl], dtype) == 0
    torch.testing.assert_close(got.float(), want.float(), atol=1e-2, rtol=1e-2)


def test_concurrent_senders_accumulate_atomically(hip):
    """Four streams add four different boxes into one destination at a time: with atomic adds
    nothing is lost (fp32 values chosen so that every order of additions gives the same bits)."""
    from syncopate_amd.communication.comm_runtime.persistent_copy import persistent_copy_last_contig
    from syncopate_amd.communication.descriptor import ReduceOp

    rows, cols = 2048, 1024
    g = torch.Generator().manual_seed(1)
    parts = [torch.randint(-1000, 1000, (rows, cols), generator=g).float() for _ in range(4)]
    dst = torch.zeros(rows, cols, dtype=torch.float32, device="cuda")
    dev = [p.cuda() for p in parts]
    streams = [torch.cuda.Stream() for _ in parts]
    torch.cuda.synchronize()
    for _ in range(3):
        for s, p in zip(streams, dev):
            persistent_copy_last_contig(p, dst, num_sms=32, reduce_op=ReduceOp.SUM, stream=s)
    torch.cuda.synchronize()
    assert torch.equal(dst.cpu(), 3 * sum(parts))


def test_argument_errors(hip):
    from syncopate_amd.communication.comm_runtime.persistent_copy import persistent_copy_last_contig
    from syncopate_amd.communication.descriptor import ReduceOp

    a = torch.zeros(8, 16, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        persistent_copy_last_contig(a, torch.zeros(8, 8, dtype=torch.bfloat16, device="cuda"))      # shape
    with pytest.raises(ValueError):
        persistent_copy_last_contig(a, torch.zeros(8, 16, dtype=torch.float16, device="cuda"))      # dtype
    with pytest.raises(ValueError):
        persistent_copy_last_contig(a.t(), torch.zeros(16, 8, dtype=torch.bfloat16, device="cuda").t().t())  # stride
    with pytest.raises(ValueError):
        persistent_copy_last_contig(torch.zeros(2, 2, 2, 2, 2, 2, device="cuda"), torch.zeros(2, 2, 2, 2, 2, 2, device="cuda"))
    with pytest.raises(ValueError):
        persistent_copy_last_contig(a, torch.zeros_like(a), num_sms=0)
    with pytest.raises(ValueError):
        persistent_copy_last_contig(a, torch.zeros_like(a), reduce_op=ReduceOp.MAX)
    i = torch.zeros(8, 16, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        persistent_copy_last_contig(i, torch.zeros_like(i), reduce_op=ReduceOp.SUM)
    with pytest.raises(ValueError):
        persistent_copy_last_contig(a.cpu(), a)
    # an empty box is a no-op
    e = torch.zeros(0, 16, dtype=torch.bfloat16, device="cuda")
    assert persistent_copy_last_contig(e, torch.zeros_like(e)).numel() == 0
