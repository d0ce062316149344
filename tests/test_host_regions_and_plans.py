"""Host compiler, regions and plan builders, checked against the vectors the reference's
own CPU tests hold (tests/test_descriptor.py of the reference; line numbers per case)."""

import pytest
import torch

from syncopate_amd.communication.common_descriptors import (
    build_all_gather_plan_1d_swizzle,
    build_all_to_all_plan,
    build_all_to_all_plan_dim,
    build_double_ring_all_gather_plan,
    build_reduce_scatter_direct_reduce_plan,
    build_ring_all_gather_plan,
)
from syncopate_amd.communication.common_descriptors.utils import row_major_strides
from syncopate_amd.communication.descriptor import (
    BufferRegion,
    CommPlan,
    DevicePlan,
    MemorySegment,
    ReduceOp,
    Transfer,
    TransferOp,
)

F16, F32 = torch.float16, torch.float32


def _gather(rank, kind, shape=(16, 2), mesh=4, name="buf"):
    return build_all_gather_plan_1d_swizzle(shape=shape, dtype=F16, axis=0, mesh_size=mesh, rank=rank,
                                            buffer_name=name, transfer_kind=kind)


# ---------------------------------------------------------------- regions (reference :294-333)

def test_region_of_row_block_is_one_segment():
    region = BufferRegion.from_slices(elem_size=2, strides=row_major_strides((4, 2)), slices=[(2, 4), (0, 2)])
    assert region.to_segments() == (MemorySegment(8, 8),)
    assert region.describe() == "[2:4, 0:2]"
    assert region.is_contiguous() and region.total_nbytes() == 8


def test_region_split_along_axes():
    region = BufferRegion.from_slices(elem_size=4, strides=row_major_strides((8, 4)), slices=[(0, 8), (0, 4)])
    rows = region.split(4, axis=0)
    assert [p.describe() for p in rows] == ["[0:2, 0:4]", "[2:4, 0:4]", "[4:6, 0:4]", "[6:8, 0:4]"]
    cols = region.split(2, axis=1)
    assert [p.describe() for p in cols] == ["[0:8, 0:2]", "[0:8, 2:4]"]
    assert sum(p.total_nbytes() for p in rows) == sum(p.total_nbytes() for p in cols) == region.total_nbytes()
    # a column block of a row-major matrix is one segment per row
    assert [s.offset for s in cols[1].to_segments()] == [8 + 16 * r for r in range(8)]
    assert region.split(1) == [region]
    # ragged split: cdiv(8, 3) = 3 rows per piece
    assert [p.describe() for p in region.split(3, axis=0)] == ["[0:3, 0:4]", "[3:6, 0:4]", "[6:8, 0:4]"]
    with pytest.raises(IndexError):
        region.split(2, axis=2)


def test_segments_merge_and_sort_and_strided_constructor():
    region = BufferRegion.from_segments([(16, 8), (0, 8), (8, 8)])
    assert region.to_segments() == (MemorySegment(0, 24),)
    assert region.as_slice() is None          # three boxes, even though they merge
    assert BufferRegion.contiguous(4, 12).as_slice() == slice(4, 16)
    strided = BufferRegion.strided(base_offset=32, segment_bytes=8, stride=16, count=2)
    assert [(s.offset, s.nbytes) for s in strided.to_segments()] == [(32, 8), (48, 8)]
    assert strided.describe() == "{[32:40], [48:56]}"
    multi = BufferRegion.from_multi_slices(elem_size=1, strides=(4, 1), regions=[[(0, 1), (0, 4)], [(1, 2), (0, 4)]])
    assert multi.to_segments() == (MemorySegment(0, 8),)


def test_region_byte_split_walks_segments():
    region = BufferRegion.from_segments([(0, 8), (16, 8)])
    parts = region.split(4)
    assert [[(s.offset, s.nbytes) for s in p.to_segments()] for p in parts] == [
        [(0, 4)], [(4, 4)], [(16, 4)], [(20, 4)]]
    thirds = region.split(3)      # cdiv(16, 3) = 6 bytes: the middle piece straddles the gap
    assert [[(s.offset, s.nbytes) for s in p.to_segments()] for p in thirds] == [
        [(0, 6)], [(6, 2), (16, 4)], [(20, 4)]]


@pytest.mark.parametrize("kwargs,exc", [
    (dict(regions=(), elem_size=1, strides=()), ValueError),
    (dict(regions=(((0, 1),),), elem_size=0, strides=(1,)), ValueError),
])
def test_region_constructor_rejects(kwargs, exc):
    with pytest.raises(exc):
        BufferRegion(**kwargs)


def test_region_slice_forms():
    a = BufferRegion.from_slices(elem_size=1, strides=(1,), slices=[slice(None, 4)])
    assert a.describe() == "[0:4]"
    with pytest.raises(ValueError):
        BufferRegion.from_slices(elem_size=1, strides=(1,), slices=[slice(0, 4, 2)])
    with pytest.raises(ValueError):
        BufferRegion.from_slices(elem_size=1, strides=(1,), slices=[slice(0, None)])
    with pytest.raises(ValueError):
        BufferRegion.from_slices(elem_size=1, strides=(1,), slices=[(3, 1)])


# ---------------------------------------------------------------- transfers (reference :266-291)

def test_scattered_push_has_no_flat_view_and_splits_by_bytes():
    push = Transfer(op=TransferOp.PUSH, src_buf="src", src_region=BufferRegion.from_segments([(0, 8), (16, 8)]),
                    peer=1, dst_buf="dst", dst_region=BufferRegion.strided(32, 8, 16, 2), chunk_idx=42)
    assert push.nbytes is None and push.src_off is None and push.dst_off is None
    assert push.to_memcpys() == [(0, 32, 8), (16, 48, 8)]
    parts = push.split(2)
    assert [(p.src_off, p.dst_off, p.nbytes, p.chunk_idx) for p in parts] == [(0, 32, 8, 84), (16, 48, 8, 85)]


def test_memcpys_zip_and_fuse():
    # same bytes, different cuts on both sides
    t = Transfer(op=TransferOp.LOCAL_COPY, src_buf="a", src_region=BufferRegion.from_segments([(0, 6), (10, 2)]),
                 dst_buf="b", dst_region=BufferRegion.from_segments([(100, 4), (200, 4)]), chunk_idx=0)
    assert t.to_memcpys() == [(0, 100, 4), (4, 200, 2), (10, 202, 2)]
    # adjacent on both sides fuses back into one copy
    u = Transfer(op=TransferOp.LOCAL_COPY, src_buf="a", src_region=BufferRegion.from_segments([(0, 4), (8, 4)]),
                 dst_buf="b", dst_region=BufferRegion.from_segments([(64, 4), (72, 4)]), chunk_idx=0)
    assert u.to_memcpys() == [(0, 64, 4), (8, 72, 4)]
    bad = Transfer(op=TransferOp.LOCAL_COPY, src_buf="a", src_region=BufferRegion.contiguous(0, 8),
                   dst_buf="b", dst_region=BufferRegion.contiguous(0, 4), chunk_idx=0)
    with pytest.raises(ValueError):
        bad.to_memcpys()
    with pytest.raises(ValueError):
        _ = bad.nbytes


def test_transfer_peer_contract():
    region = BufferRegion.contiguous(0, 4)
    with pytest.raises(AssertionError):
        Transfer(op=TransferOp.PUSH, src_buf="a", src_region=region, dst_buf="b", dst_region=region, chunk_idx=0)
    with pytest.raises(AssertionError):
        Transfer(op=TransferOp.LOCAL_COPY, src_buf="a", src_region=region, dst_buf="b", dst_region=region,
                 chunk_idx=0, peer=1)


# ---------------------------------------------------------------- builders

def test_all_gather_push_plan():        # reference :31-50
    plan = _gather(2, "push")
    assert len(plan.xfers) == 3 and not plan.local_copies
    assert [x.peer for x in plan.xfers] == [3, 0, 1]
    to0 = {x.peer: x for x in plan.xfers}[0]
    assert (to0.src_off, to0.dst_off, to0.nbytes) == (32, 32, 16)
    assert all(x.chunk_idx == 2 for x in plan.xfers)


def test_all_gather_pull_plan():        # reference :53-64
    plan = _gather(2, "pull")
    assert [x.op for x in plan.xfers] == [TransferOp.PULL] * 3
    assert [(x.peer, x.chunk_idx, x.src_off) for x in plan.xfers] == [(3, 3, 48), (0, 0, 0), (1, 1, 16)]
    assert plan.local_regions["buf"][0].describe() == "[8:12, 0:2]"
    assert plan.tensors_involved["buf"] == (torch.Size((16, 2)), F16)


def test_all_gather_argument_errors():
    with pytest.raises(ValueError):
        _gather(0, "pull", shape=(10, 2))
    with pytest.raises(ValueError):
        _gather(0, "sideways")
    with pytest.raises(IndexError):
        build_all_gather_plan_1d_swizzle((4, 4), F16, 2, 4, 0)
    with pytest.raises(ValueError):
        build_all_gather_plan_1d_swizzle((4, 4), F16, 0, 0, 0)
    # negative axes count from the end
    plan = build_all_gather_plan_1d_swizzle((2, 8), F16, -1, 4, 1, "b", "pull")
    assert plan.local_regions["b"][0].describe() == "[0:2, 2:4]"


def test_all_to_all_push_plan():        # reference :67-90
    plan = build_all_to_all_plan(shape=(4, 4), dtype=F32, mesh_size=4, rank=1, src_buffer="src",
                                 dst_buffer="dst", transfer_kind="push")
    assert plan.dst_shape == (4, 1, 4) and plan.src_shape == (4, 4)
    assert {p.peer: (p.src_off, p.dst_off, p.nbytes) for p in plan.xfers} == {
        0: (0, 16, 16), 2: (32, 16, 16), 3: (48, 16, 16)}
    (copy,) = plan.local_copies
    assert (copy.src_buf, copy.dst_buf, copy.src_off, copy.dst_off, copy.nbytes) == ("src", "dst", 16, 16, 16)
    # communication produces the data: the local copy is issued first
    assert plan.xfer[0][0] is copy
    assert [p.chunk_idx for p in plan.xfers] == [1 * 4 + 2, 1 * 4 + 3, 1 * 4 + 0]


def test_all_to_all_compute_producer_orders_local_copy_last():
    plan = build_all_to_all_plan(shape=(8, 2), dtype=F16, mesh_size=4, rank=3, src_buffer="src",
                                 dst_buffer="dst", transfer_kind="push", compute_producer=True)
    ops = plan.xfer[0]
    assert [op.op for op in ops] == [TransferOp.PUSH] * 3 + [TransferOp.LOCAL_COPY]
    assert [op.peer for op in ops] == [0, 1, 2, None]
    for op in ops:
        (dep,) = op.dependency
        assert dep.compute_rank == 3 and dep.signal is None
        assert dep.src_region == op.src_region


def test_all_to_all_dim_push():         # reference :93-121
    plan = build_all_to_all_plan_dim(shape=(2, 2, 12, 3), dtype=F32, mesh_size=4, rank=1, src_buffer="src",
                                     dst_buffer="dst", src_split_axis=1, dst_split_axis=2, transfer_kind="push")
    assert plan.dst_shape == (2, 8, 3, 3)
    assert {x.peer: x.src_region.describe() for x in plan.xfers} == {
        0: "[0:2, 0:2, 0:3, 0:3]", 2: "[0:2, 0:2, 6:9, 0:3]", 3: "[0:2, 0:2, 9:12, 0:3]"}
    assert plan.local_copies[0].dst_region.describe() == "[0:2, 2:4, 0:3, 0:3]"


def test_all_to_all_dim_pull():         # reference :166-189
    plan = build_all_to_all_plan_dim(shape=(2, 8, 3, 3), dtype=F16, mesh_size=4, rank=2, src_buffer="src",
                                     dst_buffer="dst", src_split_axis=2, dst_split_axis=1, transfer_kind="pull")
    assert plan.dst_shape == (2, 2, 12, 3)
    assert all(x.op == TransferOp.PULL for x in plan.xfers)
    assert {x.peer: x.dst_region.describe() for x in plan.xfers} == {
        0: "[0:2, 0:2, 0:3, 0:3]", 1: "[0:2, 0:2, 3:6, 0:3]", 3: "[0:2, 0:2, 9:12, 0:3]"}


def test_all_to_all_dim_peer_order_and_errors():
    kw = dict(shape=(2, 8), dtype=F16, mesh_size=4, rank=1, src_buffer="s", dst_buffer="d",
              src_split_axis=0, dst_split_axis=1)
    assert [x.peer for x in build_all_to_all_plan_dim(**kw).xfers] == [2, 3, 0]
    assert [x.peer for x in build_all_to_all_plan_dim(**kw, peer_order="counter-clockwise").xfers] == [0, 3, 2]
    with pytest.raises(ValueError):
        build_all_to_all_plan_dim(**kw, peer_order="zigzag")
    with pytest.raises(ValueError):
        build_all_to_all_plan_dim(**{**kw, "dst_split_axis": 0})
    with pytest.raises(ValueError):
        build_all_to_all_plan_dim(**{**kw, "shape": (2, 6)})


def test_ring_all_gather_dependencies():    # reference :124-163
    plans = {r: build_ring_all_gather_plan((16, 2), F16, 0, 4, r, "buf") for r in range(4)}
    cp = CommPlan(plans)
    cp.plan_signals()
    pushes = plans[2].xfers
    assert [(p.op, p.peer, p.chunk_idx) for p in pushes] == [(TransferOp.PUSH, 3, c) for c in (2, 1, 0)]
    assert not pushes[0].dependency
    for step in (1, 2):
        (dep,) = pushes[step].dependency
        assert (dep.depend_rank, dep.depend_xfer_stream, dep.depend_xfer_idx) == (1, 0, step - 1)
        assert dep.signal is plans[1].xfers[step - 1].set_signals[0]
    assert all(not p.transit_signals for p in plans.values())
    assert build_ring_all_gather_plan((4, 2), F16, 0, 1, 0, "b").xfer == [[]]


def test_double_ring_op_layout():
    """W=8, inner=2: per outer step one inner push and (except last) one outer push."""
    plans = {r: build_double_ring_all_gather_plan((8, 2), F16, 0, 8, 2, r, "b") for r in range(8)}
    ops = plans[5].xfer[0]          # rank 5 = group 2, inner 1
    assert len(ops) == 4 * 2 - 1
    assert [op.peer for op in ops] == [4, 7, 4, 7, 4, 7, 4]
    rows = [op.src_region.regions[0][0].start for op in ops]
    # shards forwarded, by owner rank: own, 4 (from inner), then groups 1, 0, 3 arriving over the outer ring
    assert rows == [5, 4, 2, 3, 1, 0, 6]
    deps = [[(d.depend_rank, d.depend_xfer_idx) for d in op.dependency] for op in ops]
    assert deps == [[], [(4, 0)], [(3, 1)], [(4, 2)], [(3, 3)], [(4, 4)], [(3, 5)]]
    with pytest.raises(ValueError):
        build_double_ring_all_gather_plan((8, 2), F16, 0, 8, 3, 0, "b")


def test_reduce_scatter_direct_reduce_plan():
    plan = build_reduce_scatter_direct_reduce_plan((8, 8), dtype=F32, axis=0, mesh_size=4, rank=1,
                                                   src_buffer="src", dst_buffer="dst")
    ops = plan.xfer[0]
    assert [op.op for op in ops] == [TransferOp.PUSH] * 3 + [TransferOp.LOCAL_COPY]
    assert [op.peer for op in ops] == [2, 3, 0, None]
    assert [op.src_region.describe() for op in ops] == ["[4:6, 0:8]", "[6:8, 0:8]", "[0:2, 0:8]", "[2:4, 0:8]"]
    assert all(op.dst_region.describe() == "[0:2, 0:8]" and op.reduce_op == ReduceOp.SUM for op in ops)
    assert [op.chunk_idx for op in ops] == [0, 1, 2, 3]
    assert plan.local_regions["src"][0].describe() == "[0:8, 0:8]"
    assert plan.tensors_involved["dst"][0] == torch.Size((2, 8))
    with pytest.raises(ValueError):
        build_reduce_scatter_direct_reduce_plan((8, 8), dtype=F32, axis=0, mesh_size=4, rank=4,
                                                src_buffer="s", dst_buffer="d")


# ---------------------------------------------------------------- device plan (reference :249-262, :336-357)

def test_device_plan_text_and_streams():
    text = _gather(1, "push").pretty()
    assert text.splitlines()[:3] == ["DevicePlan(dev=1)", "  Stream 0:",
                                     "    [0] push peer=2 buf[4:8, 0:2] -> buf[4:8, 0:2]"]
    plan = DevicePlan(dev=0)
    assert plan.add_stream() == 1
    region = BufferRegion.contiguous(0, 4)
    plan.add_op(Transfer(op=TransferOp.LOCAL_COPY, src_buf="a", src_region=region, dst_buf="b",
                         dst_region=region, chunk_idx=-1), stream_idx=1)
    assert plan.xfer[0] == [] and len(plan.xfer[1]) == 1
    assert "    (none)" in plan.pretty() and "[0] copy a[0:4] -> b[0:4]" in plan.pretty()
    with pytest.raises(ValueError):
        plan.add_op(plan.xfer[1][0], stream_idx=-1)
    split = _gather(0, "pull", shape=(16, 4)).split_xfers(2)
    assert [x.chunk_idx for x in split.xfers] == [2, 3, 4, 5, 6, 7]
    assert [x.nbytes for x in split.xfers] == [16] * 6


def test_all_to_all_dim_waves_splits_destination_axis():
    """Literal vectors of the reference's tests/test_descriptor.py:192-221."""
    import torch

    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan_dim_waves

    mesh_size, num_waves = 2, 3
    plan = build_all_to_all_plan_dim_waves(shape=(6, 2), dtype=torch.float32, mesh_size=mesh_size, rank=0,
                                           src_buffer="src", dst_buffer="dst", src_split_axis=1,
                                           dst_split_axis=0, num_waves=num_waves, transfer_kind="push")
    assert plan.dst_shape == (3, 4)
    assert len(plan.xfers) == (mesh_size - 1) * num_waves
    assert len(plan.local_copies) == num_waves
    assert [xf.src_region.describe() for xf in plan.xfers] == ["[3:4, 0:2]", "[4:5, 0:2]", "[5:6, 0:2]"]
    assert [xf.dst_region.describe() for xf in plan.xfers] == ["[0:1, 0:2]", "[1:2, 0:2]", "[2:3, 0:2]"]
    assert [c.dst_region.describe() for c in plan.local_copies] == ["[0:1, 0:2]", "[1:2, 0:2]", "[2:3, 0:2]"]
    assert sorted([xf.chunk_idx for xf in plan.xfers] + [c.chunk_idx for c in plan.local_copies]) == [0, 1, 2, 3, 4, 5]
    with pytest.raises(ValueError):
        build_all_to_all_plan_dim_waves(shape=(6, 2), dtype=torch.float32, mesh_size=2, rank=0, src_buffer="s",
                                        dst_buffer="d", src_split_axis=1, dst_split_axis=0, num_waves=2)
