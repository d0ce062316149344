"""Lowering, tile-schedule model, op-list generation and wave-table glue.

Vectors: the reference's tests/test_lowering.py, tests/test_tile_schedule.py,
tests/test_allgather_schedule.py, tests/test_*_codegen.py (cited per test) and the committed
fixture tests/golden/host_compiler.json (outputs of the reference's host modules for 15 plans,
written by tests/golden/make_host_fixtures.py)."""

import importlib.util
import json
import os

import pytest
import torch

from syncopate_amd.communication.code_gen import CodeGenOptions, CommGenerator
from syncopate_amd.communication.comm_runtime.operations import (
    CopyEngineOp,
    IntraNodeSignal,
    SMCopyOp,
    WaitIntraNodeSignal,
)
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
    ReduceOp,
    Signal,
    SignalType,
    Transfer,
    TransferOp,
)
from syncopate_amd.interface import lower_comm_plan_to_raw_schedules, tile_schedule
from syncopate_amd.interface.wave_tables import (
    all2all_attn_tables,
    allgather_attn_tables,
    gemm_consumer_tables,
    gemm_producer_tables,
    plan_layout_spec,
)

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
F16 = torch.float16

TileCoord, TileBlock, RawSchedule = tile_schedule.TileCoord, tile_schedule.TileBlock, tile_schedule.RawSchedule
SimplifiedSchedule, Mod1DSchedule = tile_schedule.SimplifiedSchedule, tile_schedule.Mod1DSchedule


def _single_rank_gather(rank, kind):
    plan = build_all_gather_plan_1d_swizzle((16, 2), F16, 0, 4, rank, "buf", kind)
    plan.tensors_involved["buf"] = ((16, 2), None)
    return plan


# ---------------------------------------------------------------- lowering (reference test_lowering.py)

def test_pull_gather_lowers_to_swizzled_row_blocks():        # :15-38, :169-193, :232-256
    cp = CommPlan({2: _single_rank_gather(2, "pull")})
    cp.plan_signals()
    sched = lower_comm_plan_to_raw_schedules(cp)[2]["buf"]
    assert (sched.num_waves, sched.global_shape) == (4, (16, 2))
    assert [[b.tile.offsets for b in w] for w in sched.block_infos] == [[(8, 0)], [(12, 0)], [(0, 0)], [(4, 0)]]
    assert all(b.tile.shape == (4, 2) for w in sched.block_infos for b in w)
    assert sched.block_infos[0][0].signal is None
    for wave in sched.block_infos[1:]:
        assert (wave[0].signal.type, wave[0].signal.dst_rank) == (SignalType.RECEIVE_DATA, 2)
    assert sched.gen_signal_lists() == [-1, 0, 1, 2]
    assert sched.gen_target_rank_list() == [2, 3, 0, 1]
    assert sched.role() == "consumer" and sched.is_reduce() is False
    simple = SimplifiedSchedule(origin_schedule=sched)
    assert simple.simplify() is True      # a swizzled gather is the Mod1D pattern, starting at the own shard
    m = simple.simplified_schedule
    assert (m.schedule_axis, m.stride, m.starting_offset) == (0, 4, 8)


def test_push_gather_only_shows_the_resident_shard():       # :41-59
    sched = lower_comm_plan_to_raw_schedules(CommPlan({1: _single_rank_gather(1, "push")}))[1]["buf"]
    assert sched.num_waves == 1 and sched.global_shape == (16, 2)
    assert sched.block_infos[0][0].tile.offsets == (4, 0)


def test_repeated_reads_keep_the_earliest_touch():          # :62-99
    region = BufferRegion.from_slices(elem_size=1, strides=row_major_strides((4,)), slices=[(0, 4)])
    plan = DevicePlan(dev=0)
    for peer in (1, 2):
        plan.add_op(Transfer(op=TransferOp.PUSH, src_buf="buf", src_region=region, dst_buf="remote",
                             dst_region=region, peer=peer, chunk_idx=peer - 1))
    plan.tensors_involved["buf"] = ((4,), torch.int8)
    sched = lower_comm_plan_to_raw_schedules(CommPlan({0: plan}))[0]["buf"]
    assert sched.num_waves == 1 and len(sched.block_infos[0]) == 1
    assert sched.block_infos[0][0].tile.offsets == (0,)
    assert sched.block_infos[0][0].peer_rank == 1


def test_parallel_streams_share_a_wave():                   # :129-166
    strides = row_major_strides((4, 4))
    top = BufferRegion.from_slices(elem_size=1, strides=strides, slices=[(0, 2), (0, 4)])
    bottom = BufferRegion.from_slices(elem_size=1, strides=strides, slices=[(2, 4), (0, 4)])
    plan = DevicePlan(dev=0)
    plan.add_op(Transfer(op=TransferOp.PULL, src_buf="remote_a", src_region=top, dst_buf="buf", dst_region=top,
                         peer=1, chunk_idx=0), stream_idx=0)
    plan.add_op(Transfer(op=TransferOp.PULL, src_buf="remote_b", src_region=bottom, dst_buf="buf",
                         dst_region=bottom, peer=2, chunk_idx=1), stream_idx=1)
    plan.tensors_involved["buf"] = ((4, 4), None)
    sched = lower_comm_plan_to_raw_schedules(CommPlan({0: plan}))[0]["buf"]
    assert sched.num_waves == 1 and sched.global_shape == (4, 4)
    assert [b.tile.offsets for b in sched.block_infos[0]] == [(0, 0), (2, 0)]


def _a2a_producer(world, shape):
    plans = {r: build_all_to_all_plan(shape=shape, dtype=F16, mesh_size=world, rank=r, src_buffer="src",
                                      dst_buffer="dst", transfer_kind="push", compute_producer=True)
             for r in range(world)}
    cp = CommPlan(plans)
    cp.plan_signals()
    return cp, lower_comm_plan_to_raw_schedules(cp)


def test_compute_producer_schedule_carries_compute_flags_and_peers():   # :102-126, :259-285
    _, lowered = _a2a_producer(4, (64, 32))
    src = lowered[0]["src"]
    flags = [b.signal for w in src.block_infos for b in w]
    assert all(f is not None and f.type == SignalType.COMPUTE_DONE for f in flags)
    assert src.gen_signal_lists() == [0, 1, 2, 3]
    assert src.gen_target_rank_list() == [1, 2, 3, -1]
    assert src.gen_block_offset_lists() == [[16, 0], [32, 0], [48, 0], [0, 0]]
    assert src.role() == "producer" and src.is_reduce() is False
    dst = lowered[0]["dst"]
    assert dst.role() == "consumer"
    assert dst.gen_block_offset_lists() == [[3, 0, 0], [2, 0, 0], [1, 0, 0], [0, 0, 0]]
    assert dst.gen_target_rank_list() == [3, 2, 1, -1]


def test_peer_side_offsets():                                            # :288-344
    plans = {r: build_reduce_scatter_direct_reduce_plan((64, 32), dtype=F16, axis=0, mesh_size=4, rank=r,
                                                        src_buffer="src", dst_buffer="dst") for r in range(4)}
    cp = CommPlan(plans)
    cp.plan_signals()
    sched = lower_comm_plan_to_raw_schedules(cp)[0]["src"]
    assert sched.gen_block_offset_lists() == [[16, 0], [32, 0], [48, 0], [0, 0]]
    assert sched.gen_dst_offset_lists() == [[0, 0]] * 4
    assert sched.is_reduce() is True
    ag = {r: build_all_gather_plan_1d_swizzle((64, 32), F16, 0, 4, r, "a", "pull") for r in range(4)}
    cp = CommPlan(ag)
    cp.plan_signals()
    sched = lower_comm_plan_to_raw_schedules(cp)[0]["a"]
    assert sched.gen_dst_offset_lists() == sched.gen_block_offset_lists()


def test_reduce_op_reaches_both_sides():                                 # :347-384
    region = BufferRegion.from_slices(elem_size=1, strides=(1,), slices=[(0, 4)])
    origin, peer = DevicePlan(dev=0), DevicePlan(dev=1)
    origin.add_op(Transfer(op=TransferOp.PUSH, src_buf="src", src_region=region, dst_buf="dst",
                           dst_region=region, peer=1, chunk_idx=0, reduce_op=ReduceOp.SUM))
    origin.tensors_involved["src"] = ((4,), None)
    peer.tensors_involved["dst"] = ((4,), None)
    cp = CommPlan({0: origin, 1: peer})
    cp.plan_signals()
    lowered = lower_comm_plan_to_raw_schedules(cp)
    src, dst = lowered[0]["src"], lowered[1]["dst"]
    assert (src.is_reduce(), src.role(), src.gen_target_rank_list()) == (True, "producer", [1])
    assert (dst.is_reduce(), dst.role(), dst.gen_target_rank_list()) == (True, "consumer", [0])
    assert dst.gen_signal_lists() == [0] and src.gen_signal_lists() == [-1]


def test_kv_gather_along_sequence_axis():                                # test_allgather_schedule.py:32-37
    plans = {r: build_all_gather_plan_1d_swizzle((2, 1, 1, 4, 1), F16, 3, 4, r, "kv", "pull") for r in range(4)}
    gen = CommGenerator(plans)
    gen.plan_signals()
    sched = lower_comm_plan_to_raw_schedules(gen)[0]["kv"]
    assert sched.gen_block_offset_lists() == [[0, 0, 0, k, 0] for k in range(4)]


def test_shape_hint_violation_is_reported():
    plan = _single_rank_gather(2, "pull")
    plan.tensors_involved["buf"] = ((8, 2), None)
    with pytest.raises(ValueError, match="exceeds expected shape"):
        lower_comm_plan_to_raw_schedules(CommPlan({2: plan}))


# ---------------------------------------------------------------- golden fixture

def _fixture_module():
    spec = importlib.util.spec_from_file_location("make_host_fixtures",
                                                  os.path.join(GOLDEN, "make_host_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


with open(os.path.join(GOLDEN, "host_compiler.json")) as _f:
    _EXPECTED = json.load(_f)


@pytest.mark.parametrize("case", sorted(_EXPECTED))
def test_matches_reference_outputs(case):
    """Every flattened schedule, signal table, period start, rendered text and op dump equals
    what the reference's host modules produced for the same plan."""
    mod = _fixture_module()
    got = json.loads(json.dumps(mod.run_case(mod.load_api(True), case), sort_keys=True))
    want = _EXPECTED[case]
    assert got.keys() == want.keys()
    for key in want:
        assert got[key] == want[key], f"{case}: {key} differs"


def test_baseline_closed_forms():
    """The tables the benchmarked configurations lower to (W=8), as closed forms."""
    c2 = _EXPECTED["ag_swizzle_pull_c2"]["schedules"]
    for r in range(8):
        s = c2[str(r)]["a"]
        assert s["offsets"] == [[((r + k) % 8) * 1024, 0] for k in range(8)]
        assert s["signals"] == [-1, 0, 1, 2, 3, 4, 5, 6]
        assert s["target_ranks"] == [(r + k) % 8 for k in range(8)]
    c5 = _EXPECTED["ag_double_ring_c5"]["schedules"]["0"]["kv"]
    assert [o[3] // 4096 for o in c5["offsets"]] == [0, 1, 7, 6, 4, 5, 3, 2]
    assert c5["signals"] == [-1, 0, 4, 1, 5, 2, 6, 3]
    c3 = _EXPECTED["a2a_push_producer_c3"]["schedules"]
    for r in range(8):
        s = c3[str(r)]["src"]
        assert [o[0] // 1024 for o in s["offsets"]] == [(r + k + 1) % 8 for k in range(8)]
        assert s["signals"] == list(range(8))
    c4 = _EXPECTED["a2a_dim_pull_c4"]["schedules"]["0"]["dst"]
    assert c4["signals"] == list(range(8)) and c4["target_ranks"] == [-1, 1, 2, 3, 4, 5, 6, 7]


# ---------------------------------------------------------------- tile schedule (reference test_tile_schedule.py)

def _two_wave():
    flag = Signal(type=SignalType.RECEIVE_DATA, dst_rank=0, dst_offset=0)
    return RawSchedule(num_waves=2, global_shape=(2, 8), block_infos=[
        [TileBlock(tile=TileCoord(offsets=(0, 0), shape=(2, 4)), signal=None)],
        [TileBlock(tile=TileCoord(offsets=(0, 4), shape=(2, 4)), signal=flag)]])


@pytest.mark.parametrize("offsets,shape,message", [
    ((0,), (), "identical length"),
    ((0, -1), (2, 2), "offsets must be non-negative"),
    ((0, 1), (2, 0), "shape must contain strictly positive sizes"),
])
def test_tile_coord_rejects(offsets, shape, message):       # :22-33
    with pytest.raises(ValueError, match=message):
        TileCoord(offsets=offsets, shape=shape)


def test_tile_coord_views():                                # :36-39
    tile = TileCoord(offsets=(1, 3), shape=(2, 5))
    assert tile.ndim == 2 and tile.as_ranges() == ((1, 3), (3, 8))
    assert repr(tile) == "TileCoord(offsets=(1, 3), shape=(2, 5))"


@pytest.mark.parametrize("kwargs,message", [            # :48-68
    (dict(num_waves=0, block_infos=[], global_shape=(2, 2)), "num_waves must be positive"),
    (dict(num_waves=1, block_infos=[], global_shape=(2, 2)), "block_infos length must match num_waves"),
    (dict(num_waves=1, block_infos=[[]], global_shape=(2, 2)), "each wave must contain at least one block"),
    (dict(num_waves=1, block_infos=[[TileBlock(tile=TileCoord(offsets=(0,), shape=(4,)))]], global_shape=(4, 4)),
     "all blocks must have the same number of dimensions as global_shape"),
])
def test_raw_schedule_rejects(kwargs, message):
    with pytest.raises(ValueError, match=message):
        RawSchedule(**kwargs)


def test_mod1d_and_simplify():                              # :71-116
    raw = _two_wave()
    m = Mod1DSchedule(raw)
    assert (m.schedule_axis, m.stride, m.starting_offset, m.global_shape, m.num_waves) == (1, 4, 0, (2, 8), 2)
    s = SimplifiedSchedule(origin_schedule=raw)
    assert s.simplify() is True and isinstance(s.simplified_schedule, Mod1DSchedule)
    block = TileBlock(tile=TileCoord(offsets=(0, 0), shape=(2, 4)))
    with pytest.raises(ValueError, match="all waves must contain exactly one block"):
        Mod1DSchedule(RawSchedule(num_waves=2, block_infos=[[block, block], [block]], global_shape=(2, 4)))
    uneven = RawSchedule(num_waves=2, global_shape=(2, 12), block_infos=[
        [TileBlock(tile=TileCoord(offsets=(0, 0), shape=(2, 4)))],
        [TileBlock(tile=TileCoord(offsets=(0, 4), shape=(2, 8)))]])
    with pytest.raises(ValueError, match="all blocks must have the same shape"):
        Mod1DSchedule(uneven)
    whole = RawSchedule(num_waves=1, global_shape=(2, 8),
                        block_infos=[[TileBlock(tile=TileCoord(offsets=(0, 0), shape=(2, 8)))]])
    with pytest.raises(ValueError, match="schedule must be defined along exactly one axis"):
        Mod1DSchedule(whole)
    hopeless = SimplifiedSchedule(origin_schedule=RawSchedule(num_waves=1, block_infos=[[block, block]],
                                                              global_shape=(2, 4)))
    assert hopeless.simplify() is False and hopeless.simplified_schedule is None


def test_schedule_roles_must_agree():
    a = TileBlock(tile=TileCoord(offsets=(0,), shape=(1,)), role="producer")
    b = TileBlock(tile=TileCoord(offsets=(1,), shape=(1,)), role="consumer")
    with pytest.raises(ValueError, match="disagree on role"):
        RawSchedule(num_waves=1, block_infos=[[a, b]], global_shape=(2,)).role()


# ---------------------------------------------------------------- op lists (reference test_*_codegen.py)

def test_swizzle_gather_op_list():          # test_codegen_all_gather.py:13-43
    gen = CommGenerator({r: build_all_gather_plan_1d_swizzle((100, 20), F16, 0, 4, r, "buf", "pull")
                         for r in range(4)})
    gen.plan_signals()
    info = gen.generate_code_for_plan()
    assert (info.world_size, info.recv_signal_num, info.transit_signal_num, info.compute_signal_num) == (4, 3, 0, 0)
    assert len(info.operations) == 4
    ops = info.operations[1][0]
    assert [type(o) for o in ops] == [CopyEngineOp, IntraNodeSignal] * 3
    assert [(o.src_rank, o.dst_rank, o.src_offset, o.dst_offset, o.size) for o in ops[::2]] == [
        (2, 1, 2000, 2000, 1000), (3, 1, 3000, 3000, 1000), (0, 1, 0, 0, 1000)]
    assert [(o.offset, o.rank) for o in ops[1::2]] == [(0, 1), (1, 1), (2, 1)]
    assert info.comm_buffer_sizes == {"buf": (torch.Size((100, 20)), F16)}
    sm = CommGenerator({r: build_all_gather_plan_1d_swizzle((100, 20), F16, 0, 4, r, "buf", "pull")
                        for r in range(4)})
    sm.plan_signals()
    box_ops = sm.generate_code_for_plan(options=CodeGenOptions(copy_engine=False)).operations[0][0]
    assert isinstance(box_ops[0], SMCopyOp) and box_ops[0].use_tma is True
    assert [(ax.start, ax.end) for ax in box_ops[0].src_slice] == [(25, 50), (0, 20)]


def test_ring_gather_op_list():             # test_ring_allgather_codegen.py:40-63
    gen = CommGenerator({r: build_ring_all_gather_plan((8, 2), F16, 0, 4, r, "buf") for r in range(4)})
    gen.plan_signals()
    info = gen.generate_code_for_plan()
    for r in range(4):
        ops = info.operations[r][0]
        assert [type(o) for o in ops] == [CopyEngineOp, IntraNodeSignal] + \
            [WaitIntraNodeSignal, CopyEngineOp, IntraNodeSignal] * 2
        assert all(o.signal_type == SignalType.RECEIVE_DATA for o in ops if isinstance(o, WaitIntraNodeSignal))
        # a rank waits on its own flag words (set by its upstream neighbour) and signals downstream
        assert [(o.rank, o.offset) for o in ops if isinstance(o, WaitIntraNodeSignal)] == [(r, 0), (r, 1)]
        assert [(o.rank, o.offset) for o in ops if isinstance(o, IntraNodeSignal)] == [((r + 1) % 4, k) for k in range(3)]


def test_double_ring_op_list_counts():      # test_double_ring_allgather_codegen.py:44-63
    gen = CommGenerator({r: build_double_ring_all_gather_plan((18, 2), F16, 0, 9, 3, r, "buf") for r in range(9)})
    gen.plan_signals()
    info = gen.generate_code_for_plan()
    for r in range(9):
        ops = info.operations[r][0]
        kinds = [type(o) for o in ops]
        assert kinds.count(CopyEngineOp) == kinds.count(IntraNodeSignal) == 8
        assert kinds.count(WaitIntraNodeSignal) == 7
        for i, o in enumerate(ops):
            if isinstance(o, WaitIntraNodeSignal):
                assert isinstance(ops[i + 1], CopyEngineOp)


def test_compute_waits_precede_copies_and_options_are_validated():
    gen = CommGenerator({r: build_all_to_all_plan(shape=(8, 4), dtype=F16, mesh_size=2, rank=r, src_buffer="src",
                                                  dst_buffer="dst", transfer_kind="push", compute_producer=True)
                         for r in range(2)})
    gen.plan_signals()
    info = gen.generate_code_for_plan()
    assert info.compute_signal_num == 2 and info.recv_signal_num == 2
    ops = info.operations[0][0]
    assert [type(o) for o in ops] == [WaitIntraNodeSignal, CopyEngineOp, IntraNodeSignal] * 2
    assert [o.signal_type for o in ops[::3]] == [SignalType.COMPUTE_DONE] * 2
    assert (ops[1].src_rank, ops[1].dst_rank, ops[4].src_rank, ops[4].dst_rank) == (0, 1, 0, 0)
    text = str(info)
    assert "WaitIntraNodeSignal(type=SignalType.COMPUTE_DONE, offset=0, rank=0)" in text
    assert "CopyEngineOp(src_rank=0, dst_rank=1, src_offset=32, dst_offset=0, size=32)" in text
    with pytest.raises(NotImplementedError):
        CodeGenOptions(low_latency=True).validate()
    with pytest.raises(ValueError):
        CodeGenOptions(copy_engine=True, fuse_with_compute_intra=True).validate()
    with pytest.raises(ValueError):
        CodeGenOptions(copy_engine=False, fuse_with_compute_inter=True).validate()
    rs = CommGenerator({r: build_reduce_scatter_direct_reduce_plan((8, 8), dtype=torch.float32, axis=0,
                                                                   mesh_size=4, rank=r, src_buffer="src",
                                                                   dst_buffer="dst") for r in range(4)})
    rs.plan_signals()
    with pytest.raises(ValueError, match="cannot do reduction"):
        rs.generate_code_for_plan()            # reducing transfers need the box-copy path
    boxes = rs.generate_code_for_plan(CodeGenOptions(copy_engine=False)).operations[0][0]
    assert all(o.reduce_op == ReduceOp.SUM for o in boxes if isinstance(o, SMCopyOp))


# ---------------------------------------------------------------- wave-table glue (hand-evaluated)

def test_gemm_tables_from_schedules():
    gen = CommGenerator({r: build_all_gather_plan_1d_swizzle((512, 64), F16, 0, 4, r, "a", "pull") for r in range(4)})
    gen.plan_signals()
    t = gemm_consumer_tables(lower_comm_plan_to_raw_schedules(gen)[1]["a"], n_per_rank=256)
    # reference glue: offsets[i][1] = 0, shapes[i][1] = N_per_rank, cum = sum rows*N (test_ag_gemm_gen.py:137-150)
    assert t.block_offsets == [[128, 0], [256, 0], [384, 0], [0, 0]]
    assert t.block_shapes == [[128, 256]] * 4
    assert t.signal_offsets == [-1, 0, 1, 2] and t.cum_tiles == 512 * 256
    _, lowered = _a2a_producer(4, (512, 256))
    p = gemm_producer_tables(lowered[3]["src"])
    assert p.block_offsets == [[0, 0], [128, 0], [256, 0], [384, 0]]
    assert p.block_shapes == [[128, 256]] * 4 and p.signal_offsets == [0, 1, 2, 3] and p.cum_tiles == 512 * 256


def test_allgather_attention_tables():
    """W=2, B=1, H=3, local Sq=256, chunk 256: by hand from tests/test_allgather_attn_transform.py:63-84."""
    shape, seq_axis, axes = plan_layout_spec("bhsd", 1, 3, 512, 128)
    assert (shape, seq_axis) == ((2, 1, 3, 512, 128), 3)
    gen = CommGenerator({r: build_all_gather_plan_1d_swizzle(shape, torch.bfloat16, seq_axis, 2, r, "kv", "pull")
                         for r in range(2)})
    gen.plan_signals()
    t = allgather_attn_tables(lower_comm_plan_to_raw_schedules(gen)[1]["kv"], 256, axes)
    assert t.wave_offsets == [[0, 0, 0, 256], [0, 0, 0, 0]]
    assert t.wave_sizes == [[1, 3, 256, 256], [1, 3, 256, 256]]
    assert t.signal_offsets == [-1, 0]
    assert t.cum_wave_sizes == [768, 1536] and t.cum_tiles == 1536
    assert plan_layout_spec("bshd", 2, 4, 8, 16) == ((2, 2, 8, 4, 16), 2, {"batch": 1, "head": 3, "seq": 2})
    with pytest.raises(ValueError):
        plan_layout_spec("sbhd", 1, 1, 1, 1)


def test_all2all_attention_tables():
    """W=3, stacked QKV (3, B=1, H/w=2, S=384, D): arrival wave w unlocks (Q_w, KV_w) and both cross terms
    with every earlier chunk; by hand from tests/test_all2all_attn_transform.py:58-117."""
    axes = {"batch": 1, "head": 2, "seq": 3}
    gen = CommGenerator({r: build_all_to_all_plan_dim(shape=(3, 1, 6, 128, 128), dtype=torch.bfloat16, mesh_size=3,
                                                      rank=r, src_buffer="src", dst_buffer="dst", src_split_axis=3,
                                                      dst_split_axis=2, transfer_kind="pull") for r in range(3)})
    gen.plan_signals()
    sched = lower_comm_plan_to_raw_schedules(gen)[1]["dst"]
    assert [o[3] for o in sched.gen_block_offset_lists()] == [128, 256, 0]      # own chunk, then ranks 2, 0
    assert sched.gen_signal_lists() == [0, 1, 2]                                 # the local copy has a flag too
    t = all2all_attn_tables(sched, axes)
    q = {0: 128, 1: 256, 2: 0}
    expect_offsets = [[0, 0, q[0], q[0]],
                      [0, 0, q[1], q[1]], [0, 0, q[0], q[1]], [0, 0, q[1], q[0]],
                      [0, 0, q[2], q[2]], [0, 0, q[0], q[2]], [0, 0, q[2], q[0]],
                      [0, 0, q[1], q[2]], [0, 0, q[2], q[1]]]
    assert t.wave_offsets == expect_offsets
    assert t.wave_sizes == [[1, 2, 128, 128]] * 9
    assert t.signal_offsets == [0, 1, 1, 1, 2, 2, 2, 2, 2]
    assert t.cum_wave_sizes == [256 * (i + 1) for i in range(9)] and t.cum_tiles == 2304


def test_attention_producer_tables_by_hand():
    """Attention that feeds an all-to-all along the sequence axis (bshd, W=2, rank 1): the rank's
    pushes go to rank 0 first, its own chunk last; one wave per outgoing sequence chunk, all of
    K/V per wave, flags = the COMPUTE_DONE offsets 0, 1 in op order
    (reference: tests/test_attn_all2all_transform.py:57-85, 137-163)."""
    import torch

    from syncopate_amd.communication.code_gen import CommGenerator
    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan_axis
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules
    from syncopate_amd.interface.wave_tables import attn_producer_tables

    B, SEQ, Hp, D, world = 3, 512, 2, 128, 2
    plans = {r: build_all_to_all_plan_axis(shape=(B, SEQ, Hp, D), dtype=torch.float16, mesh_size=world, rank=r,
                                           src_buffer="src", dst_buffer="dst", split_axis=1,
                                           transfer_kind="push", compute_producer=True) for r in range(world)}
    gen = CommGenerator(plans)
    gen.plan_signals()
    schedule = lower_comm_plan_to_raw_schedules(gen)[1]["src"]
    t = attn_producer_tables(schedule, {"batch": 0, "head": 2, "seq": 1}, SEQ)
    assert t.wave_offsets == [[0, 0, 0, 0], [0, 0, 256, 0]]
    assert t.wave_sizes == [[3, 2, 256, 512], [3, 2, 256, 512]]
    assert t.signal_offsets == [0, 1]
    assert t.cum_wave_sizes == [3 * 2 * 256, 2 * 3 * 2 * 256]
    assert t.cum_tiles == 3 * 2 * 512


def test_accumulating_box_copies_with_a_single_writer_are_found():
    """Pull form of reduce-scatter by direct reduction: every sum into a rank's result sits in
    that rank's own op list, so none needs atomics; push form: every rank adds into every
    result, all of them do."""
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_reduce_scatter_direct_reduce_plan

    world = 4
    for kind, expect in (("pull", 16), ("push", 0)):
        plans = {r: build_reduce_scatter_direct_reduce_plan(shape=(1024, 512), dtype=torch.float16, axis=0,
                                                            mesh_size=world, rank=r, src_buffer="src",
                                                            dst_buffer="dst", transfer_kind=kind)
                 for r in range(world)}
        gen = CommGenerator(plans)
        gen.plan_signals()
        info = gen.generate_code_for_plan(options=CodeGenOptions(copy_engine=False, use_tma=False))
        ctx = CommContext.__new__(CommContext)        # the analysis needs no device
        ctx.info = info
        sole = ctx._find_sole_writer_ops()
        boxes = [op for lists in info.operations for ops in lists for op in ops if isinstance(op, SMCopyOp)]
        assert len(boxes) == 16 and len(sole) == expect
        # two lists writing overlapping boxes of one destination: neither is a sole writer
        if kind == "pull":
            info.operations[0].append(list(info.operations[0][0]))
            sole = ctx._find_sole_writer_ops()
            assert not any(id(op) in sole for op in info.operations[0][0] if isinstance(op, SMCopyOp))
            assert all(id(op) in sole for op in info.operations[1][0] if isinstance(op, SMCopyOp))


# ---- library-collective plans (reference: tests/test_all_reduce_descriptor.py, tests/test_reduce_scatter_codegen.py)

def _collective_info(builder, mesh, **kwargs):
    gen = CommGenerator({r: builder(mesh_size=mesh, rank=r, **kwargs) for r in range(mesh)})
    gen.plan_signals()
    return gen, gen.generate_code_for_plan()


def test_all_reduce_slabs_become_collective_then_flag():
    from syncopate_amd.communication.comm_runtime.operations import CollectiveComm
    from syncopate_amd.communication.common_descriptors import build_all_reduce_plan
    from syncopate_amd.communication.descriptor import AxisSlice, CollectiveOp

    _, info = _collective_info(build_all_reduce_plan, 2, shape=(4, 4), dtype=torch.float32, buffer_name="buf",
                               num_all_reduces=2, split_axis=1)
    assert info.world_size == 2 and info.recv_signal_num == 2
    for rank in range(2):
        (ops,) = info.operations[rank]
        assert len(ops) == 4
        for idx in range(2):
            coll, flag = ops[2 * idx], ops[2 * idx + 1]
            assert isinstance(coll, CollectiveComm) and coll.op == CollectiveOp.ALL_REDUCE
            assert (coll.src, coll.dst) == ("buf", "buf")
            want = (AxisSlice(0, 4), AxisSlice(2 * idx, 2 * idx + 2))
            assert tuple(coll.src_slice) == want and tuple(coll.dst_slice) == want
            assert isinstance(flag, IntraNodeSignal) and (flag.offset, flag.rank) == (idx, rank)

    _, gated = _collective_info(build_all_reduce_plan, 2, shape=(4, 4), dtype=torch.float32, buffer_name="buf",
                                compute_producer=True)
    assert gated.compute_signal_num == 1
    for rank in range(2):
        wait, coll, flag = gated.operations[rank][0]
        assert isinstance(wait, WaitIntraNodeSignal) and wait.signal_type == SignalType.COMPUTE_DONE
        assert isinstance(coll, CollectiveComm) and isinstance(flag, IntraNodeSignal)


def test_reduce_scatter_collective_slabs_and_destination_schedule():
    from syncopate_amd.communication.comm_runtime.operations import CollectiveComm
    from syncopate_amd.communication.common_descriptors import build_reduce_scatter_collective_plan
    from syncopate_amd.communication.descriptor import AxisSlice, CollectiveOp

    kw = dict(shape=(4, 4), dtype=torch.float32, axis=0, split_axis=1, src_buffer="src", dst_buffer="dst")
    gen, info = _collective_info(build_reduce_scatter_collective_plan, 2, num_reduce_scatters=2, **kw)
    assert info.world_size == 2 and info.recv_signal_num == 2
    for rank in range(2):
        (ops,) = info.operations[rank]
        assert len(ops) == 4
        for idx in range(2):
            coll, flag = ops[2 * idx], ops[2 * idx + 1]
            assert isinstance(coll, CollectiveComm) and coll.op == CollectiveOp.REDUCE_SCATTER
            assert (coll.src, coll.dst) == ("src", "dst")
            assert tuple(coll.src_slice) == (AxisSlice(0, 4), AxisSlice(2 * idx, 2 * idx + 2))
            assert tuple(coll.dst_slice) == (AxisSlice(0, 2), AxisSlice(2 * idx, 2 * idx + 2))
            assert isinstance(flag, IntraNodeSignal) and (flag.offset, flag.rank) == (idx, rank)
    # the consumer of the result sees one wave per collective, one tile each
    fresh = CommGenerator({r: build_reduce_scatter_collective_plan(mesh_size=2, rank=r, num_reduce_scatters=2, **kw)
                           for r in range(2)})
    fresh.plan_signals()
    lowered = lower_comm_plan_to_raw_schedules(fresh)
    for rank in range(2):
        schedule = lowered[rank]["dst"]
        assert schedule.global_shape == (2, 4) and schedule.num_waves == 2
        assert all(len(wave) == 1 for wave in schedule.block_infos)

    _, gated = _collective_info(build_reduce_scatter_collective_plan, 2, compute_producer=True, **kw)
    assert gated.compute_signal_num == 1
    for rank in range(2):
        wait, coll, flag = gated.operations[rank][0]
        assert isinstance(wait, WaitIntraNodeSignal) and wait.signal_type == SignalType.COMPUTE_DONE
        assert isinstance(coll, CollectiveComm) and isinstance(flag, IntraNodeSignal)


def test_collective_plan_argument_errors():
    from syncopate_amd.communication.common_descriptors import (
        build_all_reduce_nvsharp_plan,
        build_all_reduce_plan,
        build_reduce_scatter_collective_plan,
    )

    ar = dict(dtype=torch.float16, mesh_size=2, rank=0, buffer_name="b")
    with pytest.raises(ValueError):
        build_all_reduce_plan((4, 4), num_all_reduces=2, **ar)                  # which axis to cut?
    with pytest.raises(ValueError):
        build_all_reduce_plan((4, 6), num_all_reduces=4, split_axis=1, **ar)    # 6 % 4
    with pytest.raises(IndexError):
        build_all_reduce_plan((4, 4), num_all_reduces=2, split_axis=2, **ar)
    with pytest.raises(ValueError):
        build_all_reduce_plan((), **ar)
    with pytest.raises(ValueError):
        build_all_reduce_plan((4, 4), num_all_reduces=0, split_axis=0, **ar)
    two = build_all_reduce_nvsharp_plan((4, 4), dtype=torch.float16, mesh_size=2, rank=1, src_name="s", dst_name="d",
                                        num_all_reduces=2, split_axis=-1)
    assert set(two.tensors_involved) == {"s", "d"} and not two.local_regions
    rs = dict(dtype=torch.float16, mesh_size=2, rank=0, src_buffer="s", dst_buffer="d")
    with pytest.raises(ValueError):
        build_reduce_scatter_collective_plan((4, 4), axis=0, split_axis=0, **rs)     # cut along the scattered axis
    with pytest.raises(ValueError):
        build_reduce_scatter_collective_plan((4,), axis=0, **rs)                      # no other axis to cut
    with pytest.raises(ValueError):
        build_reduce_scatter_collective_plan((3, 4), axis=0, **rs)                    # 3 % 2
    with pytest.raises(ValueError):
        build_reduce_scatter_collective_plan((4, 4), axis=0, num_reduce_scatters=2, **rs)
    plan = build_reduce_scatter_collective_plan((4, 4, 6), axis=2, **rs)              # default: wraps to axis 0
    assert plan.tensors_involved["d"][0] == torch.Size((4, 4, 3))
