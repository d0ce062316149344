"""Signal planning and period estimation, against the vectors in the reference's
tests/test_comm_plan.py, tests/test_plan_compute_signal.py and tests/test_descriptor.py:360-380."""

import pytest
import torch

from syncopate_amd.communication.common_descriptors import (
    build_all_gather_plan_1d_swizzle,
    build_all_to_all_plan,
    build_double_ring_all_gather_plan,
    build_ring_all_gather_plan,
)
from syncopate_amd.communication.descriptor import (
    BufferRegion,
    Collective,
    CollectiveOp,
    CommPlan,
    ComputeDependency,
    DevicePlan,
    SignalType,
    Transfer,
    TransferOp,
    XferDependency,
)


def _push(src, dst, chunk=0):
    word = BufferRegion.contiguous(offset=0, nbytes=4)
    return Transfer(op=TransferOp.PUSH, src_buf=f"buf{src}", src_region=word, dst_buf=f"buf{dst}",
                    dst_region=word, chunk_idx=chunk, peer=dst)


def test_ring_reuses_receive_signals():         # reference test_comm_plan.py:33-72
    p01, p12, p20 = _push(0, 1), _push(1, 2), _push(2, 0)
    p12.dependency.append(XferDependency(0, 0, 0))
    p20.dependency.append(XferDependency(1, 0, 0))
    cp = CommPlan({0: DevicePlan(dev=0, xfer=[[p01]]), 1: DevicePlan(dev=1, xfer=[[p12]]),
                   2: DevicePlan(dev=2, xfer=[[p20]])})
    cp.plan_signals()
    s0, s1, s2 = (p.set_signals[0] for p in (p01, p12, p20))
    assert [(s.dst_rank, s.dst_offset, s.type) for s in (s0, s1, s2)] == [
        (1, 0, SignalType.RECEIVE_DATA), (2, 0, SignalType.RECEIVE_DATA), (0, 0, SignalType.RECEIVE_DATA)]
    assert p12.dependency[0].signal is s0 and p20.dependency[0].signal is s1
    assert all(not p.transit_signals for p in cp.device_plans.values())
    assert cp.visualize_signals() == "\n".join([
        "CommPlan Signals:",
        "  Device 0:",
        "    Stream 0:",
        "      op[0] push -> signals: receive_data@1[0]",
        "  Device 1:",
        "    Stream 0:",
        "      op[0] push -> signals: receive_data@2[0]",
        "        dep[0] <- xfer(0,0,0) -> receive_data@1[0]",
        "  Device 2:",
        "    Stream 0:",
        "      op[0] push -> signals: receive_data@0[0]",
        "        dep[0] <- xfer(1,0,0) -> receive_data@2[0]",
    ])


def test_third_party_dependency_gets_transit_signal():    # reference test_comm_plan.py:75-118
    push = _push(0, 1)
    word = BufferRegion.contiguous(0, 4)
    copy = Transfer(op=TransferOp.LOCAL_COPY, src_buf="buf2", src_region=word, dst_buf="buf2_out",
                    dst_region=word, chunk_idx=0)
    copy.dependency.append(XferDependency(0, 0, 0))
    cp = CommPlan({0: DevicePlan(dev=0, xfer=[[push]]), 1: DevicePlan(dev=1, xfer=[[]]),
                   2: DevicePlan(dev=2, xfer=[[copy]])})
    cp.plan_signals()
    landed, own = push.set_signals[0], copy.set_signals[0]
    assert (landed.dst_rank, landed.type) == (1, SignalType.RECEIVE_DATA)
    assert (own.dst_rank, own.type) == (2, SignalType.RECEIVE_DATA)
    ((got, relay),) = cp.device_plans[1].transit_signals
    assert got is landed and (relay.type, relay.dst_rank, relay.dst_offset) == (SignalType.REMOTE_DATA_READY, 2, 0)
    assert copy.dependency[0].signal is relay
    viz = cp.visualize_signals()
    assert "    Stream 0: (none)" in viz
    assert viz.endswith("    Transit signals:\n      receive_data@1[0] -> remote_data_ready@2[0]") is False
    assert "    Transit signals:\n      receive_data@1[0] -> remote_data_ready@2[0]" in viz
    assert cp.transit_signal_counters == {0: 0, 1: 0, 2: 1}


def test_dependency_on_remote_pull_adds_a_second_set_signal():
    word = BufferRegion.contiguous(0, 4)
    pull = Transfer(op=TransferOp.PULL, src_buf="a", src_region=word, dst_buf="a", dst_region=word,
                    chunk_idx=0, peer=1)
    local = Transfer(op=TransferOp.LOCAL_COPY, src_buf="a", src_region=word, dst_buf="b", dst_region=word,
                     chunk_idx=0, dependency=[XferDependency(0, 0, 0)])
    watcher = Transfer(op=TransferOp.LOCAL_COPY, src_buf="a", src_region=word, dst_buf="b", dst_region=word,
                       chunk_idx=0, dependency=[XferDependency(0, 0, 0)])
    cp = CommPlan({0: DevicePlan(dev=0, xfer=[[pull, local]]), 1: DevicePlan(dev=1, xfer=[[watcher]])})
    cp.plan_signals()
    assert local.dependency[0].signal is pull.set_signals[0]            # same rank: reuse
    extra = watcher.dependency[0].signal
    assert pull.set_signals == [pull.set_signals[0], extra]
    # rank 1's own op took receive offset 0 in pass 1; the extra signal is the next word
    assert (extra.type, extra.dst_rank, extra.dst_offset) == (SignalType.REMOTE_DATA_READY, 1, 1)


def _a2a_plans(kind, mesh=4):
    return {r: build_all_to_all_plan(shape=(4, 4), dtype=torch.float32, mesh_size=mesh, rank=r,
                                     src_buffer="src", dst_buffer="dst", transfer_kind=kind,
                                     compute_producer=True) for r in range(mesh)}


@pytest.mark.parametrize("kind", ["push", "pull"])
def test_compute_dependencies_get_one_flag_each(kind):   # reference test_plan_compute_signal.py:39-81
    cp = CommPlan(_a2a_plans(kind))
    cp.plan_signals(plan_compute_signals=True)
    for dev, plan in cp.device_plans.items():
        deps = [d for op in plan.xfer[0] for d in op.dependency if isinstance(d, ComputeDependency)]
        assert [d.signal.dst_offset for d in deps] == [0, 1, 2, 3]
        assert all(d.signal.type == SignalType.COMPUTE_DONE for d in deps)
        if kind == "push":
            assert all(d.signal.dst_rank == dev for d in deps)
        else:
            assert [d.signal.dst_rank for d in deps] == [(dev + i) % 4 for i in (1, 2, 3)] + [dev]
        assert plan.transit_signals == []
    assert cp.compute_signal_counters == {r: 4 for r in range(4)}


def test_push_receive_offsets_follow_device_iteration_order():
    """PUSH signals are numbered at the DESTINATION in the order devices are visited."""
    cp = CommPlan(_a2a_plans("push"))
    cp.plan_signals()
    recv = {r: [(op.set_signals[0].dst_rank, op.set_signals[0].dst_offset) for op in cp.device_plans[r].xfer[0]]
            for r in range(4)}
    assert recv[0] == [(1, 0), (2, 0), (3, 0), (0, 0)]
    assert recv[1] == [(2, 1), (3, 1), (0, 1), (1, 1)]
    assert recv[2] == [(3, 2), (0, 2), (1, 2), (2, 2)]
    assert recv[3] == [(0, 3), (1, 3), (2, 3), (3, 3)]


def test_planning_preconditions():
    cp = CommPlan(_a2a_plans("push"))
    cp.plan_signals()
    with pytest.raises(AssertionError):
        cp.plan_signals()                       # set_signals already present
    cp2 = CommPlan(_a2a_plans("push"))
    with pytest.raises(AssertionError):
        cp2.plan_signals(plan_compute_signals=False)   # compute signals must then be pre-set
    word = BufferRegion.contiguous(0, 4)
    coll = Collective(op=CollectiveOp.ALL_REDUCE, src_buf="a", src_region=word, dst_buf="a", dst_region=word,
                      dependency=[XferDependency(0, 0, 0)])
    cp3 = CommPlan({0: DevicePlan(dev=0, xfer=[[_push(0, 1), coll]]), 1: DevicePlan(dev=1)})
    with pytest.raises(ValueError):
        cp3.plan_signals()
    cp4 = CommPlan({0: DevicePlan(dev=0, xfer=[[_push(0, 2)]])})
    with pytest.raises(ValueError):
        cp4.plan_signals()                      # peer 2 has no counter
    with pytest.raises(ValueError):
        cp4.add_device_plan(DevicePlan(dev=0))


def test_period_estimate_swizzle_and_ring():   # reference test_descriptor.py:360-380
    plans = {r: build_all_gather_plan_1d_swizzle((16, 2), torch.float16, 0, 4, r, "buf", "push") for r in range(4)}
    cp = CommPlan(device_plans=plans)
    cp.estimate_period()
    assert [x.period.start for x in plans[1].xfers] == pytest.approx([0.0, 1.0, 2.0])
    ring = {r: build_ring_all_gather_plan((16, 2), torch.float16, 0, 4, r, "buf") for r in range(4)}
    cp = CommPlan(ring)
    cp.plan_signals()
    cp.estimate_period()
    for r in range(4):
        assert [x.period.start for x in ring[r].xfers] == [0.0, 1.0, 2.0]
        assert [x.set_signals[0].period.start for x in ring[r].xfers] == [1.0, 2.0, 3.0]


def test_period_estimate_double_ring_and_cycle():
    plans = {r: build_double_ring_all_gather_plan((8, 2), torch.float16, 0, 8, 2, r, "b") for r in range(8)}
    cp = CommPlan(plans)
    cp.estimate_period()
    assert [op.period.start for op in plans[0].xfer[0]] == [0.0, 1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
    a, b = _push(0, 1), _push(1, 0)
    a.dependency.append(XferDependency(1, 0, 0))
    b.dependency.append(XferDependency(0, 0, 0))
    loop = CommPlan({0: DevicePlan(dev=0, xfer=[[a]]), 1: DevicePlan(dev=1, xfer=[[b]])})
    with pytest.raises(RuntimeError):
        loop.estimate_period()
    a.dependency[0] = XferDependency(5, 0, 0)
    with pytest.raises(ValueError):
        loop.estimate_period()
    CommPlan({}).estimate_period()


def test_plan_pretty_with_signals():
    plans = {r: build_all_gather_plan_1d_swizzle((8, 2), torch.float16, 0, 2, r, "buf", "pull") for r in range(2)}
    cp = CommPlan(plans)
    cp.plan_signals()
    assert cp.pretty(include_signals=True) == "\n".join([
        "CommPlan(devices=2)",
        "  DevicePlan(dev=0)",
        "    Stream 0:",
        "      [0] pull peer=1 buf[4:8, 0:2] -> buf[4:8, 0:2]",
        "    Stream 0:",
        "      op[0] pull -> signals: receive_data@0[0]",
        "  DevicePlan(dev=1)",
        "    Stream 0:",
        "      [0] pull peer=0 buf[0:4, 0:2] -> buf[0:4, 0:2]",
        "    Stream 0:",
        "      op[0] pull -> signals: receive_data@1[0]",
    ])


def test_compute_unit_groups_and_mask_words():
    from syncopate_amd.communication.comm_runtime.cu_partition import cu_mask_words, group_sizes

    assert group_sizes(256, 1, 10) == [16, 240]          # a whole number of units per XCD
    assert group_sizes(256, 1, 32) == [32, 224]
    assert group_sizes(256, 3, 8) == [8, 8, 8, 232]
    with pytest.raises(RuntimeError):
        group_sizes(256, 1, 250)                         # nothing would be left for compute
    with pytest.raises(ValueError):
        group_sizes(256, 0, 8)
    assert cu_mask_words(0, 32, 256) == [0xFFFFFFFF] + [0] * 7
    assert cu_mask_words(32, 224, 256) == [0] + [0xFFFFFFFF] * 7
    assert cu_mask_words(30, 4, 64) == [0xC0000000, 0x3]
    with pytest.raises(ValueError):
        cu_mask_words(250, 10, 256)
