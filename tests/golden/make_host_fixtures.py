"""Write tests/golden/host_compiler.json: outputs of a host-side compiler for a fixed list of cases.

Run once in the build container, where the reference checkout is mounted:

    python tests/golden/make_host_fixtures.py            # reference implementation -> fixture
    python tests/golden/make_host_fixtures.py --self     # this repository's implementation (for diffing)

Only the reference's pure-Python host modules are imported (IR, plan builders, op-list
generation, lowering); none of its device code.  The fixture holds inputs (the case list
below) and outputs (flattened schedules, signal tables, op dumps, rendered text) — data only.
These cases cover what the reference's own CPU tests leave open: full-mesh signal-offset
tables at W=8, whole rendered texts, whole op lists.
"""

import argparse
import hashlib
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def load_api(use_self: bool):
    if use_self:
        sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
        import syncopate_amd.communication.common_descriptors as builders
        from syncopate_amd.communication.common_descriptors.reduce_scatter import (
            build_reduce_scatter_direct_reduce_plan,
        )
        from syncopate_amd.communication.code_gen import CodeGenOptions, CommGenerator
        from syncopate_amd.interface.lowering import lower_comm_plan_to_raw_schedules
    else:
        sys.path.insert(0, os.environ.get("SYNCOPATE_REFERENCE", "/root/reference"))
        import syncopate.communication.common_descriptors as builders
        from syncopate.communication.common_descriptors.reduce_scatter import (
            build_reduce_scatter_direct_reduce_plan,
        )
        from syncopate.communication.code_gen import CodeGenOptions, CommGenerator
        from syncopate.interface.lowering import lower_comm_plan_to_raw_schedules
    return builders, build_reduce_scatter_direct_reduce_plan, CodeGenOptions, CommGenerator, \
        lower_comm_plan_to_raw_schedules


# name -> (builder name, kwargs without rank, mesh size, codegen copy_engine flags to dump)
CASES = {
    "ag_swizzle_pull_c1_readme": ("build_all_gather_plan_1d_swizzle",
                                  dict(shape=(1024, 512), dtype="float16", axis=0, buffer_name="a",
                                       transfer_kind="pull"), 4, [True]),
    "ag_swizzle_pull_c1_gathered": ("build_all_gather_plan_1d_swizzle",
                                    dict(shape=(4096, 512), dtype="float16", axis=0, buffer_name="a",
                                         transfer_kind="pull"), 4, [True, False]),
    "ag_swizzle_pull_c2": ("build_all_gather_plan_1d_swizzle",
                           dict(shape=(8192, 8192), dtype="bfloat16", axis=0, buffer_name="a",
                                transfer_kind="pull"), 8, [True]),
    "ag_swizzle_push_small": ("build_all_gather_plan_1d_swizzle",
                              dict(shape=(16, 2), dtype="float16", axis=0, buffer_name="buf",
                                   transfer_kind="push"), 4, [True]),
    "ag_swizzle_pull_kv_seq": ("build_all_gather_plan_1d_swizzle",
                               dict(shape=(2, 1, 4, 1024, 128), dtype="bfloat16", axis=3, buffer_name="kv",
                                    transfer_kind="pull"), 4, [True]),
    "ag_ring_w8": ("build_ring_all_gather_plan",
                   dict(shape=(2, 1, 2, 2048, 128), dtype="bfloat16", axis=3, buffer_name="kv"), 8, [True]),
    "ag_double_ring_c5": ("build_double_ring_all_gather_plan",
                          dict(shape=(2, 1, 32, 32768, 128), dtype="bfloat16", axis=3, inner_mesh_size=2,
                               buffer_name="kv"), 8, [True]),
    "ag_double_ring_9x3": ("build_double_ring_all_gather_plan",
                           dict(shape=(18, 2), dtype="float16", axis=0, inner_mesh_size=3,
                                buffer_name="buf"), 9, [True]),
    "a2a_push_producer_c3": ("build_all_to_all_plan",
                             dict(shape=(8192, 8192), dtype="bfloat16", src_buffer="src", dst_buffer="dst",
                                  transfer_kind="push", compute_producer=True), 8, [True]),
    "a2a_push_consumer_small": ("build_all_to_all_plan",
                                dict(shape=(16, 8), dtype="float16", src_buffer="src", dst_buffer="dst",
                                     transfer_kind="push", compute_producer=False), 4, [True, False]),
    "a2a_pull_producer_small": ("build_all_to_all_plan",
                                dict(shape=(16, 8), dtype="float16", src_buffer="src", dst_buffer="dst",
                                     transfer_kind="pull", compute_producer=True), 4, [True]),
    "a2a_dim_pull_c4": ("build_all_to_all_plan_dim",
                        dict(shape=(3, 1, 32, 2048, 128), dtype="bfloat16", src_buffer="src", dst_buffer="dst",
                             src_split_axis=3, dst_split_axis=2, transfer_kind="pull"), 8, [True]),
    "a2a_dim_push_ccw_small": ("build_all_to_all_plan_dim",
                               dict(shape=(2, 2, 12, 3), dtype="float32", src_buffer="src", dst_buffer="dst",
                                    src_split_axis=1, dst_split_axis=2, transfer_kind="push",
                                    peer_order="counter-clockwise"), 4, [True, False]),
    "a2a_axis_push_producer_attn": ("build_all_to_all_plan_axis",
                                    dict(shape=(2, 12288, 8, 128), dtype="float16", src_buffer="src",
                                         dst_buffer="dst", split_axis=1, transfer_kind="push",
                                         compute_producer=True), 4, [True]),
    "a2a_axis_pull_small": ("build_all_to_all_plan_axis",
                            dict(shape=(2, 8, 3), dtype="float32", src_buffer="src", dst_buffer="dst",
                                 split_axis=-2, transfer_kind="pull", compute_producer=False), 4, [True, False]),
    "a2a_axis_push_w8": ("build_all_to_all_plan_axis",
                         dict(shape=(1, 16384, 4, 128), dtype="bfloat16", src_buffer="src", dst_buffer="dst",
                              split_axis=1, transfer_kind="push", compute_producer=True), 8, [True]),
    "a2a_dim_waves_push_small": ("build_all_to_all_plan_dim_waves",
                                 dict(shape=(2, 8, 2), dtype="float32", src_buffer="src", dst_buffer="dst",
                                      src_split_axis=2, dst_split_axis=1, num_waves=2, transfer_kind="push"),
                                 4, [True, False]),
    "a2a_dim_waves_pull_producer": ("build_all_to_all_plan_dim_waves",
                                    dict(shape=(6, 4), dtype="float16", src_buffer="src", dst_buffer="dst",
                                         src_split_axis=1, dst_split_axis=0, num_waves=3, transfer_kind="pull",
                                         compute_producer=True, peer_order="counter-clockwise"), 2, [True]),
    "a2a_dim_waves_push_producer_gemm": ("build_all_to_all_plan_dim_waves",
                                         dict(shape=(8192, 1024), dtype="bfloat16", src_buffer="src",
                                              dst_buffer="dst", src_split_axis=1, dst_split_axis=0, num_waves=4,
                                              transfer_kind="push", compute_producer=True), 8, [True]),
    "rs_collective_split2_producer": ("build_reduce_scatter_collective_plan",
                                      dict(shape=(64, 32), dtype="float16", axis=0, split_axis=1,
                                           src_buffer="src", dst_buffer="dst", num_reduce_scatters=2,
                                           compute_producer=True), 4, [True]),
    "rs_collective_single_3d": ("build_reduce_scatter_collective_plan",
                                dict(shape=(2, 8, 6), dtype="float32", axis=1, src_buffer="src",
                                     dst_buffer="dst"), 4, [True]),
    "rs_collective_rows_w8": ("build_reduce_scatter_collective_plan",
                              dict(shape=(8192, 1024), dtype="bfloat16", axis=0, split_axis=-1,
                                   src_buffer="src", dst_buffer="dst", num_reduce_scatters=4,
                                   compute_producer=True), 8, [True]),
    "ar_inplace_split4_producer": ("build_all_reduce_plan",
                                   dict(shape=(8192, 1024), dtype="bfloat16", buffer_name="c", num_all_reduces=4,
                                        split_axis=0, compute_producer=True), 8, [True]),
    "ar_inplace_single": ("build_all_reduce_plan",
                          dict(shape=(16, 8), dtype="float16", buffer_name="c"), 4, [True]),
    "ar_two_buffers_split2_producer": ("build_all_reduce_nvsharp_plan",
                                       dict(shape=(64, 32), dtype="float16", src_name="src", dst_name="dst",
                                            num_all_reduces=2, split_axis=1, compute_producer=True), 4, [True]),
    "rs_direct_push": ("build_reduce_scatter_direct_reduce_plan",
                       dict(shape=(64, 32), dtype="float16", axis=0, src_buffer="src", dst_buffer="dst",
                            transfer_kind="push"), 4, [False]),
    "rs_direct_pull": ("build_reduce_scatter_direct_reduce_plan",
                       dict(shape=(64, 32), dtype="float16", axis=0, src_buffer="src", dst_buffer="dst",
                            transfer_kind="pull"), 4, [False]),
}


def text_or_digest(text, limit=4096):
    """Short texts are stored whole; long ones as their length, first lines and SHA-256."""
    if len(text) <= limit:
        return text
    return {"sha256": hashlib.sha256(text.encode()).hexdigest(), "chars": len(text),
            "head": text.splitlines()[:6]}


def dump_schedule(schedule):
    return {
        "num_waves": schedule.num_waves,
        "global_shape": list(schedule.global_shape),
        "blocks_per_wave": [len(w) for w in schedule.block_infos],
        "offsets": schedule.gen_block_offset_lists(),
        "shapes": schedule.gen_block_shape_lists(),
        "signals": schedule.gen_signal_lists(),
        "signal_types": [None if b.signal is None else b.signal.type.value
                         for w in schedule.block_infos for b in w],
        "target_ranks": schedule.gen_target_rank_list(),
        "dst_offsets": schedule.gen_dst_offset_lists(),
        "roles": [b.role for w in schedule.block_infos for b in w],
        "is_reduce": schedule.is_reduce(),
    }


def run_case(api, name):
    import torch

    builders, rs_direct, CodeGenOptions, CommGenerator, lower = api
    builder_name, kwargs, mesh, engines = CASES[name]
    kwargs = dict(kwargs)
    kwargs["dtype"] = getattr(torch, kwargs["dtype"])
    build = rs_direct if builder_name == "build_reduce_scatter_direct_reduce_plan" else getattr(builders, builder_name)

    def fresh():
        gen = CommGenerator({r: build(mesh_size=mesh, rank=r, **kwargs) for r in range(mesh)})
        gen.plan_signals()
        return gen

    gen = fresh()
    out = {
        "plan_text": text_or_digest(gen.pretty()),
        "signal_text": text_or_digest(gen.visualize_signals()),
        "counters": {"recv": dict(gen.receive_signal_counters), "transit": dict(gen.transit_signal_counters),
                     "compute": dict(gen.compute_signal_counters)},
        "comm_info": {},
    }
    lowered = lower(gen)
    out["period_starts"] = {str(r): [[op.period.start for op in stream] for stream in plan.xfer]
                            for r, plan in gen.device_plans.items()}
    out["schedules"] = {str(r): {buf: dump_schedule(s) for buf, s in per.items()} for r, per in lowered.items()}
    for engine in engines:
        info = fresh().generate_code_for_plan(CodeGenOptions(copy_engine=engine))
        out["comm_info"]["copy_engine" if engine else "sm_copy"] = text_or_digest(str(info))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--self", dest="use_self", action="store_true")
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    api = load_api(args.use_self)
    result = {name: run_case(api, name) for name in CASES}
    path = args.out or os.path.join(HERE, "host_compiler_self.json" if args.use_self else "host_compiler.json")
    with open(path, "w") as f:
        json.dump(result, f, separators=(",", ":"), sort_keys=True)
    print(f"wrote {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
