"""The `@sy.*` annotation parser and binder against the reference's parser and argument lists
(tests/golden/annotation_cases.json, made by tests/golden/make_annotation_fixtures.py from
syncopate/computation/transform/annotations.py and transformer.py), and the rules of the binder
that have no counterpart there (template choice, `//` comments).
"""

import dataclasses
import json
import os

import pytest
import torch

from syncopate_amd.communication.code_gen import CommGenerator
from syncopate_amd.communication.common_descriptors import (
    build_all_gather_plan_1d_swizzle,
    build_reduce_scatter_direct_reduce_plan,
)
from syncopate_amd.computation.transform import (
    AnnotationError,
    AnnotationTransformer,
    RemoteBinding,
    parse_annotations,
)
from syncopate_amd.interface import lower_comm_plan_to_raw_schedules

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "annotation_cases.json")))
TRANSFORMERS = {
    "local": {},
    "consumer": {"enable_consumer": True},
    "producer": {"enable_producer": True},
    "consumer_and_producer": {"enable_consumer": True, "enable_producer": True},
    "one_peer_descriptor": {"enable_producer": True, "remote": ["c_desc"]},
    "two_peer_descriptors": {"enable_consumer": True, "remote": ["a_desc", "c_desc"]},
}


@pytest.mark.parametrize("name", sorted(GOLDEN["snippets"]))
def test_parsed_fields_match_the_reference_parser(name):
    parsed = parse_annotations(GOLDEN["snippets"][name].splitlines())
    assert dataclasses.asdict(parsed) == GOLDEN["parsed"][name]


@pytest.mark.parametrize("name", sorted(GOLDEN["errors"]))
def test_malformed_annotations_raise_like_the_reference(name):
    kind, text = GOLDEN["errors"][name]
    assert kind == "AnnotationError"
    with pytest.raises(AnnotationError) as caught:
        parse_annotations(GOLDEN["broken_sources"][name].splitlines())
    assert str(caught.value) == text


@pytest.mark.parametrize("name", sorted(TRANSFORMERS))
def test_appended_arguments_match_the_reference_transformer(name):
    cfg = dict(TRANSFORMERS[name])
    remote = cfg.pop("remote", [])
    assert sorted(GOLDEN["argument_lists"]) == sorted(TRANSFORMERS)

    class _Schedule:                      # only the names matter for the argument lists
        def role(self):
            return "producer"

        def is_reduce(self):
            return False

    transformer = AnnotationTransformer(
        remote_descriptors={d: RemoteBinding(base_ptr_arg="c_ptr", schedule=_Schedule()) for d in remote}, **cfg)
    want = GOLDEN["argument_lists"][name]
    source = {True: GOLDEN["snippets"]["gemm_persistent_with_epilogue"],
              False: GOLDEN["snippets"]["gemm_one_tile_per_program"]}
    for persistent, key in ((True, "persistent"), (False, "one_tile_per_program")):
        if cfg.get("enable_producer") and not persistent:
            with pytest.raises(AnnotationError):        # no @sy.producer_epilogue in that snippet
                transformer.transform(source[persistent])
            continue
        binding = transformer.transform(source[persistent])
        assert binding.signature() == want[key]
        assert binding.persistent is persistent and binding.template == "gemm"
        assert binding.tile_shape == ("BM", "BN")


def test_hip_comments_parse_like_python_comments():
    python_form = GOLDEN["snippets"]["gemm_persistent_with_epilogue"]
    hip_form = """
    __global__ void looping_matmul(Params p) {
        const int tiles_m = ceil_div(p.M, BM);   // @sy.axis_count M block=BM
        const int tiles_n = ceil_div(p.N, BN);   // @sy.axis_count N block=BN
        int tile = blockIdx.x - gridDim.x;       // @sy.tile_id persistent
        // @sy.persistent_init begin
        // @sy.persistent_init end
        for (;;) {
            tile += gridDim.x;
            // @sy.dispatch begin
            const int2 pid = swizzle(tile, tiles_m, tiles_n, 8);
            // @sy.pid_map M=pid_m N=pid_n
            // @sy.dispatch end
            // @sy.producer_epilogue
        }
    }
    """
    a = parse_annotations(python_form.splitlines())
    b = parse_annotations(hip_form.splitlines())
    assert [(c.axis, c.var, c.kind, c.block) for c in b.axis_counts] == \
        [(c.axis, c.var, c.kind, c.block) for c in a.axis_counts]
    assert b.axis_counts[0].expr == "ceil_div(p.M, BM)"
    assert (b.tile_id_var, b.tile_id_expr, b.persistent) == ("tile", "blockIdx.x - gridDim.x", True)
    assert b.pid_map == a.pid_map and b.producer_epilogue is not None and b.persistent_init is not None
    assert AnnotationTransformer(enable_producer=True).transform(hip_form).template == "gemm"


def test_template_choice():
    snippets = GOLDEN["snippets"]
    attention = AnnotationTransformer(enable_consumer=True).transform(snippets["attention_with_kv_range"])
    assert attention.template == "attention" and not attention.persistent
    assert attention.tile_shape == ("1", "1", "BQ")
    assert [n for n, _ in attention.extra_args] == ["wave_offsets", "wave_sizes", "cum_wave_sizes", "signal_ptr",
                                                    "signal_offsets", "cum_tiles", "NUM_WAVES"]
    split_k = AnnotationTransformer(enable_consumer=True).transform(snippets["gemm_split_k_persistent"])
    assert split_k.template == "gemm_splitk" and split_k.persistent and split_k.tile_shape == ("BM", "BN")
    assert [a.kind for a in split_k.annotations.axis_counts] == ["single", "single", "range"]
    with pytest.raises(AnnotationError, match="no HIP template"):
        AnnotationTransformer().transform(snippets["batched_rows_have_no_template"])
    with pytest.raises(AnnotationError, match="producer_epilogue"):
        AnnotationTransformer(enable_producer=True).transform(snippets["attention_with_kv_range"])
    with pytest.raises(ValueError):
        AnnotationTransformer(enable_consumer=True, consumer_descriptors=())


def _schedule(plans, rank, name):
    gen = CommGenerator(plans)
    gen.plan_signals()
    return lower_comm_plan_to_raw_schedules(gen)[rank][name]


def test_bound_descriptors_take_role_and_reduce_flag_from_the_schedule():
    world = 4
    push = _schedule({r: build_reduce_scatter_direct_reduce_plan(
        shape=(1024, 512), dtype=torch.float16, axis=0, mesh_size=world, rank=r, src_buffer="src",
        dst_buffer="dst", transfer_kind="push") for r in range(world)}, 1, "src")
    gathered = _schedule({r: build_all_gather_plan_1d_swizzle((1024, 256), torch.float16, 0, world, r, "a", "pull")
                          for r in range(world)}, 1, "a")
    source = GOLDEN["snippets"]["gemm_persistent_with_epilogue"]
    one = AnnotationTransformer(remote_descriptors={"c_desc": RemoteBinding("c_ptr", push)}).transform(source)
    slot = one.remote["c_desc"]
    assert (slot.role, slot.is_reduce, slot.target_rank_arg, slot.dst_offsets_arg) == \
        ("producer", True, "target_rank", "dst_offsets")
    two = AnnotationTransformer(remote_descriptors={"a_desc": RemoteBinding("a_ptr", gathered),
                                                    "c_desc": RemoteBinding("c_ptr", push)}).transform(source)
    assert (two.remote["a_desc"].role, two.remote["a_desc"].is_reduce) == ("consumer", False)
    assert two.remote["a_desc"].target_rank_arg == "target_rank_a_desc"
    assert two.remote["c_desc"].dst_offsets_arg == "dst_offsets_c_desc"


def test_launch_checks_its_tables_before_touching_the_device():
    source = GOLDEN["snippets"]["gemm_persistent_with_epilogue"]
    consumer = AnnotationTransformer(enable_consumer=True).transform(source)
    with pytest.raises(ValueError, match="cur_wave_sizes"):
        consumer.launch(None, None, None, 4, 8, signal_ptr=object(), signal_offsets=[0])
    producer = AnnotationTransformer(enable_producer=True).transform(source)
    with pytest.raises(ValueError, match="counter_ptr"):
        producer.launch(None, None, None, 4, 8, cur_wave_sizes=[[1, 1]], wave_offsets=[[0, 0]])
    both = AnnotationTransformer(enable_consumer=True, enable_producer=True).transform(source)
    with pytest.raises(ValueError, match="counter_ptr"):          # the producer's tables go by producer_* names
        both.launch(None, None, None, 4, 8, cur_wave_sizes=[[1, 1]], wave_offsets=[[0, 0]])
    split = AnnotationTransformer(enable_consumer=True, enable_producer=True) \
        .transform(GOLDEN["snippets"]["gemm_split_k_persistent"])
    with pytest.raises(NotImplementedError):                      # both roles: GEMM and attention templates only
        split.launch(None, None, None, 4, 8, cur_wave_sizes=[[1, 1, 1]], wave_offsets=[[0, 0, 0]])
