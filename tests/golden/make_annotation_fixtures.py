"""Write tests/golden/annotation_cases.json: what a parser of the `@sy.*` annotations and the
argument lists of an annotation transformer give for the annotated snippets below.

Run once in the build container, where the reference checkout is mounted:

    python tests/golden/make_annotation_fixtures.py            # reference implementation -> fixture
    python tests/golden/make_annotation_fixtures.py --self     # this repository's implementation (for diffing)

Only the reference's pure-Python transform modules are imported (annotation parser, the
transformer's constructor and its argument-list helpers); no kernel is compiled or run.  The
snippets are written for this fixture; the file holds them (inputs) and the parsed fields, argument
lists and error messages (outputs) - data only.
"""

import argparse
import dataclasses
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))

SNIPPETS = {
    "gemm_one_tile_per_program": """
def scaled_matmul(a_ptr, b_ptr, c_ptr, M, N, K, BM: tl.constexpr, BN: tl.constexpr, GROUP: tl.constexpr):
    pid = tl.program_id(axis=0)  # @sy.tile_id
    tiles_m = tl.cdiv(M, BM)  # @sy.axis_count M block=BM
    tiles_n = tl.cdiv(N, BN)  # @sy.axis_count N block=BN
    # @sy.dispatch begin
    pid_m, pid_n = swizzle(pid, tiles_m, tiles_n, GROUP)
    # @sy.pid_map M=pid_m N=pid_n
    # @sy.dispatch end
    run_tile(pid_m, pid_n)
""",
    "gemm_persistent_with_epilogue": """
def looping_matmul(a_ptr, b_ptr, c_ptr, M, N, K, BM: tl.constexpr, BN: tl.constexpr, PROGRAMS: tl.constexpr):
    first = tl.program_id(axis=0)
    tiles_m = tl.cdiv(M, BM)   # @sy.axis_count M block=BM
    tiles_n = tl.cdiv(N, BN)   # @sy.axis_count N block=BN
    total = tiles_m * tiles_n  # @sy.num_tiles
    tile = first - PROGRAMS    # @sy.tile_id persistent
    # @sy.persistent_init begin
    # @sy.persistent_init end
    for _ in range(first, total, PROGRAMS):
        tile += PROGRAMS
        # @sy.dispatch begin
        pid_m, pid_n = swizzle(tile, tiles_m, tiles_n, 8)
        # @sy.pid_map M=pid_m N=pid_n
        # @sy.dispatch end
        acc = run_tile(pid_m, pid_n)
        store_tile(c_ptr, pid_m, pid_n, acc)
        # @sy.producer_epilogue
""",
    "attention_with_kv_range": """
def flash_forward(q, k, v, o, Z, H, SQ, SKV, BQ: tl.constexpr, BKV: tl.constexpr):
    work = tl.program_id(0) + tl.program_id(1) * tl.num_programs(0)  # @sy.tile_id
    zs = Z                      # @sy.axis_count Z
    hs = H                      # @sy.axis_count H
    qs = tl.cdiv(SQ, BQ)        # @sy.axis_count Q block=BQ
    kvs = tl.cdiv(SKV, BKV)     # @sy.axis_count KV=range block=BKV
    # @sy.dispatch begin
    pid_z, pid_h, pid_q, kv_lo, kv_hi = unravel(work, zs, hs, qs, kvs)
    # @sy.pid_map Z=pid_z H=pid_h Q=pid_q KV=kv_lo..kv_hi
    # @sy.dispatch end
    attend(pid_z, pid_h, pid_q, kv_lo, kv_hi)
""",
    "batched_rows_have_no_template": """
def rowwise(x, y, B, R, BR: tl.constexpr):
    pid = tl.program_id(0)      # @sy.tile_id
    nb = B                      # @sy.axis_count B
    nr = tl.cdiv(R, BR)         # @sy.axis_count R block=BR
    # @sy.dispatch begin
    pid_b, pid_r = divmod(pid, nr)
    # @sy.pid_map B=pid_b R=pid_r
    # @sy.dispatch end
""",
    "gemm_split_k_persistent": """
def split_k(a, b, c, M, N, K, BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr, PROGRAMS: tl.constexpr):
    first = tl.program_id(0)
    tm = tl.cdiv(M, BM)         # @sy.axis_count M block=BM
    tn = tl.cdiv(N, BN)         # @sy.axis_count N block=BN
    tk = tl.cdiv(K, BK)         # @sy.axis_count K=range block=BK
    tile = first - PROGRAMS     # @sy.tile_id persistent
    # @sy.persistent_init begin
    # @sy.persistent_init end
    for _ in range(first, tm * tn, PROGRAMS):
        tile += PROGRAMS
        # @sy.dispatch begin
        pid_m, pid_n, k_lo, k_hi = split(tile, tm, tn, tk)
        # @sy.pid_map M=pid_m N=pid_n K=k_lo..k_hi
        # @sy.dispatch end
        add_into(c, pid_m, pid_n, contract(a, b, pid_m, pid_n, k_lo, k_hi))
        # @sy.producer_epilogue
""",
}

# every line of `base` that contains `drop` is removed, then `add` lines are appended
BROKEN = {
    "no_tile_id": ("gemm_one_tile_per_program", "@sy.tile_id", []),
    "no_dispatch": ("gemm_one_tile_per_program", "@sy.dispatch", []),
    "no_axis_count": ("gemm_one_tile_per_program", "@sy.axis_count", []),
    "no_pid_map": ("gemm_one_tile_per_program", "@sy.pid_map", []),
    "persistent_without_init": ("gemm_persistent_with_epilogue", "@sy.persistent_init", []),
    "two_epilogues": ("gemm_persistent_with_epilogue", "\0", ["        # @sy.producer_epilogue"]),
    "bad_axis_suffix": ("gemm_one_tile_per_program", "\0", ["    extra = 3  # @sy.axis_count K=span block=4"]),
    "empty_block": ("gemm_one_tile_per_program", "\0", ["    extra = 3  # @sy.axis_count K block="]),
    "bad_pid_map_entry": ("gemm_one_tile_per_program", "\0", ["    # @sy.pid_map K"]),
    "count_not_an_assignment": ("gemm_one_tile_per_program", "\0", ["    tl.cdiv(M, 3)  # @sy.axis_count K"]),
    "end_before_begin": ("gemm_one_tile_per_program", "@sy.dispatch begin", ["    # @sy.dispatch begin"]),
}

TRANSFORMERS = {
    "local": {},
    "consumer": {"enable_consumer": True},
    "producer": {"enable_producer": True},
    "consumer_and_producer": {"enable_consumer": True, "enable_producer": True},
    "one_peer_descriptor": {"enable_producer": True, "remote": ["c_desc"]},
    "two_peer_descriptors": {"enable_consumer": True, "remote": ["a_desc", "c_desc"]},
}


def broken_source(name):
    base, drop, add = BROKEN[name]
    lines = [l for l in SNIPPETS[base].splitlines() if drop not in l]
    return "\n".join(lines + add) + "\n"


def load(use_self):
    if use_self:
        sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
        from syncopate_amd.computation.transform import AnnotationTransformer, RemoteBinding, parse_annotations
    else:
        sys.path.insert(0, os.environ.get("SYNCOPATE_REFERENCE", "/root/reference"))
        from syncopate.computation.transform.annotations import parse_annotations
        from syncopate.computation.transform.transformer import AnnotationTransformer, RemoteBinding
    return parse_annotations, AnnotationTransformer, RemoteBinding


def arg_lists(transformer, use_self):
    if use_self:
        from syncopate_amd.computation.transform.binder import KernelBinding

        def text(persistent):
            return KernelBinding(template="gemm", persistent=persistent, annotations=None, consumer=False,
                                 producer=False, extra_args=transformer.extra_args(persistent)).signature()
        return {"persistent": text(True), "one_tile_per_program": text(False)}
    return {"persistent": transformer._persistent_extra_args(),
            "one_tile_per_program": transformer._nonpersistent_extra_args()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--self", dest="use_self", action="store_true")
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    parse_annotations, AnnotationTransformer, RemoteBinding = load(args.use_self)

    result = {"snippets": SNIPPETS, "parsed": {}, "errors": {}, "broken_sources": {}, "argument_lists": {}}
    for name, source in SNIPPETS.items():
        result["parsed"][name] = dataclasses.asdict(parse_annotations(source.splitlines()))
    for name in BROKEN:
        source = broken_source(name)
        result["broken_sources"][name] = source
        try:
            parse_annotations(source.splitlines())
            result["errors"][name] = None
        except Exception as exc:  # noqa: BLE001 - the class and the text are what the fixture records
            result["errors"][name] = [type(exc).__name__, str(exc)]
    for name, cfg in TRANSFORMERS.items():
        kwargs = {k: v for k, v in cfg.items() if k != "remote"}
        if "remote" in cfg:
            kwargs["remote_descriptors"] = {d: RemoteBinding(base_ptr_arg="c_ptr", schedule=None) for d in cfg["remote"]}
        result["argument_lists"][name] = arg_lists(AnnotationTransformer(**kwargs), args.use_self)

    path = args.out or os.path.join(HERE, "annotation_cases_self.json" if args.use_self else "annotation_cases.json")
    with open(path, "w") as f:
        json.dump(result, f, indent=1, sort_keys=True)
    print(f"wrote {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
