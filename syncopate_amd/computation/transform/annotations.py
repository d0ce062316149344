"""The `@sy.*` annotation vocabulary, read from the comments of a kernel's source.

The reference marks up a Triton kernel with these comments and rewrites its text
(syncopate/computation/transform/annotations.py:86-175 parses them).  Here the same vocabulary
describes a kernel's tiling to a binder that picks a HIP kernel template, so the parser reads both
`#` and `//` comments:

    <var> = <expr>      @sy.tile_id [persistent]          the linear tile id
    <var> = <expr>      @sy.axis_count AXIS[=range] [block=<expr>]   tiles along one axis
                        @sy.pid_map AXIS=var ... AXIS=lo..hi          names the dispatch produces
                        @sy.dispatch begin / @sy.dispatch end         the tile-id -> pids block
                        @sy.persistent_init begin / end               loop-carried state of a persistent kernel
                        @sy.producer_epilogue                         where a finished tile is reported
"""

from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Tuple


class AnnotationError(RuntimeError):
    """Malformed, missing or contradictory annotations."""


@dataclass
class AxisCount:
    axis: str       # name as written, e.g. "M", "KV"
    var: str        # variable holding the tile count
    kind: str       # "single": one tile index per work item; "range": a [lo, hi) span of tiles
    expr: str       # right-hand side of the count
    block: str      # elements per tile along the axis ("1" when not given)


@dataclass
class DispatchBlock:
    start: int      # line index of the opening marker
    end: int        # line index of the closing marker (== start for a single marker)
    indent: str


@dataclass
class ParsedAnnotations:
    tile_id_var: str
    tile_id_expr: str
    axis_counts: List[AxisCount]
    pid_map: Dict[str, str]
    dispatch: DispatchBlock
    persistent: bool
    persistent_init: Optional[DispatchBlock]
    producer_epilogue: Optional[DispatchBlock]


_ASSIGN = re.compile(r"^\s*(?P<lhs>[^=]+?)\s*=\s*(?P<rhs>.+?)\s*$")
_COMMENT = re.compile(r"#|//")


def _code_part(line: str) -> str:
    """The line without its trailing comment (and without a statement-ending semicolon)."""
    m = _COMMENT.search(line)
    code = line[:m.start()] if m else line
    return code.rstrip().rstrip(";").rstrip()


def _assignment(line: str) -> Tuple[str, str]:
    code = _code_part(line)
    m = _ASSIGN.match(code)
    if not m:
        raise AnnotationError(f"Expected assignment, got: {code!r}")
    lhs = m.group("lhs").strip().split()[-1]          # drops a C++ type in front of the name
    return lhs, m.group("rhs").strip()


def _after(line: str, tag: str) -> str:
    return line.split(tag, 1)[1].strip()


def _axis_count_fields(line: str) -> Tuple[str, str, str]:
    payload = _after(line, "@sy.axis_count")
    block = "1"
    m = re.search(r"\bblock\s*=\s*(.+)", payload)      # `block=` with nothing behind it is not a block clause
    if m:
        block = m.group(1).strip()
        payload = payload[:m.start()].strip()
    axis, eq, suffix = payload.partition("=")
    axis = axis.strip()
    kind = suffix.strip().lower() if eq else "single"
    if kind not in ("single", "range"):
        raise AnnotationError(f"Unsupported axis_count suffix: {suffix!r}")
    if not axis:
        raise AnnotationError("@sy.axis_count annotation missing axis identifier")
    return axis, kind, block


def _pid_map_fields(line: str) -> Dict[str, str]:
    out: Dict[str, str] = {}
    for part in _after(line, "@sy.pid_map").split():
        if "=" not in part:
            raise AnnotationError(f"Invalid pid_map entry: {part!r}")
        axis, value = part.split("=", 1)
        out[axis.strip()] = value.strip()
    return out


def _indent(line: str) -> str:
    return line[:len(line) - len(line.lstrip())]


def parse_annotations(lines: Iterable[str]) -> ParsedAnnotations:
    tile_id: Optional[Tuple[str, str]] = None
    persistent = False
    counts: List[AxisCount] = []
    pid_map: Dict[str, str] = {}
    marks: Dict[str, Tuple[int, str]] = {}          # marker -> (line index, indent)

    for idx, line in enumerate(lines):
        if "@sy." not in line:
            continue
        if "@sy.tile_id" in line:
            tile_id = _assignment(line)
            persistent = persistent or "persistent" in _after(line, "@sy.tile_id")
        if "@sy.axis_count" in line:
            axis, kind, block = _axis_count_fields(line)
            var, expr = _assignment(line)
            counts.append(AxisCount(axis=axis, var=var, kind=kind, expr=expr, block=block))
        if "@sy.pid_map" in line:
            pid_map.update(_pid_map_fields(line))
        for marker in ("@sy.dispatch begin", "@sy.dispatch end", "@sy.persistent_init begin",
                       "@sy.persistent_init end"):
            if marker in line:
                marks[marker] = (idx, _indent(line))
        if "@sy.producer_epilogue" in line:
            if "@sy.producer_epilogue" in marks:
                raise AnnotationError("Multiple @sy.producer_epilogue annotations found")
            marks["@sy.producer_epilogue"] = (idx, _indent(line))

    if tile_id is None:
        raise AnnotationError("Missing @sy.tile_id annotation")
    if "@sy.dispatch begin" not in marks or "@sy.dispatch end" not in marks:
        raise AnnotationError("Missing @sy.dispatch begin/end annotations")
    if marks["@sy.dispatch begin"][0] >= marks["@sy.dispatch end"][0]:
        raise AnnotationError("@sy.dispatch begin must precede end")
    if not counts:
        raise AnnotationError("At least one @sy.axis_count annotation is required")
    if not pid_map:
        raise AnnotationError("Missing @sy.pid_map annotation")
    has_init = "@sy.persistent_init begin" in marks and "@sy.persistent_init end" in marks
    if persistent and not has_init:
        raise AnnotationError("Persistent kernels must mark initialization with @sy.persistent_init begin/end")

    def block(first: str, last: str) -> DispatchBlock:
        return DispatchBlock(start=marks[first][0], end=marks[last][0], indent=marks[first][1])

    return ParsedAnnotations(
        tile_id_var=tile_id[0],
        tile_id_expr=tile_id[1],
        axis_counts=counts,
        pid_map=pid_map,
        dispatch=block("@sy.dispatch begin", "@sy.dispatch end"),
        persistent=persistent,
        persistent_init=block("@sy.persistent_init begin", "@sy.persistent_init end")
        if "@sy.persistent_init begin" in marks and "@sy.persistent_init end" in marks else None,
        producer_epilogue=block("@sy.producer_epilogue", "@sy.producer_epilogue")
        if "@sy.producer_epilogue" in marks else None,
    )


__all__ = ["AnnotationError", "AxisCount", "DispatchBlock", "ParsedAnnotations", "parse_annotations"]
