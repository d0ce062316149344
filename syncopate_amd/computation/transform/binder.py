"""Binding an annotated kernel to a HIP kernel template.

The reference's `AnnotationTransformer` (syncopate/computation/transform/transformer.py:1059-1430)
rewrites the text of an annotated Triton kernel: it replaces the marked dispatch block by a lookup
in the wave tables, appends keyword arguments to the kernel's signature and, for a producer, puts a
tile counter and a flag write at the marked epilogue.  The kernels here are compiled HIP templates
that already contain the wave walk, the flag waits and the producer epilogue, so the same
annotations select a template and fix its call form instead: `transform(source)` returns a
`KernelBinding` that knows

  * which template the annotated tiling is (GEMM: single axes M, N; split-K GEMM: the same with a
    range axis K; attention: single axes Z, H, Q and a range axis KV),
  * the keyword arguments the reference would have appended to the kernel (same names, same
    order, same defaults: transformer.py:1125-1178), which are the keywords `launch()` takes,
  * per bound descriptor, whether the compute kernel reads it from a peer or writes / atomically
    adds into a peer (from the schedule's role and reduce flag, transformer.py:1244-1262).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional, Tuple

from ...interface.tile_schedule import RawSchedule
from .annotations import AnnotationError, AxisCount, ParsedAnnotations, parse_annotations


@dataclass(frozen=True)
class RemoteBinding:
    """A kernel-local descriptor bound to a base pointer argument and the schedule of its buffer
    (transformer.py:13-29): the schedule says whether the kernel reads or writes the descriptor
    (`role()`), whether writes accumulate (`is_reduce()`) and which peer each wave addresses
    (`gen_target_rank_list()`, `gen_dst_offset_lists()`)."""

    base_ptr_arg: str
    schedule: RawSchedule


@dataclass(frozen=True)
class RemoteSlot:
    descriptor: str
    base_ptr_arg: str
    target_rank_arg: str
    dst_offsets_arg: str
    is_reduce: bool
    role: Optional[str]


@dataclass
class KernelBinding:
    template: str                               # "gemm", "gemm_splitk" or "attention"
    persistent: bool
    annotations: ParsedAnnotations
    consumer: bool
    producer: bool
    extra_args: List[Tuple[str, Any]]           # (keyword, default) the annotated kernel gains
    remote: Dict[str, RemoteSlot] = field(default_factory=dict)

    @property
    def tile_shape(self) -> Tuple[str, ...]:
        """Block expressions of the axes a work item owns one tile of."""
        return tuple(a.block for a in self.annotations.axis_counts if a.kind != "range")

    def signature(self) -> str:
        """The appended keyword arguments as the reference writes them into the kernel's `def`."""
        parts = []
        for name, default in self.extra_args:
            parts.append("NUM_WAVES: tl.constexpr=0" if name == "NUM_WAVES" else f"{name}={default}")
        return ", ".join(parts)

    # ---- launching the bound template ---------------------------------------------------

    def _take(self, kwargs: Dict[str, Any]) -> Dict[str, Any]:
        known = {name for name, _ in self.extra_args}
        tables = {k: kwargs.pop(k) for k in list(kwargs) if k in known}
        return tables

    def _signal_tables(self, tables: Mapping[str, Any]) -> Tuple[Any, Any, Any]:
        """(flag words, per-wave flag offsets, tile counters) under whichever names the roles gave them;
        with both roles these are the producer's, and the consumer's travel as a second pair."""
        if self.consumer and self.producer:
            if self.template == "gemm_splitk" or self.remote:
                raise NotImplementedError(
                    "both roles at once are bound for the GEMM template without peer descriptors and for "
                    "the attention template")
            return (tables.get("producer_signal_ptr"), tables.get("producer_signal_offsets"),
                    tables.get("producer_counter_ptr"))
        return tables.get("signal_ptr"), tables.get("signal_offsets"), tables.get("counter_ptr")

    def launch(self, *args, **kwargs):
        """Run the bound template.  Positional arguments and tuning keywords are the template's own
        (`computation.gemm.gemm` / `gemm_remote`, `computation.attn.attention_forward`); the wave
        tables, flag arguments and peer tables go by the names in `extra_args`."""
        tables = self._take(kwargs)
        flags, flag_offsets, counters = self._signal_tables(tables)
        if self.producer and counters is None:
            raise ValueError("a producer needs counter_ptr (one zeroed int32 per wave)")
        if not self.producer and counters is not None:
            raise TypeError("counter_ptr given to a kernel bound without enable_producer")
        if self.template == "gemm":
            return self._launch_gemm(args, kwargs, tables, flags, flag_offsets, counters)
        if self.template == "gemm_splitk":
            return self._launch_gemm_splitk(args, kwargs, tables, flags, flag_offsets, counters)
        return self._launch_attention(args, kwargs, tables, flags, flag_offsets, counters)

    def _launch_gemm_splitk(self, args, kwargs, tables, flags, flag_offsets, counters):
        from ..gemm import gemm_splitk

        if self.remote or counters is not None:
            raise NotImplementedError("the split-K template is a consumer that adds into a local result")
        if not self.persistent:
            raise NotImplementedError("the split-K template takes the persistent kernel's tables (cur_wave_sizes)")
        return gemm_splitk(*args, cur_wave_sizes=self._wave_sizes(tables), wave_offsets=tables["wave_offsets"],
                           signal_ptr=flags, signal_offsets=flag_offsets, cum_tiles=tables.get("cum_tiles", 0),
                           **kwargs)

    def _wave_sizes(self, tables: Mapping[str, Any]):
        name = "cur_wave_sizes" if self.persistent else "wave_sizes"
        if tables.get(name) is None or tables.get("wave_offsets") is None:
            raise ValueError(f"{name} and wave_offsets are required")
        return tables[name]

    def _launch_gemm(self, args, kwargs, tables, flags, flag_offsets, counters):
        from ..gemm import gemm, gemm_remote

        sizes = self._wave_sizes(tables)
        if not self.remote:
            if flags is None or flag_offsets is None:
                raise ValueError("signal_ptr and signal_offsets are required")
            if self.consumer and self.producer:
                kwargs = dict(kwargs, consumer_signal_ptr=tables.get("consumer_signal_ptr"),
                              consumer_signal_offsets=tables.get("consumer_signal_offsets"))
            return gemm(*args, cur_wave_sizes=sizes, wave_offsets=tables["wave_offsets"], signal_ptr=flags,
                        signal_offsets=flag_offsets, counter_ptr=counters, cum_tiles=tables.get("cum_tiles", 0),
                        **kwargs)
        if counters is not None:
            raise NotImplementedError("tile counters together with peer-bound descriptors")
        # (a, b, c, world_size, num_gemm_sms, ...) -> gemm_remote has no world_size
        if len(args) < 5:
            raise TypeError("launch(a, b, c, world_size, num_gemm_sms, ...)")
        a, b, c, _world, num_sms, *rest = args
        remote_kw: Dict[str, Any] = {}
        for slot in self.remote.values():
            ranks = tables.get(slot.target_rank_arg)
            if ranks is None:
                raise ValueError(f"{slot.target_rank_arg} is required for descriptor {slot.descriptor}")
            if slot.role == "consumer":
                remote_kw["a_target_rank"] = ranks
            else:
                remote_kw["target_rank"] = ranks
                remote_kw["dst_offsets"] = tables.get(slot.dst_offsets_arg)
                remote_kw["atomic_add"] = slot.is_reduce
        return gemm_remote(a, b, c, num_sms, *rest, cur_wave_sizes=sizes, wave_offsets=tables["wave_offsets"],
                           signal_ptr=flags, signal_offsets=flag_offsets, cum_tiles=tables.get("cum_tiles", 0),
                           **remote_kw, **kwargs)

    def _launch_attention(self, args, kwargs, tables, flags, flag_offsets, counters):
        from ..attn import attention_forward

        if self.remote:
            raise NotImplementedError("peer-bound descriptors of the attention template")
        sizes = self._wave_sizes(tables)
        if self.persistent:
            raise NotImplementedError("the attention template takes cumulative wave sizes (non-persistent form)")
        if tables.get("cum_wave_sizes") is None:
            raise ValueError("cum_wave_sizes is required")
        if flags is None or flag_offsets is None:
            raise ValueError("signal_ptr and signal_offsets are required")
        waves = tables.get("NUM_WAVES") or None
        if self.consumer and self.producer:
            kwargs = dict(kwargs, consumer_signal_ptr=tables.get("consumer_signal_ptr"),
                          consumer_signal_offsets=tables.get("consumer_signal_offsets"))
        return attention_forward(*args, wave_offsets=tables["wave_offsets"], wave_sizes=sizes,
                                 cum_wave_sizes=tables["cum_wave_sizes"], signal_ptr=flags,
                                 signal_offsets=flag_offsets, NUM_WAVES=waves,
                                 cum_tiles=tables.get("cum_tiles") or None, counter_ptr=counters, **kwargs)


def _template_for(parsed: ParsedAnnotations) -> str:
    singles = [a.axis.lower() for a in parsed.axis_counts if a.kind == "single"]
    ranges = [a.axis.lower() for a in parsed.axis_counts if a.kind == "range"]
    if singles == ["m", "n"] and not ranges:
        return "gemm"
    if singles == ["m", "n"] and ranges == ["k"]:
        return "gemm_splitk"
    if singles == ["z", "h", "q"] and ranges == ["kv"]:
        return "attention"
    raise AnnotationError(
        f"no HIP template tiles single axes {singles} with range axes {ranges}: there is a GEMM over "
        "(M, N), the same with a K range per wave, and an attention over (Z, H, Q) with a KV range")


class AnnotationTransformer:
    """Same constructor as the reference's (transformer.py:1062-1123)."""

    def __init__(self, *, enable_consumer: bool = False, consumer_descriptors: Tuple[str, ...] = ("desc_k", "desc_v"),
                 enable_producer: bool = False,
                 remote_descriptors: Optional[Mapping[str, RemoteBinding]] = None) -> None:
        if enable_consumer and not consumer_descriptors:
            raise ValueError("consumer_descriptors must be provided when enabling consumer mode")
        self.enable_consumer = enable_consumer
        self.enable_producer = enable_producer
        self.consumer_descriptors = tuple(consumer_descriptors)
        self.remote_descriptors: Dict[str, RemoteBinding] = dict(remote_descriptors or {})

    # the names below follow transformer.py:1077-1178: with one role the flag arguments are
    # plain `signal_ptr` / `signal_offsets` / `counter_ptr`, with both they carry the role's name
    def _signal_args(self) -> List[Tuple[str, Any]]:
        both = self.enable_consumer and self.enable_producer
        out: List[Tuple[str, Any]] = []
        if self.enable_consumer:
            prefix = "consumer_" if both else ""
            out += [(f"{prefix}signal_ptr", None), (f"{prefix}signal_offsets", None)]
        if self.enable_producer:
            prefix = "producer_" if both else ""
            out += [(f"{prefix}signal_ptr", None), (f"{prefix}signal_offsets", None)]
        return out

    def _counter_args(self) -> List[Tuple[str, Any]]:
        if not self.enable_producer:
            return []
        return [("producer_counter_ptr" if self.enable_consumer else "counter_ptr", None)]

    def _remote_names(self, descriptor: str) -> Tuple[str, str]:
        if len(self.remote_descriptors) <= 1:
            return "target_rank", "dst_offsets"
        return f"target_rank_{descriptor}", f"dst_offsets_{descriptor}"

    def _remote_args(self) -> List[Tuple[str, Any]]:
        out: List[Tuple[str, Any]] = []
        for name in self.remote_descriptors:
            ranks, offsets = self._remote_names(name)
            out += [(ranks, None), (offsets, None)]
        return out

    def extra_args(self, persistent: bool) -> List[Tuple[str, Any]]:
        head = [("cur_wave_sizes", None), ("wave_offsets", None)] if persistent else \
            [("wave_offsets", None), ("wave_sizes", None), ("cum_wave_sizes", None)]
        tail = [("cum_tiles", 0)] + ([] if persistent else [("NUM_WAVES", 0)])
        return head + self._signal_args() + self._counter_args() + self._remote_args() + tail

    def transform(self, source: str) -> KernelBinding:
        parsed = parse_annotations(source.splitlines())
        if self.enable_producer and parsed.producer_epilogue is None:
            raise AnnotationError("Producer kernels must mark epilogue with @sy.producer_epilogue")
        template = _template_for(parsed)
        remote = {}
        for name, binding in self.remote_descriptors.items():
            ranks, offsets = self._remote_names(name)
            role = binding.schedule.role()
            remote[name] = RemoteSlot(descriptor=name, base_ptr_arg=binding.base_ptr_arg, target_rank_arg=ranks,
                                      dst_offsets_arg=offsets, is_reduce=binding.schedule.is_reduce(),
                                      role=None if role is None else str(getattr(role, "value", role)))
        return KernelBinding(template=template, persistent=parsed.persistent, annotations=parsed,
                             consumer=self.enable_consumer, producer=self.enable_producer,
                             extra_args=self.extra_args(parsed.persistent), remote=remote)


__all__ = ["AnnotationTransformer", "KernelBinding", "RemoteBinding", "RemoteSlot"]
