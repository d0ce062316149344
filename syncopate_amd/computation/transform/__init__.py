"""The `@sy.*` annotations as a schedule-binding vocabulary for the HIP kernel templates."""

from .annotations import AnnotationError, AxisCount, DispatchBlock, ParsedAnnotations, parse_annotations
from .binder import AnnotationTransformer, KernelBinding, RemoteBinding, RemoteSlot

__all__ = [
    "AnnotationError",
    "AnnotationTransformer",
    "AxisCount",
    "DispatchBlock",
    "KernelBinding",
    "ParsedAnnotations",
    "RemoteBinding",
    "RemoteSlot",
    "parse_annotations",
]
