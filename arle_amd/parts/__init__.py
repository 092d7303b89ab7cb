from .base import Part, Runtime, build_part, expected_tensors, lookup, register
from .spec import LayerSpec, ModelSpec, PartSpec, Rows, ScheduleEntry, WeightDecl

__all__ = ["Part", "Runtime", "build_part", "expected_tensors", "lookup", "register", "LayerSpec",
           "ModelSpec", "PartSpec", "Rows", "ScheduleEntry", "WeightDecl"]
