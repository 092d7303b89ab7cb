"""Weights from a model folder, by tensor name, with one error that says everything wrong.

A folder holds `model.safetensors`, or `model.safetensors.index.json` whose `weight_map`
names the shard of every tensor (infer/src/weight_loader.rs:27-84,102-120).  The model's
spec says which tensors it needs and with which shapes; the loader compares that list with
what the files hold and raises a single `WeightsError` listing missing tensors, wrong shapes
and the tensors the model does not know.  Tensors the model does not know are not an error
by themselves: the reference reads by name and never looks at the rest (a tied checkpoint
that still stores lm_head.weight loads there: infer/src/model/qwen3/weights.rs:305-316), so
they are reported in a warning and left in the file; `strict=True` makes them fatal.

Element types: in the bfloat16 engine a tensor keeps the type it is stored in -- bfloat16
stays bfloat16, a tensor stored in 32 bits stays float32 (float16 is widened to float32),
integer tables become int32.  In the float32 engine every floating tensor is widened to
float32, which is exact for bfloat16 and float16.
"""
from __future__ import annotations

import json
import os
import warnings

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile

SINGLE_FILE = "model.safetensors"
INDEX_FILE = "model.safetensors.index.json"


class WeightsError(ValueError):
    """The checkpoint does not fit the model; `.missing`, `.unexpected`, `.wrong_shape` say how."""

    def __init__(self, message, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


class Checkpoint:
    """All shards of a model folder behind one name -> tensor lookup."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        single = os.path.join(model_dir, SINGLE_FILE)
        index = os.path.join(model_dir, INDEX_FILE)
        self._files: dict = {}
        self._where: dict = {}
        try:
            if os.path.exists(single):
                self._open(SINGLE_FILE)
            elif os.path.exists(index):
                with open(index, "r", encoding="utf-8") as fh:
                    weight_map = json.load(fh).get("weight_map")
                if not isinstance(weight_map, dict):
                    raise WeightsError("Invalid index.json: missing weight_map")
                for shard in sorted(set(weight_map.values())):
                    self._open(shard)
            else:
                raise WeightsError(f"no {SINGLE_FILE} or {INDEX_FILE} in {model_dir}")
        except SafetensorsError as exc:
            raise WeightsError(str(exc)) from exc

    def _open(self, fname: str) -> None:
        f = SafetensorsFile(os.path.join(self.model_dir, fname))
        self._files[fname] = f
        for name in f.names():
            self._where.setdefault(name, fname)

    def names(self) -> list:
        return list(self._where)

    def info(self, name: str):
        return self._files[self._where[name]].info(name)

    def read(self, name: str) -> torch.Tensor:
        return self._files[self._where[name]].read(name)

    def close(self) -> None:
        for f in self._files.values():
            f.close()


def _engine_dtype(stored: torch.dtype, act_dtype: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if act_dtype == torch.float32:
        return torch.float32
    return torch.bfloat16 if stored == torch.bfloat16 else torch.float32


class UnexpectedTensors(UserWarning):
    """The checkpoint holds tensors the model does not read; they are ignored."""


def compare_with_expected(found: dict, expected: dict, strict: bool = False) -> list:
    """found: name -> shape; expected: name -> WeightDecl.  Raises one WeightsError, or returns the
    names the model does not know (never fatal alone unless `strict`)."""
    missing = sorted(n for n in expected if n not in found)
    unexpected = sorted(n for n in found if n not in expected)
    wrong = sorted((n, tuple(expected[n].shape), tuple(found[n])) for n in expected
                   if n in found and tuple(found[n]) != tuple(expected[n].shape))
    if not (missing or wrong or (strict and unexpected)):
        return unexpected
    lines = ["checkpoint does not match the model:"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong:
        lines.append(f"  wrong shapes ({len(wrong)}): " + "; ".join(
            f"{n}: expected {list(e)}, found {list(f)}" for n, e, f in wrong))
    raise WeightsError("\n".join(lines), missing, unexpected, wrong)


def load_weights(model_dir: str, expected: dict, device, act_dtype: torch.dtype, strict: bool = False) -> dict:
    """name -> tensor on `device` for every expected tensor, or one WeightsError."""
    ckpt = Checkpoint(model_dir)
    try:
        ignored = compare_with_expected({n: ckpt.info(n)[1] for n in ckpt.names()}, expected, strict)
        if ignored:
            shown = ", ".join(ignored[:8]) + (f", ... ({len(ignored)} in all)" if len(ignored) > 8 else "")
            warnings.warn(f"{model_dir}: ignoring tensors the model does not read: {shown}", UnexpectedTensors,
                          stacklevel=2)
        out = {}
        for name in expected:
            t = ckpt.read(name)
            out[name] = t.to(device=device, dtype=_engine_dtype(t.dtype, act_dtype)).contiguous()
        return out
    finally:
        ckpt.close()
