"""Binds a model's declared tensors to what a model folder holds, by name.

All problems of a folder are reported at once, in one error: tensors the model
declares and the file lacks, tensors the file has and the model does not know,
and tensors whose shape differs (expected against found).  The reference finds
missing weights only at the first inference, and then only the global ones
(internal/engine/engine.go:1316-1324); here nothing loads half-way.

Dtype rule: bfloat16 tensors stay bfloat16 (float16 becomes bfloat16), integer
tables become int32, a tensor stored in 32-bit stays so, norm weights are
always held in float32 (internal/engine/engine.go:788-792 does the same); in the
float32 mode every floating tensor is widened to float32.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Mapping, Sequence

import torch

from ..parts.base import MATRIX, TABLE, VECTOR32, TensorSpec
from .safetensors_io import SafetensorsFile, WeightFileError, open_model_files


class WeightError(ValueError):
    """Missing, unexpected or wrongly shaped tensors; `missing`, `unexpected` and
    `wrong_shape` hold the names."""

    def __init__(self, where: str, missing: Sequence[str], unexpected: Sequence[str],
                 wrong_shape: Sequence[str], other: Sequence[str] = ()) -> None:
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.other = list(other)
        lines = [f"weights in {where} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + "; ".join(self.wrong_shape))
        if self.other:
            lines.append(f"  other ({len(self.other)}): " + "; ".join(self.other))
        super().__init__("\n".join(lines))


def storage_dtype(spec: TensorSpec, stored: torch.dtype, run_dtype: torch.dtype) -> torch.dtype:
    if spec.kind == TABLE:
        return torch.int32
    if spec.kind == VECTOR32 or run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def check_names_and_shapes(specs: Sequence[TensorSpec], found: Mapping[str, tuple], where: str) -> None:
    """`found` maps name -> shape.  Raises WeightError unless everything fits."""
    declared = {s.name: s for s in specs}
    missing = [s.name for s in specs if s.name not in found and not s.optional]
    unexpected = [n for n in found if n not in declared]
    wrong = [
        f"{n}: expected {list(declared[n].shape)}, found {list(found[n])}"
        for n in found
        if n in declared and tuple(found[n]) != tuple(declared[n].shape)
    ]
    if missing or unexpected or wrong:
        raise WeightError(where, sorted(missing), sorted(unexpected), sorted(wrong))


def load_tensors(folder: str, specs: Sequence[TensorSpec], run_dtype: torch.dtype,
                 device: torch.device) -> Dict[str, torch.Tensor]:
    files = open_model_files(folder)
    try:
        where: Dict[str, SafetensorsFile] = {}
        dup: List[str] = []
        for f in files:
            for n in f.names():
                if n in where:
                    dup.append(f"{n}: in both {where[n].path} and {f.path}")
                where[n] = f
        if dup:
            raise WeightError(folder, [], [], [], dup)
        check_names_and_shapes(specs, {n: f.info(n)[1] for n, f in where.items()}, folder)
        bad = []
        for s in specs:
            if s.name in where:
                stored = where[s.name].info(s.name)[0]
                ok = stored in (torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8) if s.kind == TABLE \
                    else stored.is_floating_point
                if not ok:
                    bad.append(f"{s.name}: stored as {stored}, which a {s.kind} tensor cannot be")
        if bad:
            raise WeightError(folder, [], [], [], bad)
        out: Dict[str, torch.Tensor] = {}
        for s in specs:
            if s.name not in where:
                continue
            t = where[s.name].tensor(s.name)
            out[s.name] = t.to(storage_dtype(s, t.dtype, run_dtype)).to(device)
        return out
    finally:
        for f in files:
            f.close()
