"""Binding weights to a model by tensor name.

A model declares every tensor it wants (:class:`ParamDecl`: shape and role) under the name
the checkpoint uses; :func:`load_declared` compares that list with what a source holds and
raises ONE error that lists all missing tensors, all unexpected ones and all wrong shapes.
The reference prints a message and carries on with a null pointer when a tensor is missing
(include/safetensores.h:39-42) and refuses every dtype but bf16 (src/safetensors.cc:66-71).

Kept as stored: bfloat16 stays bfloat16 and a tensor stored in 32-bit stays 32-bit; float16
and float64 become float32; integer tables become int32.  Small vectors that kernels read as
float32 (norm weights) are widened to float32, which changes no value.  No matrix is ever
rounded at load; what keeping a wide matrix costs in a bfloat16 engine (its products do not
run on the matrix cores) is said once per class of tensor (:func:`precision_notices`).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Optional, Tuple

import torch

from .safetensors_io import SafetensorsFile


class WeightsError(ValueError):
    """Raised once per load, with everything that is wrong."""

    def __init__(self, where: str, missing: List[str], unexpected: List[str],
                 wrong_shape: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]],
                 wrong_dtype: List[Tuple[str, str]] = ()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = [f"weights in {where} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n}: file has {list(have)}, model wants {list(want)}"
                for n, have, want in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong dtype ({len(self.wrong_dtype)}): " + ", ".join(
                f"{n}: {why}" for n, why in self.wrong_dtype))
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class ParamDecl:
    """A tensor the model wants.

    role: "matrix" (a projection or table, kept as stored), "vector" (read as float32 by
    kernels), "int" (an integer table, kept as int32).
    init: how the random-weights mode fills it: "normal" N(0, std), "ones_plus_normal"
    1 + N(0, std) (norm weights), "zeros", "ones".
    """

    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"


class WeightSource:
    """Where tensors come from: ``names``, ``shape_dtype(name)`` and ``get(name)`` (CPU or device)."""

    where = "<memory>"

    def names(self) -> List[str]:
        raise NotImplementedError

    def shape_dtype(self, name: str) -> Tuple[Tuple[int, ...], torch.dtype]:
        raise NotImplementedError

    def get(self, name: str) -> torch.Tensor:
        raise NotImplementedError

    def close(self) -> None:
        pass


class FolderSource(WeightSource):
    """The weights of a model folder: ``model.safetensors`` (src/qwen.cc:69: a single file of
    that name), or, for checkpoints that are cut into shards, the files that
    ``model.safetensors.index.json`` names under ``weight_map``."""

    def __init__(self, folder: str):
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, "model.safetensors.index.json")
        self._files: Dict[str, SafetensorsFile] = {}
        self._where_is: Dict[str, str] = {}
        if os.path.isfile(single) or not os.path.isfile(index):
            self.where = single
            self._files[single] = SafetensorsFile(single)      # raises if there is none
            for name in self._files[single].names():
                self._where_is[name] = single
            return
        self.where = index
        with open(index, "r", encoding="utf-8") as fh:
            try:
                weight_map = json.load(fh)["weight_map"]
            except (json.JSONDecodeError, KeyError, TypeError) as exc:
                raise WeightsError(index, [], [], [], [("weight_map", f"unreadable index ({exc})")]) from exc
        for name, shard in weight_map.items():
            path = os.path.join(folder, shard)
            if path not in self._files:
                self._files[path] = SafetensorsFile(path)
            if name not in self._files[path].entries:
                raise WeightsError(index, [name], [], [])
            self._where_is[name] = path

    def names(self) -> List[str]:
        return list(self._where_is)

    def shape_dtype(self, name):
        e = self._files[self._where_is[name]].entries[name]
        return e.shape, e.dtype

    def get(self, name: str) -> torch.Tensor:
        return self._files[self._where_is[name]].get(name)

    def close(self) -> None:
        for f in self._files.values():
            f.close()


class DictSource(WeightSource):
    def __init__(self, tensors: Mapping[str, torch.Tensor], where: str = "<memory>"):
        self._tensors = dict(tensors)
        self.where = where

    def names(self) -> List[str]:
        return list(self._tensors)

    def shape_dtype(self, name):
        t = self._tensors[name]
        return tuple(t.shape), t.dtype

    def get(self, name: str) -> torch.Tensor:
        return self._tensors[name]


def kept_dtype(stored: torch.dtype, role: str) -> Optional[torch.dtype]:
    """The dtype a stored tensor has in device memory, or None if it cannot be used."""
    if role == "int":
        return torch.int32 if stored in (torch.int64, torch.int32, torch.int16, torch.int8,
                                         torch.uint8) else None
    if not stored.is_floating_point:
        return None
    if role == "vector":
        return torch.float32
    if stored == torch.bfloat16:
        return torch.bfloat16
    return torch.float32


def precision_notices(stored: Mapping[str, torch.dtype], declared: Mapping[str, ParamDecl],
                      engine_dtype: torch.dtype) -> List[str]:
    """What the kept dtypes mean for speed, one line per class of tensor: in a bfloat16 engine
    a matrix that is stored wider than bfloat16 stays float32, and every product with it takes
    the general kernel instead of the matrix cores."""
    if engine_dtype != torch.bfloat16:
        return []
    classes: Dict[torch.dtype, List[str]] = {}
    for name, dtype in stored.items():
        decl = declared.get(name)
        if decl is not None and decl.role == "matrix" and kept_dtype(dtype, "matrix") == torch.float32:
            classes.setdefault(dtype, []).append(name)
    return [f"{len(names)} matrices stored as {str(dtype).replace('torch.', '')} stay float32 (for one, {names[0]}): "
            "in a bfloat16 engine their products run on the general kernel, without the matrix cores, "
            "correct and many times slower; store them as bfloat16 to have the fast kernels"
            for dtype, names in classes.items()]


def load_declared(source: WeightSource, declared: Mapping[str, ParamDecl],
                  device: torch.device, optional: Iterable[str] = (),
                  stored_dtypes: Optional[Dict[str, torch.dtype]] = None) -> Dict[str, torch.Tensor]:
    """Check ``source`` against ``declared`` and bring every declared tensor to ``device``.

    ``optional`` names may be present in the source without being declared (a tied model's
    checkpoint may still carry ``lm_head.weight``); they are not loaded.  ``stored_dtypes``: a
    dict that is filled with the dtype every loaded tensor has in the source.
    """
    have = set(source.names())
    optional = set(optional)
    missing = [n for n in declared if n not in have]
    unexpected = sorted(n for n in have if n not in declared and n not in optional)
    wrong_shape, wrong_dtype = [], []
    for name, decl in declared.items():
        if name not in have:
            continue
        shape, dtype = source.shape_dtype(name)
        if tuple(shape) != tuple(decl.shape):
            wrong_shape.append((name, tuple(shape), tuple(decl.shape)))
        if kept_dtype(dtype, decl.role) is None:
            wrong_dtype.append((name, f"stored as {dtype}, which a {decl.role} cannot be"))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightsError(source.where, missing, unexpected, wrong_shape, wrong_dtype)

    out: Dict[str, torch.Tensor] = {}
    for name, decl in declared.items():
        t = source.get(name)
        if stored_dtypes is not None:
            stored_dtypes[name] = t.dtype
        target = kept_dtype(t.dtype, decl.role)
        # one copy: to the device first (as stored), then widen there if needed
        t = t.to(device=device, non_blocking=False)
        if t.dtype != target:
            t = t.to(target)
        out[name] = t.contiguous()
    return out
