"""Random weights from a configuration and a seed.

The reference has no such mode (it only reads a checkpoint, src/qwen.cc:69-84).  Projections
and tables are N(0, std); norm weights are 1 + N(0, std) so that a norm applied in the wrong
place or left out changes the result.

Every value is a function of (seed, tensor name, element index) alone: it does not depend on
the order in which tensors are made, on the device that makes them, or on torch's generators,
and anyone can compute it again with integer arithmetic:

    key   = mix(seed mod 2^64  xor  first 8 bytes, little-endian, of sha256(tensor name))
    h_j   = mix(key + (3 * index + j + 1) * GOLDEN)          for j = 0, 1, 2    (mod 2^64)
    s     = sum of the twelve 16-bit fields of h_0, h_1, h_2
    z     = (s - 6 * 65535) / 65536                           (float32, exact)
    value = z * std  (+ 1 for norm weights)                   (float32, one rounding each)

``mix`` is the splitmix64 finaliser and GOLDEN its increment 0x9E3779B97F4A7C15.  ``z`` is the
classic sum of twelve uniform numbers less six: mean 0, variance 1 - 2^-32, tails cut at six
standard deviations.  Only integer operations and two IEEE float32 operations are involved,
so the CPU, the GPU and numpy give the same bits.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Iterator, Mapping, Tuple

import torch

from .loader import ParamDecl
from .safetensors_io import write_safetensors

_MASK64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
_M1, _M2 = 0xBF58476D1CE4E5B9, 0x94D049BB133111EB
_CHUNK = 1 << 24      # elements made at a time: bounds the int64 temporaries to a few 100 MB


def _signed(x: int) -> int:
    """The int64 with the bits of the unsigned 64-bit ``x``."""
    x &= _MASK64
    return x - (1 << 64) if x >> 63 else x


def _mix_int(x: int) -> int:
    x = (x + _GOLDEN) & _MASK64
    x = ((x ^ (x >> 30)) * _M1) & _MASK64
    x = ((x ^ (x >> 27)) * _M2) & _MASK64
    return x ^ (x >> 31)


def tensor_key(seed: int, name: str) -> int:
    """The 64-bit key of a tensor's stream."""
    digest = hashlib.sha256(name.encode("utf-8")).digest()
    return _mix_int((int(seed) & _MASK64) ^ int.from_bytes(digest[:8], "little"))


def _mix_tensor(x: torch.Tensor) -> torch.Tensor:
    """splitmix64's finaliser on int64 tensors: products wrap, and a logical shift right is an
    arithmetic one with the sign's copies masked away."""
    x = x + _signed(_GOLDEN)
    x = (x ^ ((x >> 30) & ((1 << 34) - 1))) * _signed(_M1)
    x = (x ^ ((x >> 27) & ((1 << 37) - 1))) * _signed(_M2)
    return x ^ ((x >> 31) & ((1 << 33) - 1))


def unit_normal(key: int, first: int, count: int, device) -> torch.Tensor:
    """float32 [count]: the stream's values ``z`` at indices first .. first + count - 1."""
    index = torch.arange(first, first + count, dtype=torch.int64, device=device)
    total = torch.zeros(count, dtype=torch.int64, device=device)
    for j in range(3):
        h = _mix_tensor((index * 3 + (j + 1)) * _signed(_GOLDEN) + _signed(key))
        for shift in (0, 16, 32, 48):
            total += (h >> shift) & 0xFFFF
    return (total - 6 * 65535).to(torch.float32) * (1.0 / 65536.0)


def random_tensor(name: str, decl: ParamDecl, seed: int, std: float, dtype: torch.dtype,
                  device="cpu") -> torch.Tensor:
    dev = torch.device(device)
    if decl.role == "int":
        return torch.zeros(decl.shape, dtype=torch.int32, device=dev)
    if decl.init == "zeros":
        return torch.zeros(decl.shape, dtype=dtype, device=dev)
    if decl.init == "ones":
        return torch.ones(decl.shape, dtype=dtype, device=dev)
    if decl.init not in ("normal", "ones_plus_normal"):
        raise ValueError(f"tensor '{name}': unknown init '{decl.init}'")
    count = 1
    for n in decl.shape:
        count *= int(n)
    key = tensor_key(seed, name)
    out = torch.empty(count, dtype=dtype, device=dev)
    scale = torch.tensor(std, dtype=torch.float32, device=dev)
    for first in range(0, count, _CHUNK):
        n = min(_CHUNK, count - first)
        t = unit_normal(key, first, n, dev) * scale
        if decl.init == "ones_plus_normal":
            t = t + 1.0
        out[first:first + n] = t.to(dtype)
    return out.view(tuple(decl.shape))


def random_tensors(declared: Mapping[str, ParamDecl], seed: int, std: float,
                   dtype: torch.dtype = torch.bfloat16,
                   device: str = "cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    """Yield ``(name, tensor)`` for every declared tensor; values are made in float32 and
    rounded to ``dtype`` once.  The same on every device."""
    for name, decl in declared.items():
        yield name, random_tensor(name, decl, seed, std, dtype, device)


def write_model_folder(folder: str, config_dict: Dict[str, Any], seed: int,
                       dtype: torch.dtype = torch.bfloat16, std: float = None,
                       device: str = None) -> str:
    """Make ``folder`` a model folder: config.json and model.safetensors with random weights
    for the architecture that ``config_dict`` names.  ``device``: where the values are worked
    out (they are the same everywhere; a GPU makes a model of 8B size in seconds, a CPU in
    minutes); None: the GPU if there is one."""
    if device is None:
        device = "cuda:0" if torch.cuda.is_available() else "cpu"
    from ..config.registry import architecture_for
    from ..models.causal_lm import declared_tensors

    arch = architecture_for(config_dict)
    config = arch.read_config(config_dict)
    spec = arch.model_spec(config)
    declared = declared_tensors(spec)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(config_dict, fh, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      random_tensors(declared, seed, spec.init_std if std is None else std, dtype,
                                     device=device))
    return folder
