"""Random weights: a model folder (config.json, model.safetensors) from a config and a seed.

The reference has this only in its tests (tests/tiny_model.py:21-50:
`torch.manual_seed(seed)`, every matrix randn * 0.02, zero biases, unit norm
weights).  Here biases are drawn as well, so that the bias path carries signal,
and norm weights may be spread about one.  Values are drawn in float32 and stored
as bfloat16, the precision checkpoints of this family ship in, so that the
32-bit and the bfloat16 paths start from the same numbers.

Every tensor has a generator of its own, seeded from (seed, name): any tensor
can be produced alone, on the CPU or on the device that will hold it (the two
devices' generators give different numbers for one seed; a folder is always drawn
on the CPU).  `RandomWeights` is the mode for models too large to write out: a
read-only mapping that draws each tensor on the device at the moment a part asks
for it and keeps none, so that 145 GB of weights never exist twice.
"""

from __future__ import annotations

import json
import os
import zlib
from typing import Dict, Iterator, Mapping, Tuple

import torch

from .safetensors_io import save_file


def _tensor_seed(seed: int, name: str) -> int:
    return (int(seed) * 1000003 + zlib.crc32(name.encode("utf-8"))) & 0x7FFFFFFFFFFFFFFF


def std_of(name: str, std) -> float:
    """`std` is one number for every tensor, or a mapping from name endings to numbers with the
    fallback under "" (so that, say, query and key projections can be drawn wider than the rest
    and attention is peaked instead of flat)."""
    if not isinstance(std, Mapping):
        return float(std)
    for ending, value in std.items():
        if ending and name.endswith(ending):
            return float(value)
    return float(std.get("", 0.02))


def random_tensor(name: str, shape: Tuple[int, ...], seed: int, std=0.02,
                  norm_std: float = 0.0, device: str = "cpu",
                  dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """`shape` is what the part declared: a plain tuple is drawn about zero with `std`; a shape with
    a `centre` (a tensor that scales activations, see `parts.ScaleShape`) about that centre with
    `norm_std`.  Nothing is read from the tensor's name but its seed and, if `std` is a mapping, its std."""
    gen = torch.Generator(device=device).manual_seed(_tensor_seed(seed, name))
    std = std_of(name, std)
    centre = float(getattr(shape, "centre", 0.0))
    shape = tuple(shape)
    if centre:
        t = torch.full(shape, centre, device=device)
        if norm_std:
            t += norm_std * torch.randn(shape, generator=gen, device=device)
    else:
        t = torch.randn(shape, generator=gen, device=device)
        t *= std
    return t.to(dtype)


def random_weights(expected: Mapping[str, Tuple[int, ...]], seed: int, std=0.02,
                   norm_std: float = 0.0, device: str = "cpu",
                   dtype: torch.dtype = torch.bfloat16) -> Dict[str, torch.Tensor]:
    return {name: random_tensor(name, shape, seed, std, norm_std, device, dtype)
            for name, shape in expected.items()}


class RandomWeights(Mapping):
    """name -> tensor, drawn anew at every lookup on `device` from (seed, name); nothing is kept.
    Two lookups of one name give equal tensors, so the same mapping can feed a model and, in a
    test, the plain implementation it is compared with."""

    def __init__(self, expected: Mapping[str, Tuple[int, ...]], seed: int, std=0.02,
                 norm_std: float = 0.0, device: str = "cuda:0", dtype: torch.dtype = torch.bfloat16) -> None:
        self.shapes = dict(expected)  # as declared: a shape may say how its tensor is drawn
        self.seed, self.std, self.norm_std, self.device, self.dtype = seed, std, norm_std, device, dtype

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self.shapes:
            raise KeyError(name)
        return random_tensor(name, self.shapes[name], self.seed, self.std, self.norm_std, self.device, self.dtype)

    def __iter__(self) -> Iterator[str]:
        return iter(self.shapes)

    def __len__(self) -> int:
        return len(self.shapes)


def write_model_folder(config, seed: int, out_dir: str, std=0.02, norm_std: float = 0.0,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write `config.json` and `model.safetensors` for the typed `config` (any
    registered architecture's config object) with random weights."""
    from ..engine.model import expected_tensors  # late: parts register on import

    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(config.to_json_dict(), handle, indent=2)
    tensors = random_weights(expected_tensors(config.plan()), seed, std, norm_std, "cpu", dtype)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"),
              {"format": "pt", "seed": str(seed), "std": str(std), "norm_std": str(norm_std)})
    return out_dir
