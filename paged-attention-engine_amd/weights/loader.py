"""Weights by tensor name from a model folder, checked against what the model declares.

The reference looks tensors up by their checkpoint names in a state dict and
fails with a bare KeyError on the first missing one, with no shape checks
(engine/model.py:198-227).  Here the model declares every name and shape it needs
first; the folder is compared with that declaration as a whole and one error
lists everything that is missing, unexpected or of the wrong shape.

Stored precision is kept: bfloat16 stays bfloat16 and a tensor stored in 32-bit
floating point stays so; float16/float64 become float32; integer tables become
int32.  Casting to what a kernel consumes is the binding part's business.
"""

from __future__ import annotations

import json
import os
from typing import Dict, Mapping, Optional, Sequence, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile

SINGLE_FILE = "model.safetensors"
INDEX_FILE = "model.safetensors.index.json"


class WeightsError(ValueError):
    """The folder's tensors do not match the model; the message lists every difference."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = tuple(missing)
        self.unexpected = tuple(unexpected)
        self.wrong_shape = tuple(wrong_shape)


def _open_shards(model_dir: str) -> Dict[str, SafetensorsFile]:
    """name -> the file that holds it, for a single file or a sharded index."""
    index_path = os.path.join(model_dir, INDEX_FILE)
    single = os.path.join(model_dir, SINGLE_FILE)
    files: Dict[str, SafetensorsFile] = {}
    by_name: Dict[str, SafetensorsFile] = {}
    if os.path.exists(index_path):
        with open(index_path, "r", encoding="utf-8") as handle:
            weight_map = json.load(handle)["weight_map"]
        for name, shard in weight_map.items():
            if shard not in files:
                files[shard] = SafetensorsFile(os.path.join(model_dir, shard))
            by_name[name] = files[shard]
    elif os.path.exists(single):
        shard = SafetensorsFile(single)
        for name in shard.names():
            by_name[name] = shard
    else:
        raise WeightsError(f"{model_dir}: neither {SINGLE_FILE} nor {INDEX_FILE} found")
    return by_name


def _keep_precision(t: torch.Tensor) -> torch.Tensor:
    if t.dtype in (torch.bfloat16, torch.float32, torch.int32):
        return t
    if t.is_floating_point():
        return t.to(torch.float32)
    return t.to(torch.int32)


def load_weights(model_dir: str, expected: Mapping[str, Tuple[int, ...]],
                 optional: Sequence[str] = (), device: Optional[str] = None) -> Dict[str, torch.Tensor]:
    """Tensors named in `expected`, each with exactly the declared shape.

    `optional` names may be present in the folder without being expected (a tied
    head that a file stores anyway); they are ignored.  Anything else that the
    folder holds and the model does not declare is reported as unexpected."""
    try:
        by_name = _open_shards(model_dir)
    except SafetensorsError as err:
        raise WeightsError(str(err)) from err
    missing = [n for n in expected if n not in by_name]
    unexpected = [n for n in by_name if n not in expected and n not in optional]
    wrong = [(n, by_name[n].shape(n), tuple(expected[n])) for n in expected
             if n in by_name and tuple(by_name[n].shape(n)) != tuple(expected[n])]
    if missing or unexpected or wrong:
        lines = [f"{model_dir}: weights do not match the model"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(sorted(missing)))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(sorted(unexpected)))
        if wrong:
            lines.append(f"  wrong shape ({len(wrong)}): " + "; ".join(
                f"{n} is {list(got)}, model needs {list(want)}" for n, got, want in sorted(wrong)))
        raise WeightsError("\n".join(lines), missing, unexpected, wrong)
    out = {}
    for name in expected:
        t = _keep_precision(by_name[name].tensor(name))
        out[name] = t.to(device) if device is not None else t.clone()
    return out
