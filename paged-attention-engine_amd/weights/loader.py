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
        try:
            with open(index_path, "r", encoding="utf-8") as handle:
                weight_map = json.load(handle)["weight_map"]
        except (json.JSONDecodeError, KeyError, TypeError) as err:
            raise WeightsError(f"{index_path}: not a shard index with a 'weight_map' ({err})") from err
        absent = []  # names the index sends to a shard that does not hold them
        for name, shard in weight_map.items():
            if shard not in files:
                # the index is as little to be trusted as the checkpoint: a shard is a file of this folder
                if not isinstance(shard, str) or not shard or os.path.basename(shard) != shard or shard in (".", ".."):
                    raise WeightsError(f"{index_path}: the entry '{name}' names the shard {shard!r}, "
                                       "which is not a plain file name inside the model folder")
                shard_path = os.path.join(model_dir, shard)
                if not os.path.exists(shard_path):
                    raise WeightsError(f"{index_path} names the shard {shard}, which is not in the folder")
                files[shard] = SafetensorsFile(shard_path)
            if name in files[shard].entries:
                by_name[name] = files[shard]
            else:
                absent.append(f"{name} (not in {shard})")
        if absent:
            raise WeightsError(f"{index_path}: the index names tensors that their shards lack: "
                               + ", ".join(sorted(absent)), missing=[a.split(" ")[0] for a in absent])
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


class FolderWeights(Mapping):
    """name -> tensor of a checked folder.  A lookup returns a view of the memory-mapped file (a
    converting copy only for precisions that are not kept), so a part that sends it to the device
    copies straight from the file's pages: no second copy of the model ever sits in host memory.
    The views are private to this process (copy-on-write); the files stay open while the mapping
    lives."""

    def __init__(self, by_name: Mapping[str, SafetensorsFile], names) -> None:
        self._by_name = {name: by_name[name] for name in names}

    def __getitem__(self, name: str) -> torch.Tensor:
        return _keep_precision(self._by_name[name].tensor(name))

    def __iter__(self):
        return iter(self._by_name)

    def __len__(self) -> int:
        return len(self._by_name)


def load_weights(model_dir: str, expected: Mapping[str, Tuple[int, ...]],
                 optional: Sequence[str] = (), device: Optional[str] = None) -> Mapping[str, torch.Tensor]:
    """Tensors named in `expected`, each with exactly the declared shape.

    `optional` names may be present in the folder without being expected (a tied
    head that a file stores anyway); they are ignored.  Anything else that the
    folder holds and the model does not declare is reported as unexpected.
    Without `device` the result is a `FolderWeights` over the mapped files; with
    one, a dict of tensors on that device."""
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
    weights = FolderWeights(by_name, expected)
    if device is None:
        return weights
    return {name: weights[name].to(device) for name in expected}
