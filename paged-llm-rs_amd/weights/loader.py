"""Weights by tensor name, checked against what the model declares.

The model's parts declare every tensor they need (name, shape, role).  The
file is checked against that list before anything is copied, and every problem
(tensors the model needs and the file lacks, tensors the file holds and the
model does not know, tensors at the wrong shape) is reported in one error
(reference: weights.rs:51-66, tests/forward.rs:81-92 for the per-tensor form).

Files.  ``model.safetensors`` when the folder has it (the reference reads only
that, weights.rs:24-32); otherwise ``model.safetensors.index.json``, whose
``weight_map`` names the shard that holds each tensor.  Shards stand behind the
same by-name interface, so the one report covers the whole checkpoint.

Dtype rule.  In ``float32`` every floating tensor is widened to 32-bit.  In
``bfloat16`` tensors stored in 16 bits are kept (float16 is converted),
matrices stored in 32 bits are rounded to bfloat16 as the reference's
``cast_to`` does (weights.rs:34-44), and vectors stored in 32 bits (norm gains)
stay 32-bit.  Integer tensors become int32.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from fnmatch import fnmatchcase
from pathlib import Path

import torch

from ..errors import IoError, WeightError
from .safetensors_io import SafetensorsFile


@dataclass(frozen=True)
class ParamDecl:
    """One tensor a part needs.  ``role`` is ``matrix``, ``embedding``, ``gain`` or
    ``bias``; it picks the random initialisation and nothing else."""
    name: str
    shape: tuple
    role: str = "matrix"
    optional: bool = False


def check_declared(decls, shapes: dict, where: str, ignored=()) -> None:
    """Raise one WeightError listing every missing, unexpected and mis-shaped tensor.  ``ignored``:
    shell patterns of tensor names that a checkpoint may carry without the model using them."""
    declared = {d.name: d for d in decls}
    missing = [d.name for d in decls if not d.optional and d.name not in shapes]
    unexpected = [n for n in shapes if n not in declared and not any(fnmatchcase(n, p) for p in ignored)]
    wrong = [
        f"{n} has shape {list(shapes[n])}, expected {list(d.shape)}"
        for n, d in declared.items() if n in shapes and tuple(shapes[n]) != tuple(d.shape)
    ]
    if not (missing or unexpected or wrong):
        return
    lines = [f"{where} does not fit the model:"]
    if missing:
        lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong:
        lines.append(f"  wrong shape ({len(wrong)}): " + "; ".join(wrong))
    raise WeightError("\n".join(lines))


def stored_dtype_to_resident(stored: torch.dtype, ndim: int, compute: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if compute == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32 if ndim <= 1 else compute
    return compute


INDEX_NAME = "model.safetensors.index.json"


class CheckpointFiles:
    """The tensors of a model folder by name, whether they lie in one file or in shards."""

    def __init__(self, model_dir):
        model_dir = Path(model_dir)
        single, index = model_dir / "model.safetensors", model_dir / INDEX_NAME
        self.files: dict = {}
        self.where: dict = {}
        if single.exists() or not index.exists():
            self.label = str(single)
            self._open(single)                      # (a folder with neither: the error names model.safetensors)
            self.where = {name: single for name in self.files[single].names()}
            return
        self.label = str(index)
        try:
            listed = json.loads(index.read_text())
        except OSError as e:
            raise IoError(f"reading {index}: {e}") from e
        except json.JSONDecodeError as e:
            raise WeightError(f"{index} is not JSON: {e}") from e
        weight_map = listed.get("weight_map") if isinstance(listed, dict) else None
        if not isinstance(weight_map, dict) or not weight_map:
            raise WeightError(f"{index} has no weight_map")
        absent = []
        for name, shard in weight_map.items():
            path = model_dir / str(shard)
            if path not in self.files:
                self._open(path)
            if name in self.files[path].entries:
                self.where[name] = path
            else:
                absent.append(f"{name} (not in {shard})")
        if absent:
            raise WeightError(f"{index} lists tensors that their shards do not hold: " + ", ".join(absent))

    def _open(self, path) -> None:
        self.files[path] = SafetensorsFile(path)    # IoError naming the file when it cannot be read

    def shapes(self) -> dict:
        return {name: self.files[path].shape(name) for name, path in self.where.items()}

    def names(self) -> list:
        return list(self.where)

    def dtype(self, name) -> torch.dtype:
        return self.files[self.where[name]].dtype(name)

    def __contains__(self, name) -> bool:
        return name in self.where

    def tensor(self, name) -> torch.Tensor:
        return self.files[self.where[name]].tensor(name)

    def close(self) -> None:
        for f in self.files.values():
            f.close()


def load_weights(model_dir, decls, compute_dtype: torch.dtype, device, ignored=()) -> dict:
    """All declared tensors of the checkpoint in ``model_dir`` on ``device``."""
    files = CheckpointFiles(model_dir)
    check_declared(decls, files.shapes(), files.label, ignored)
    out = {}
    for d in decls:
        if d.name not in files:
            continue
        t = files.tensor(d.name)
        resident = stored_dtype_to_resident(t.dtype, t.dim(), compute_dtype)
        # copy to the device in the stored width, convert there: one pass over the mapped bytes
        out[d.name] = t.to(device).to(resident).contiguous() if t.dtype != resident \
            else t.to(device, copy=True).contiguous()
    files.close()
    return out
