"""Weights by tensor name, checked against what the model declares.

The model's parts declare every tensor they need (name, shape, role).  The
file is checked against that list before anything is copied, and every problem
(tensors the model needs and the file lacks, tensors the file holds and the
model does not know, tensors at the wrong shape) is reported in one error
(reference: weights.rs:51-66, tests/forward.rs:81-92 for the per-tensor form).

Dtype rule.  In ``float32`` every floating tensor is widened to 32-bit.  In
``bfloat16`` tensors stored in 16 bits are kept (float16 is converted),
matrices stored in 32 bits are rounded to bfloat16 as the reference's
``cast_to`` does (weights.rs:34-44), and vectors stored in 32 bits (norm gains)
stay 32-bit.  Integer tensors become int32.
"""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path

import torch

from ..errors import WeightError
from .safetensors_io import SafetensorsFile


@dataclass(frozen=True)
class ParamDecl:
    """One tensor a part needs.  ``role`` is ``matrix``, ``embedding``, ``gain`` or
    ``bias``; it picks the random initialisation and nothing else."""
    name: str
    shape: tuple
    role: str = "matrix"
    optional: bool = False


def check_declared(decls, shapes: dict, where: str) -> None:
    """Raise one WeightError listing every missing, unexpected and mis-shaped tensor."""
    declared = {d.name: d for d in decls}
    missing = [d.name for d in decls if not d.optional and d.name not in shapes]
    unexpected = [n for n in shapes if n not in declared]
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


def load_weights(model_dir, decls, compute_dtype: torch.dtype, device) -> dict:
    """All declared tensors of ``model_dir/model.safetensors`` on ``device``."""
    path = Path(model_dir) / "model.safetensors"
    file = SafetensorsFile(path)
    check_declared(decls, {n: file.shape(n) for n in file.names()}, str(path))
    out = {}
    for d in decls:
        if d.name not in file.entries:
            continue
        t = file.tensor(d.name)
        resident = stored_dtype_to_resident(t.dtype, t.dim(), compute_dtype)
        # copy to the device in the stored width, convert there: one pass over the mapped bytes
        out[d.name] = t.to(device).to(resident).contiguous() if t.dtype != resident \
            else t.to(device, copy=True).contiguous()
    file.close()
    return out
