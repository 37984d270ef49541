"""Binding of checkpoint tensors to a model's parts by tensor name.

A model declares what it expects as a list of TensorSpec (name, shape, role).
`load_folder` reads every ``*.safetensors`` file of the folder (sorted, a name
may appear once: runtime/checkpoint.py:18-19,36 in the reference), checks the
whole set at once and raises ONE error that lists missing tensors, unexpected
tensors and wrong shapes.  Nothing is renamed.

A tensor that the model does not declare is no fault by itself: the reference
checks the expected names and shapes only (runtime/checkpoint.py:44-58), and
checkpoints carry buffers such as ``...rotary_emb.inv_freq``.  Such a folder
loads, with one line on stderr that names the extras; they are listed in the
error when something else is wrong (a misspelt name shows as one missing and
one unexpected tensor), and ``strict=True`` makes them an error of their own.

Dtype rule.  ``dtype=bfloat16``: bfloat16 tensors stay bfloat16, a tensor that
the file stores in 32 bits stays in 32 bits, float16 is widened to float32
first, integer tables become int32.  ``dtype=float32``: every floating tensor
is widened to float32 (exact).  What a kernel then needs (a bf16 matrix operand,
a float norm weight) is the business of the part that owns the tensor.
"""
import sys
from dataclasses import dataclass
from pathlib import Path
from typing import Tuple

import torch

from .safetensors_io import SafetensorsFile, SafetensorsError


class WeightError(ValueError):
    pass


@dataclass(frozen=True)
class TensorSpec:
    name: str
    shape: Tuple[int, ...]
    init: str = "normal"        # "normal": N(0, std); "one_plus_normal": 1 + N(0, std)  (random-weights mode)
    integer: bool = False       # an integer table (kept as int32)


def open_folder(folder):
    folder = Path(folder)
    files = sorted(folder.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no safetensors file in {folder}")
    index = {}
    for path in files:
        try:
            f = SafetensorsFile(path)
        except SafetensorsError as exc:
            raise WeightError(str(exc)) from exc
        for name in f.names():
            if name in index:
                raise WeightError(f"tensor {name} appears in {index[name].path.name} and {path.name}")
            index[name] = f
    return index


def check_against(specs, index, ignored=(), strict=False):
    """Raise one WeightError naming every missing, unexpected and mis-shaped tensor, if a tensor is
    missing or mis-shaped (or, with `strict`, unexpected).  Returns the unexpected names otherwise.
    `ignored` names tensors a checkpoint may carry without the model using them."""
    expected = {s.name: s for s in specs}
    missing = sorted(n for n in expected if n not in index)
    unexpected = sorted(n for n in index if n not in expected and n not in ignored)
    wrong = []
    for name, spec in expected.items():
        if name in index:
            _, shape = index[name].info(name)
            if tuple(shape) != tuple(spec.shape):
                wrong.append(f"{name}: file has {list(shape)}, model expects {list(spec.shape)}")
    if missing or wrong or (strict and unexpected):
        lines = ["checkpoint does not match the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shape ({len(wrong)}): " + "; ".join(sorted(wrong)))
        raise WeightError("\n".join(lines))
    return unexpected


def _kept_dtype(stored, integer, dtype):
    if integer or not stored.is_floating_point:
        return torch.int32
    if dtype == torch.float32:
        return torch.float32
    if stored == torch.bfloat16:
        return torch.bfloat16
    return torch.float32  # stored in 32 bits (or float16/float64): kept in 32 bits


def load_folder(folder, specs, dtype, device, ignored=(), strict=False):
    """{name: tensor on `device`} for every spec, after the whole-set check."""
    index = open_folder(folder)
    extras = check_against(specs, index, ignored, strict)
    if extras:
        shown = ", ".join(extras[:8]) + (f", ... ({len(extras)} in all)" if len(extras) > 8 else "")
        print(f"[runtime.weights] {folder}: tensors that the model does not use are left alone: {shown}", file=sys.stderr)
    out = {}
    for spec in specs:
        t = index[spec.name].tensor(spec.name)
        out[spec.name] = t.to(_kept_dtype(t.dtype, spec.integer, dtype)).to(device).contiguous()
    return out
