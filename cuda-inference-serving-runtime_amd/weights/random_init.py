"""Random-weights mode: writes a model folder (config.json, model.safetensors)
from a configuration and a seed.

Matrices are N(0, 0.02); norm weights are 1 + N(0, 0.02).  Tensors are drawn in
the order of their names with one generator, so a folder is a function of
(config, seed, stored dtype) only.  (The reference's own toy weights are
N(0,1)/sqrt(in) with norms of exactly 1, runtime/model.py:38-55; the recipe here
makes norms non-trivial so that a misplaced norm weight shows.)
"""
import json
from pathlib import Path

import numpy as np
import torch

from .safetensors_io import write_safetensors

STD = 0.02


def random_tensors(specs, seed, dtype=torch.bfloat16, std=STD):
    """`std`: the spread of the normal draws (0.02 unless a caller wants layers that outweigh the embedding)."""
    rng = np.random.default_rng(seed)
    out = {}
    for spec in sorted(specs, key=lambda s: s.name):
        if spec.integer:
            raise ValueError(f"{spec.name}: integer tables have no random initialisation")
        values = rng.standard_normal(size=spec.shape, dtype=np.float32) * np.float32(std)
        if spec.init == "one_plus_normal":
            values = values + np.float32(1.0)
        out[spec.name] = torch.from_numpy(values).to(dtype)
    return out


def write_model_folder(folder, config_dict, specs, seed, dtype=torch.bfloat16, std=STD):
    """config_dict is what goes into config.json; specs are the model's tensor specs."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    raw = dict(config_dict)
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype]
    (folder / "config.json").write_text(json.dumps(raw, indent=2) + "\n")
    write_safetensors(folder / "model.safetensors", random_tensors(specs, seed, dtype, std),
                      metadata={"format": "pt", "seed": seed})
    return folder
