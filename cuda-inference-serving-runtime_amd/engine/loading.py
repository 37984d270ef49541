"""From a model folder to a model on the GPU, and the random-weights mode.

The architecture is chosen by config.json through the registry; weights are
bound by tensor name (reference: runtime/checkpoint.py:9-41 for loading,
runtime/model.py:38-55 for seeded random weights)."""
import torch

from ..config import architecture_of, read_config_json, preset
from ..weights import load_folder, write_model_folder

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def parse_dtype(dtype):
    if isinstance(dtype, torch.dtype):
        if dtype not in DTYPES.values():
            raise ValueError(f"dtype {dtype} is not float32 or bfloat16")
        return dtype
    try:
        return DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype {dtype!r} is not one of {sorted(DTYPES)}") from None


def import_plugins(names):
    """Import the modules `names`: a module that registers parts or an architecture of its own at import
    (runtime.register_part, runtime.register_architecture) thereby makes them known to the entry points, which choose
    the model class by config.json.  The modules come from the caller's command line, never from a model folder."""
    import importlib
    for name in names or ():
        importlib.import_module(name)


def build_from_config_dict(raw):
    arch = architecture_of(raw)
    config = arch.config_cls.from_dict(raw)
    return arch, config, arch.build(config)


def load_model(folder, dtype="bfloat16", device="cuda:0", strict=False):
    """The model of `folder` with its weights on `device`, ready to step.  Tensors that the model does not
    declare are left alone unless `strict`."""
    dtype = parse_dtype(dtype)
    raw = read_config_json(folder)
    _, _, model = build_from_config_dict(raw)
    tensors = load_folder(folder, model.tensor_specs(), dtype, torch.device(device), ignored=model.ignored_tensors(),
                          strict=strict)
    model.bind(tensors, dtype, torch.device(device))
    return model


def write_random_model(folder, config, seed, dtype="bfloat16", std=None):
    """Write config.json and model.safetensors for `config` (a config.json dict or
    the name of a preset) with seeded random weights: N(0, std), norms 1 + N(0, std); std 0.02 unless given."""
    raw = preset(config) if isinstance(config, str) else dict(config)
    _, typed, model = build_from_config_dict(raw)
    return write_model_folder(folder, typed.to_dict() if hasattr(typed, "to_dict") else raw,
                              model.tensor_specs(), seed, parse_dtype(dtype), **({} if std is None else {"std": std}))


def random_model(config, seed=0, dtype="bfloat16", device="cuda:0", std=0.02):
    """The model of `config` (a config.json dict or the name of a preset) with random weights drawn on the device:
    matrices N(0, std), norm weights 1 + N(0, std), bound through the model's own declarations, without a folder.
    For measurements at sizes whose files would take minutes to write; the draws are not those of
    write_random_model (another generator), so results are not comparable token by token."""
    dtype = parse_dtype(dtype)
    raw = preset(config) if isinstance(config, str) else dict(config)
    _, _, model = build_from_config_dict(raw)
    generator = torch.Generator(device=device).manual_seed(seed)
    tensors = {}
    for spec in sorted(model.tensor_specs(), key=lambda s: s.name):
        if spec.integer:
            raise ValueError(f"{spec.name}: integer tables have no random initialisation")
        values = torch.randn(spec.shape, generator=generator, device=device, dtype=torch.float32) * std
        if spec.init == "one_plus_normal":
            values += 1.0
        tensors[spec.name] = values.to(torch.bfloat16 if dtype == torch.bfloat16 else torch.float32)
    model.bind(tensors, dtype, torch.device(device))
    return model
