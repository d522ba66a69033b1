"""The random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.  The distributions are the family's (``Family.init``); the draws come
from torch's CPU generator, so a seed gives the same folder on every machine."""

import json
import os

import torch

from ..config.registry import resolve_family
from .safetensors_io import write_safetensors

STORE_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def random_tensors(config_json, seed):
    """(typed config, {checkpoint name: float32 CPU tensor}) for a config.json dictionary."""
    family = resolve_family(config_json)
    config = family.config_class.from_dict(config_json)
    generator = torch.Generator(device="cpu")
    generator.manual_seed(int(seed))
    return config, family.init(config, generator)


def write_random_model(model_dir, config_json, seed, store_dtype="bfloat16"):
    """Creates ``model_dir`` with config.json and model.safetensors; returns the stored tensors
    (rounded to ``store_dtype`` and widened back to float32, i.e. exactly what a load will see)."""
    if store_dtype not in STORE_DTYPES:
        raise ValueError(f"store_dtype must be one of {sorted(STORE_DTYPES)}, got {store_dtype!r}")
    config, tensors = random_tensors(config_json, seed)
    stored = {name: t.to(STORE_DTYPES[store_dtype]) for name, t in tensors.items()}
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as handle:
        json.dump(config.to_dict(), handle, indent=1)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), stored,
                      {"format": "pt", "seed": seed})
    return {name: t.to(torch.float32) for name, t in stored.items()}
