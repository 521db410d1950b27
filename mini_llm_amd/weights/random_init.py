"""Random-weights mode: draws every tensor a model's parts declare, from a seed, and writes a
model folder (config.json, model.safetensors) that the loader reads like any other."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from .counter_rng import normal_tensor
from .safetensors_io import write_safetensors
from .spec import INT_TABLE


def random_tensors(model, seed: int, dtype: torch.dtype = torch.float32) -> dict:
    """name -> CPU tensor in the stored layout. Every element is a function of (seed, the tensor's
    name, its index in the tensor) alone (``counter_rng``): the same seed gives the same model
    whatever the order of the tensors, the installed libraries or the language of whoever draws it."""
    out = {}
    for name, spec in model.named_tensor_specs().items():
        if spec.role == INT_TABLE:
            raise ValueError(f"{name}: no random recipe for integer tables")
        values = normal_tensor(int(seed), name, tuple(spec.shape), spec.init.mean, spec.init.std)
        out[name] = torch.from_numpy(values).to(dtype)
    return out


def write_model_dir(config, seed: int, out_dir, dtype="float32") -> Path:
    """Writes config.json and model.safetensors of a randomly initialised model of this
    configuration; ``dtype`` is the element type stored in the file."""
    from ..config import get_architecture
    from ..precision import Precision

    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    stored = Precision.from_name(dtype).compute
    model = get_architecture(config.architecture).build(config, Precision.from_name("float32"))
    tensors = random_tensors(model, seed, stored)
    (out_dir / "config.json").write_text(json.dumps(config.to_dict(), indent=2) + "\n")
    write_safetensors(out_dir / "model.safetensors", tensors, metadata={"format": "pt", "seed": seed})
    return out_dir
