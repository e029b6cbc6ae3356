"""From a model folder (or a configuration and a seed) to a loaded model."""
from __future__ import annotations

import json
import os

import torch

from ..models.registry import architecture_of, config_from_folder, resolve
from ..weights.random_init import RandomSource
from ..weights.safetensors_io import Checkpoint, LazyTensor, write_safetensors
from .model import Model

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
          "f32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"the engine computes in bfloat16 or float32, not {name}")
        return name
    if name not in DTYPES:
        raise ValueError(f"unknown dtype '{name}' (one of {', '.join(sorted(DTYPES))})")
    return DTYPES[name]


def load_model(folder: str, dtype="bfloat16", device="cuda:0") -> Model:
    """config.json chooses the model class; weights are bound by tensor name."""
    arch, cfg = config_from_folder(folder)
    ckpt = Checkpoint(folder)
    model = Model(arch.build_spec(cfg, ckpt.names()))
    model.config = cfg
    model.load(ckpt, parse_dtype(dtype), device, where=folder)
    return model


def random_model(config, seed: int, dtype="bfloat16", device="cuda:0", std: float = 0.02) -> Model:
    """A model with seeded random weights made on the device; no file is involved.
    `config` is a typed configuration or a raw config.json dict."""
    if isinstance(config, dict):
        arch = resolve(config)
        config = arch.config_class.from_dict(config)
    else:
        arch = architecture_of(config)
    act = parse_dtype(dtype)
    model = Model(arch.build_spec(config, None))
    model.config = config
    model.load(RandomSource(seed, act, device, std), act, device, where=f"(random, seed {seed})")
    return model


def write_random_model(config, folder: str, seed: int, dtype="bfloat16", std: float = 0.02, device="cpu") -> None:
    """Writes config.json and model.safetensors with the same tensors `random_model` makes.  `device`: where the
    values are worked out before they are written (the same numbers on the CPU and on the GPU up to the last bit
    of either's logarithm and cosine; a GPU makes a billion of them in seconds)."""
    if isinstance(config, dict):
        arch = resolve(config)
        config = arch.config_class.from_dict(config)
    else:
        arch = architecture_of(config)
    store = parse_dtype(dtype)
    os.makedirs(folder, exist_ok=True)
    model = Model(arch.build_spec(config, None))
    specs = model.named_params()
    src = RandomSource(seed, store, device, std)
    src.expect(specs)
    items = [(name, LazyTensor(torch.int32 if spec.integer else store, spec.shape,
                               lambda n=name: src.tensor(n))) for name, spec in specs.items()]
    write_safetensors(os.path.join(folder, "model.safetensors"), items, {"format": "pt", "seed": seed})
    with open(os.path.join(folder, "config.json"), "w") as f:
        cfg = config.to_dict()
        cfg["torch_dtype"] = "bfloat16" if store == torch.bfloat16 else "float32"
        json.dump(cfg, f, indent=2)
