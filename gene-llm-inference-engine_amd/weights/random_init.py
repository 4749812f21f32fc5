"""Random weights from a configuration and a seed, as tensors or as a model folder.

Distributions: matrices N(0, std) with std 0.02, scale vectors of norms 1 + 0.1 * N(0, 1) so
that a norm applied in the wrong place or with the wrong weight shows in the output (the
reference's test generator draws its norm weights the same way, tools/make_dummy_hf.py:99-106).
One torch CPU generator seeded with `seed` draws the tensors in the model's own order, each in
float32, then rounds to the storage dtype.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Iterable

import torch

from .loader import TensorNeed, merge_needs
from .safetensors_io import write_safetensors

_STORAGE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "bf16": torch.bfloat16, "fp32": torch.float32,
            torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def random_tensors(needs: Iterable[TensorNeed], seed: int, dtype="bfloat16", std: float = 0.02,
                   norm_dtype=None) -> Dict[str, torch.Tensor]:
    store = _STORAGE[dtype]
    norm_store = store if norm_dtype is None else _STORAGE[norm_dtype]
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    out = {}
    for name, need in merge_needs(needs).items():
        if need.role == "table":
            raise ValueError(f"tensor '{name}': integer tables have no random initialisation")
        t = torch.randn(need.shape, generator=gen, dtype=torch.float32)
        if need.role == "norm":
            out[name] = (1.0 + 0.1 * t).to(norm_store)
        else:
            out[name] = (std * t).to(store)
    return out


def write_random_model(folder, config, seed: int, dtype="bfloat16", std: float = 0.02, norm_dtype=None) -> Path:
    """Writes config.json and model.safetensors for `config` (any registered architecture's typed
    configuration: it needs `to_dict()` and `model_spec()`)."""
    from ..parts import model_tensor_needs
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    cfg = config.to_dict()
    cfg["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[_STORAGE[dtype]]
    (folder / "config.json").write_text(json.dumps(cfg, indent=2))
    tensors = random_tensors(model_tensor_needs(config.model_spec()), seed, dtype, std, norm_dtype)
    names = list(tensors)
    order = torch.randperm(len(names), generator=torch.Generator().manual_seed(int(seed) + 1)).tolist()
    write_safetensors(folder / "model.safetensors", {names[i]: tensors[names[i]] for i in order},
                      metadata={"format": "pt", "seed": seed})
    return folder
