"""Random weights from a configuration and a seed, as tensors or as a model folder.

Distributions: matrices N(0, std) with std 0.02, scale vectors of norms 1 + 0.1 * N(0, 1) so
that a norm applied in the wrong place or with the wrong weight shows in the output (the
reference's test generator draws its norm weights the same way, tools/make_dummy_hf.py:99-106).
One torch CPU generator seeded with `seed` draws the tensors in the model's own order, each in
float32, then rounds to the storage dtype.

Large models are drawn on the device instead (`formula_tensors`), by a formula of (seed, tensor
name, element index) that anybody can restate, so that such a model can be re-made elsewhere (the
tests' plain implementation does) without a file in between:
    key  = (fnv1a64(name) + (seed + 1) * 0x9E3779B97F4A7C15) mod 2^64
    r_i  = mix(key + (i + 1) * 0x9E3779B97F4A7C15)       mix: the splitmix64 finaliser, i the index in row-major order
    u1   = ((r_i >> 40) + 1) / 2^24,   u2 = ((r_i >> 8) & 0xFFFFFF) / 2^24
    z_i  = sqrt(-2 ln u1) * cos(2 pi u2)                  in 64-bit
    w_i  = std * z_i (matrices) or 1 + 0.1 * z_i (norm weights), rounded to 32-bit, then to the storage dtype
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


_MASK = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15


def tensor_key(name: str, seed: int) -> int:
    h = 0xCBF29CE484222325
    for b in name.encode("utf-8"):
        h = ((h ^ b) * 0x100000001B3) & _MASK
    return (h + (int(seed) + 1) * _GOLDEN) & _MASK


def formula_values(name: str, shape, seed: int, offset: float, scale: float) -> torch.Tensor:
    """The formula above on the host, float32 (the statement the device kernel is tested against; slow for large tensors)."""
    import numpy as np
    n = 1
    for d in shape:
        n *= int(d)
    z = (np.uint64(tensor_key(name, seed)) + (np.arange(1, n + 1, dtype=np.uint64) * np.uint64(_GOLDEN)))
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    r = z ^ (z >> np.uint64(31))
    u1 = ((r >> np.uint64(40)) + np.uint64(1)).astype(np.float64) / 16777216.0
    u2 = ((r >> np.uint64(8)) & np.uint64(0xFFFFFF)).astype(np.float64) / 16777216.0
    normal = np.sqrt(-2.0 * np.log(u1)) * np.cos(6.283185307179586476925 * u2)
    return torch.from_numpy((offset + scale * normal).astype(np.float32)).reshape(tuple(int(d) for d in shape))


def formula_tensors(needs: Iterable[TensorNeed], seed: int, dtype="bfloat16", std: float = 0.02, device="cuda:0") -> Dict[str, torch.Tensor]:
    """The model's tensors by the formula above, made on the device (seconds for billions of weights)."""
    from ..kernels import ops
    store = _STORAGE[dtype]
    out = {}
    for name, need in merge_needs(needs).items():
        if need.role == "table":
            raise ValueError(f"tensor '{name}': integer tables have no random initialisation")
        t = torch.empty(need.shape, dtype=store, device=device)
        offset, scale = (1.0, 0.1) if need.role == "norm" else (0.0, std)
        out[name] = ops.random_normal(t, tensor_key(name, seed), offset, scale)
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
