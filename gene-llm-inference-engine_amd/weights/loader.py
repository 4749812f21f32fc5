"""Weights from a model folder, bound by tensor name.

The model says which tensors it needs (`TensorNeed`: name, shape, role); this module finds
them in `model.safetensors`, checks all of them and reports every problem in one error, and
puts them on the device.  Precision rules: a bfloat16 tensor stays bfloat16 for bfloat16
compute and is widened exactly for float32 compute; a tensor stored in 32-bit stays 32-bit
in both; float16 is widened exactly to float32 (the reference does the same,
src/loader/hf_checkpoint.cpp:186-199); integer tables become int32.  No tensor is renamed,
split or fused here; the file's order does not matter.
"""
from __future__ import annotations

import re
from dataclasses import dataclass
from pathlib import Path
from typing import Dict, Iterable, Sequence, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightsError(ValueError):
    """The folder's tensors do not fit the model; the message lists every misfit."""


@dataclass(frozen=True)
class TensorNeed:
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"        # "matrix", "norm" (a scale vector around 1) or "table" (integers)


_FLOATS = ("F32", "F16", "BF16")
_INTS = ("I64", "I32", "I16", "I8", "U8")


def merge_needs(needs: Iterable[TensorNeed]) -> Dict[str, TensorNeed]:
    """By name; a name needed twice (tied tables) must be needed with one shape."""
    out: Dict[str, TensorNeed] = {}
    for n in needs:
        n = TensorNeed(n.name, tuple(int(s) for s in n.shape), n.role)
        if n.name in out and out[n.name].shape != n.shape:
            raise WeightsError(f"the model needs tensor '{n.name}' with shapes {list(out[n.name].shape)} and {list(n.shape)}")
        out.setdefault(n.name, n)
    return out


def _converted(t: torch.Tensor, stored: str, role: str, compute_dtype: torch.dtype) -> torch.Tensor:
    if role == "table":
        return t.to(torch.int32)
    if stored == "BF16":
        return t if compute_dtype == torch.bfloat16 else t.to(torch.float32)
    return t.to(torch.float32)           # F32 stays, F16 widens exactly


def load_tensors(folder, needs: Iterable[TensorNeed], compute_dtype: torch.dtype, device,
                 ignorable: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    folder = Path(folder)
    path = folder / "model.safetensors"
    if not path.exists():
        if (folder / "model.safetensors.index.json").exists():
            raise WeightsError(f"{folder}: sharded checkpoints (model.safetensors.index.json) are not supported")
        raise WeightsError(f"no model.safetensors in {folder}")
    if compute_dtype not in (torch.bfloat16, torch.float32):
        raise WeightsError(f"compute dtype {compute_dtype} is not supported (bfloat16 or float32)")
    wanted = merge_needs(needs)
    try:
        st = SafetensorsFile(path)
    except SafetensorsError as e:
        raise WeightsError(str(e)) from None

    missing, wrong_shape, wrong_dtype = [], [], []
    for name, need in wanted.items():
        e = st.entries.get(name)
        if e is None:
            missing.append(name)
        elif e.shape != need.shape:
            wrong_shape.append(f"{name}: file has {list(e.shape)}, the model needs {list(need.shape)}")
        elif e.dtype_name not in (_INTS if need.role == "table" else _FLOATS):
            kinds = "an integer type" if need.role == "table" else "F32, F16 or BF16"
            wrong_dtype.append(f"{name}: {e.dtype_name} (needs {kinds})")
    patterns = [re.compile(p) for p in ignorable]
    unexpected = [n for n in st.entries if n not in wanted and not any(p.fullmatch(n) for p in patterns)]
    if missing or wrong_shape or wrong_dtype or unexpected:
        lines = [f"{path} does not fit the model:"]
        for title, items in (("missing tensors", missing), ("unexpected tensors", unexpected),
                             ("wrong shapes", wrong_shape), ("unsupported dtypes", wrong_dtype)):
            if items:
                lines.append(f"  {title} ({len(items)}):")
                lines += [f"    {i}" for i in sorted(items)]
        raise WeightsError("\n".join(lines))

    out = {}
    for name, need in wanted.items():
        src = st.tensor(name)
        t = _converted(src, st.entries[name].dtype_name, need.role, compute_dtype).to(device).contiguous()
        out[name] = t.clone() if t.data_ptr() == src.data_ptr() else t       # never a view of the read-only mapping
    st.close()
    return out
