"""What a mixer asks of the cache manager for one layer of the run order."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class PagedKvNeed:
    """Keys and values of every position (or of the last `window` positions) in pages."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None

    def elements_per_position(self) -> int:
        return 2 * self.n_kv_heads * self.head_dim


@dataclass(frozen=True)
class StateNeed:
    """A state of fixed size per request (for instance a recurrent state), zeroed when a request starts."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
