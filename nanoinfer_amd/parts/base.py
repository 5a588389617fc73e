"""What every part has in common, and the few types that parts and the engine exchange.

A part is built from its :class:`~nanoinfer_amd.config.spec.PartSpec` (kind, constants, tensor
names), the checkpoint tensors it asked for, and a :class:`Runtime` (compute type, device).  It
knows nothing of the model it sits in.  Interfaces, by family:

``embedding``     ``forward(token_ids[T] int32, ctx) -> h[T, d] float32`` (``ctx.positions`` for a learned position table)
``norm``          ``forward(h float32, pending | None, rows=None) -> x`` in the compute type;
                  without ``rows`` it first adds ``pending`` into ``h`` (the residual sum)
``position``      ``tables() -> (cos, sin) | None`` for the mixer that owns it
``mixer``         ``cache_need() -> CacheNeed``; ``forward(x, ctx, cache) -> y[T, d]``
``feed_forward``  ``forward(x, ctx) -> y[T, d]``
``block``         ``forward(h, pending, ctx, cache) -> (h, pending)``
``head``          ``forward(x[R, d]) -> logits[R, vocab] float32``
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..config.spec import PartSpec


@dataclass(frozen=True)
class WeightRequest:
    """A tensor a part wants from the checkpoint: its name there and the shape it must have."""

    name: str
    shape: Tuple[int, ...]


@dataclass(frozen=True)
class KVNeed:
    """Keys and values in pages.  ``window`` None: every earlier key; n: the last n keys only."""

    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """A fixed-size state per request: one tensor of this shape and type for every live request."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass(frozen=True)
class CacheNeed:
    kv: Optional[KVNeed] = None
    state: Optional[StateNeed] = None


class Runtime:
    """Compute type and device of a model, and buffers that parts share (one rotation table for
    all layers with the same constants, one device copy of a tensor used twice)."""

    def __init__(self, dtype: torch.dtype, device: torch.device):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute type {dtype} is not supported (float32 or bfloat16)")
        self.dtype = dtype
        self.device = device
        self.shared: Dict[object, object] = {}

    def matrix(self, name: str, cpu: torch.Tensor) -> torch.Tensor:
        """A checkpoint matrix on the device in the compute type; the same name gives the same buffer."""
        key = ("matrix", name, self.dtype)
        t = self.shared.get(key)
        if t is None:
            t = cpu.to(device=self.device, dtype=self.dtype).contiguous()
            self.shared[key] = t
        return t

    def weight(self, name: str, cpu: torch.Tensor, tiled: bool = True):
        """A checkpoint matrix as a :class:`nanoinfer_amd.kernels.Weight`: its rows on the device in the
        compute type (shared with :meth:`matrix`) plus, when ``tiled``, the copy that the skinny
        product of decoding streams."""
        from .. import kernels as K
        key = ("weight", name, self.dtype, tiled)
        w = self.shared.get(key)
        if w is None:
            w = K.Weight(self.matrix(name, cpu), tiled=tiled)
            self.shared[key] = w
        return w

    def vector32(self, name: str, cpu: torch.Tensor) -> torch.Tensor:
        """A one-dimensional parameter (a norm's weight) on the device, always float32."""
        key = ("vector", name)
        t = self.shared.get(key)
        if t is None:
            t = cpu.to(device=self.device, dtype=torch.float32).contiguous()
            self.shared[key] = t
        return t


class Part:
    """Base of all parts.  ``family`` and ``kind`` are set by ``register_part``."""

    family = ""
    kind = ""
    # True when a part's launches depend only on device data and on the sizes of the step, so that
    # a step may be recorded once and replayed; a part that reads the step's host lists says False
    graph_safe = False

    @classmethod
    def weight_requests(cls, spec: PartSpec) -> List[WeightRequest]:
        return []

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        self.spec = spec
        self.rt = rt


def pending_for(norm, pending: Optional[torch.Tensor], dtype: torch.dtype) -> Optional[torch.Tensor]:
    """``pending`` as ``norm`` takes it.  A product of a few rows may hand its result on as float32
    addends [S, T, d] (its K range was cut into S shares); a norm that says ``takes_addends`` sums
    them itself, for any other they are summed here into one [T, d] of the compute type."""
    if pending is not None and pending.dim() == 3 and not getattr(norm, "takes_addends", False):
        return pending.sum(dim=0).to(dtype)
    return pending


@dataclass
class LayerCache:
    """What one entry of the execution order sees of the cache in one step."""

    kpool: Optional[torch.Tensor] = None          # [pages, kv_heads, page_size, head_dim]
    vpool: Optional[torch.Tensor] = None
    block_table: Optional[torch.Tensor] = None    # int32 [sequences, pages]; -1 where a page was given back
    slot_mapping: Optional[torch.Tensor] = None   # int32 [tokens]: page * page_size + slot of each new token
    page_size: int = 0
    state: Optional[torch.Tensor] = None          # [slots, *StateNeed.shape]
    writes: bool = True
