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
``block``         ``forward(h, pending, ctx, cache) -> (h, pending)``; its parts by role (:class:`Block`)
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

    def __init__(self, dtype: torch.dtype, device: torch.device, tiled: bool = True):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute type {dtype} is not supported (float32 or bfloat16)")
        self.dtype = dtype
        self.device = device
        # False: no layer matrix gets the second, re-tiled copy that the products of decode steps stream; they
        # then read the rows as stored (slower), and device memory holds the checkpoint once
        self.tiled = bool(tiled)
        self.shared: Dict[object, object] = {}

    def device_bytes(self) -> int:
        """Bytes of device memory that the model's tensors take (every shared buffer once)."""
        seen, total = set(), 0
        for value in self.shared.values():
            for t in (value if isinstance(value, tuple) else (getattr(value, "rows", value), getattr(value, "tiles", None))):
                if isinstance(t, torch.Tensor) and t.is_cuda and t.untyped_storage().data_ptr() not in seen:
                    seen.add(t.untyped_storage().data_ptr())
                    total += t.untyped_storage().nbytes()
        return total

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
        tiled = tiled and self.tiled
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
    # False when running the same step a second time changes what the part leaves behind (a state
    # updated in place: keys and values written again at the same places are the same).  Whoever runs
    # a step more than once (the recording of a step into a HIP graph does) then puts the
    # per-request state back in between.
    idempotent = True

    @classmethod
    def weight_requests(cls, spec: PartSpec) -> List[WeightRequest]:
        return []

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        self.spec = spec
        self.rt = rt


def flag_of(part, name: str, default: bool) -> bool:
    """A yes/no property of a part (``graph_safe``, ``idempotent``) that a simple part states as a
    class attribute and a part made of parts (a block) as a method."""
    value = getattr(part, name, default)
    return bool(value() if callable(value) else value)


class Block:
    """Base of the blocks: an arrangement of parts around the residual stream.

    A block class names its roles and the family of each in ``ROLES`` (role -> family); the base
    asks every role's part for its tensors, builds the parts as attributes of those names, and
    answers for the whole block what each part answers for itself.  ``forward(h, pending, ctx,
    cache) -> (h, pending)`` is the subclass's: ``h`` is the float32 residual stream [T, d],
    ``pending`` an addend that the stream has not received yet (or None), which the next norm sums
    in; the cache goes to the block's ``mixer``.  ``pending`` may also be something that is no tensor:
    the next norm's input as the last product left it half done, beside a stream that is complete
    (:class:`nanoinfer_amd.kernels.ScaledInput`); :func:`pending_for` turns that into None for a norm
    that runs as a step of its own.  A block that sets ``leaves_for_next = True`` takes ``leave=`` in
    its ``forward``: what ``wants_scaled(T)`` of the block that runs next returned, if that block has
    such a method and returned anything."""

    family = "block"
    kind = ""
    ROLES: Dict[str, str] = {}

    @classmethod
    def _roles(cls, spec):
        missing = [r for r in cls.ROLES if r not in spec.parts]
        extra = [r for r in spec.parts if r not in cls.ROLES]
        if missing or extra:
            raise ValueError(f"a block of kind {spec.kind!r} has the parts {sorted(cls.ROLES)}; "
                             f"missing: {missing}, not known: {extra}")
        return cls.ROLES.items()

    @classmethod
    def weight_requests(cls, spec) -> List[WeightRequest]:
        from ..registry import get_part
        out: List[WeightRequest] = []
        for role, family in cls._roles(spec):
            out += get_part(family, spec.parts[role].kind).weight_requests(spec.parts[role])
        return out

    def __init__(self, spec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        from .standard import build_part
        self.spec = spec
        self.rt = rt
        self.roles = []
        for role, family in self._roles(spec):
            setattr(self, role, build_part(family, spec.parts[role], tensors, rt))
            self.roles.append(role)

    def parts(self):
        return [getattr(self, r) for r in self.roles]

    def cache_need(self) -> "CacheNeed":
        """What the block wants of the cache: what its mixer wants."""
        return self.mixer.cache_need()

    def graph_safe(self) -> bool:
        return all(flag_of(p, "graph_safe", False) for p in self.parts())

    def idempotent(self) -> bool:
        return all(flag_of(p, "idempotent", True) for p in self.parts())


def pending_for(norm, pending: Optional[torch.Tensor], dtype: torch.dtype) -> Optional[torch.Tensor]:
    """``pending`` as ``norm`` takes it.  A product of a few rows may hand its result on as float32
    addends [S, T, d] (its K range was cut into S shares); a norm that says ``takes_addends`` sums
    them itself, for any other they are summed here into one [T, d] of the compute type."""
    if pending is not None and not isinstance(pending, torch.Tensor):
        return None       # a norm's input left half done by the product before it: the stream itself is complete
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
