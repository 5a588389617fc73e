"""The description of a model as data: parts, their parameters, and the order they run in.

An architecture's builder turns its typed configuration into a :class:`ModelSpec`.  Nothing in
a spec names the architecture it came from: a part is ``kind`` (a key of a part registry) plus
``params`` (its sizes and constants) plus ``weights`` (logical weight name -> tensor name in the
checkpoint).  The reference wires these by hand for one model (src/model/llama.cpp:398-412,
568-706); here the wiring is a value that another builder can fill differently, layer by layer.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass
class PartSpec:
    """One part: which implementation (``kind``), with which constants, fed by which tensors."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    weights: Dict[str, str] = field(default_factory=dict)


@dataclass
class BlockSpec:
    """A residual block: which arrangement (``kind``, a key of the block registry) of which parts.

    ``parts`` maps the role a part plays in the block to its spec; which roles a kind of block has,
    and of which family each is, is that block class's own knowledge (the ``prenorm`` block, x +
    mixer(norm(x)) then x + ffn(norm(x)), src/model/llama.cpp:324-379, has ``mixer_norm``,
    ``mixer``, ``ffn_norm`` and ``ffn``).  Another arrangement (more norms, a mixer beside the
    feed-forward) is another block class with other roles; nothing else changes.  ``params``
    holds constants of the arrangement itself.  A role reads as an attribute: ``spec.mixer``.
    """

    kind: str
    parts: Dict[str, PartSpec] = field(default_factory=dict)
    params: Dict[str, Any] = field(default_factory=dict)

    def __getattr__(self, role: str) -> PartSpec:
        parts = self.__dict__.get("parts")
        if parts is not None and role in parts:
            return parts[role]
        raise AttributeError(f"block of kind {self.__dict__.get('kind')!r} has no part {role!r}; "
                             f"it has {sorted(parts or ())}")


@dataclass
class LayerRun:
    """One entry of the execution order: run block ``block`` on cache ``cache``.

    A block may appear in several entries (its weights are used again); ``cache`` is the index
    of the per-layer cache it reads, and writes when ``writes_cache`` holds.  An entry with
    ``writes_cache=False`` reads what an earlier entry with the same ``cache`` wrote.
    """

    block: int
    cache: int
    writes_cache: bool = True


@dataclass
class ModelSpec:
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    blocks: List[BlockSpec]
    order: List[LayerRun]
    final_norm: PartSpec
    head: PartSpec
    bos_token_id: Optional[int] = None
    eos_token_ids: tuple = ()
    # tensor name -> name of the tensor it may merely repeat (a tied head stored a second time);
    # such a tensor is accepted in a checkpoint when it equals the original and is not loaded
    duplicates: Dict[str, str] = field(default_factory=dict)
    # endings of tensor names that a checkpoint may hold without the model asking for them (buffers that
    # exporters write along, such as a rotation's stored frequencies); they are not loaded
    ignorable_suffixes: tuple = ()

    def num_caches(self) -> int:
        return 1 + max((r.cache for r in self.order), default=-1)
