"""A model put together from parts according to a :class:`ModelSpec`, and one forward pass of it
over the tokens of a step.

Order of a pass (src/model/llama.cpp:297-386): embedding, the blocks in the order the spec lists
them, then, on the wanted rows only, the last norm and the output head.  The reference computes
logits for every row and throws most away (src/engine/engine.cpp:310-338).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.spec import ModelSpec
from ..parts.base import CacheNeed, LayerCache, Runtime, flag_of, pending_for
from ..parts.standard import build_part
from ..registry import get_part


class Model:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        self.spec = spec
        self.rt = rt
        self.embedding = build_part("embedding", spec.embedding, tensors, rt)
        self.blocks = [get_part("block", b.kind)(b, tensors, rt) for b in spec.blocks]
        self.final_norm = build_part("norm", spec.final_norm, tensors, rt)
        self.head = build_part("head", spec.head, tensors, rt)
        for run in spec.order:
            if not 0 <= run.block < len(self.blocks):
                raise ValueError(f"the order names block {run.block}, the model has {len(self.blocks)}")
        self._needs: Dict[int, CacheNeed] = {}
        writers = set()
        for run in spec.order:
            need = self.blocks[run.block].cache_need()
            if run.cache in self._needs and self._needs[run.cache] != need:
                raise ValueError(f"cache {run.cache} is used by blocks with different needs: "
                                 f"{self._needs[run.cache]} and {need}")
            self._needs[run.cache] = need
            if run.writes_cache:
                writers.add(run.cache)
            elif run.cache not in writers:
                raise ValueError(f"block {run.block} reads cache {run.cache} before any block has written it")
        self.max_positions = spec.max_positions

    def _all_parts(self):
        return [self.embedding, self.final_norm, self.head] + list(self.blocks)

    def graph_safe(self) -> bool:
        """Whether a step of this model may be recorded into a HIP graph: every part says of itself
        that its launches depend on device data only (``graph_safe``), never on the host lists."""
        return all(flag_of(p, "graph_safe", False) for p in self._all_parts())

    def idempotent(self) -> bool:
        """Whether running the same step twice leaves the caches as running it once does: true of keys
        and values written to their places, not of a per-request state that a part updates in place."""
        return all(flag_of(p, "idempotent", True) for p in self._all_parts())

    def cache_needs(self) -> Dict[int, CacheNeed]:
        return dict(self._needs)

    def forward(self, ctx, layer_cache, logits_out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run the step described by ``ctx``; ``layer_cache(cache_id, writes)`` gives the
        :class:`LayerCache` of an entry of the order.  Returns float32 logits of ``ctx.logit_rows``
        (None when no row is wanted; the caches are filled all the same).  ``logits_out``: float32
        [at least as many rows, vocab] whose first rows are to take the logits, for a head that
        ``writes_into`` a given tensor (any other head returns a tensor of its own)."""
        h = self.embedding.forward(ctx.token_ids, ctx)
        pending = None
        order = self.spec.order
        T = h.shape[0]
        for i, run in enumerate(order):
            cache: LayerCache = layer_cache(run.cache, run.writes_cache)
            block = self.blocks[run.block]
            # what the block behind this one would like to find beside the stream (its first norm's input half
            # done by this block's last product), if both blocks know of that
            wants = getattr(self.blocks[order[i + 1].block], "wants_scaled", None) if i + 1 < len(order) else None
            leave = wants(T) if wants is not None and getattr(block, "leaves_for_next", False) else None
            if leave is not None:
                h, pending = block.forward(h, pending, ctx, cache, leave=leave)
            else:
                h, pending = block.forward(h, pending, ctx, cache)
        if ctx.logit_rows is None or ctx.logit_rows.shape[0] == 0:
            return None
        x = self.final_norm.forward(h, pending_for(self.final_norm, pending, self.rt.dtype), rows=ctx.logit_rows)
        if logits_out is not None and getattr(self.head, "writes_into", False):
            return self.head.forward(x, out=logits_out[:x.shape[0]])
        return self.head.forward(x)
