"""The step function: one batch of (request, its next tokens) through the model, from the cache.

The reference runs each prompt chunk as a forward of its own and then one forward for all decode
tokens, under a single ``is_prefill`` flag (include/nanoinfer/model/model.h:19-31,
src/engine/engine.cpp:215-250).  Here a step is one flat list of tokens: portions of prompts of
any length beside single decoded tokens, each token with its position, its sequence and its
place in the cache; a decode token is a portion of length one.  Only the tokens given are run;
everything earlier is read from the pages that earlier steps filled.

The scheduler and the trace-replay program both drive :meth:`ModelRunner.step`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, Iterable, List, Optional, Sequence

import torch

from .. import kernels as K
from ..cache.block_manager import OutOfPages
from ..cache.manager import KVCacheManager
from ..parts.base import LayerCache, Runtime
from ..weights.loader import load_tensors, read_model_folder
from .model import Model


@dataclass
class StepEntry:
    """The next tokens of one request and the places among them whose logits are wanted."""

    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


class StepError(RuntimeError):
    pass


@dataclass
class GroupView:
    block_table: torch.Tensor     # int32 [B, pages]
    slot_mapping: torch.Tensor    # int32 [T]
    page_size: int


class StepContext:
    """Everything a part may want to know about the step it is running in.

    Device tensors (int32): ``token_ids``, ``positions``, ``seq_of_token`` [T]; ``logit_rows`` [R];
    per cache group a block table [B, pages] and a slot mapping [T].  Host lists, one entry per
    sequence of the step, in batch order: ``requests``, ``q_start`` (first row of its portion),
    ``q_len``, ``context_len`` (tokens in the cache after this step), ``state_slot``.
    """

    def __init__(self, device: torch.device):
        self.device = device
        self.n_tokens = 0
        self.n_seqs = 0
        self.requests: List[Hashable] = []
        self.q_start: List[int] = []
        self.q_len: List[int] = []
        self.context_len: List[int] = []
        self.state_slot: List[int] = []
        self.max_context = 0
        self.max_q_len = 0
        self.token_ids: torch.Tensor = None
        self.positions: torch.Tensor = None
        self.seq_of_token: torch.Tensor = None
        self.logit_rows: Optional[torch.Tensor] = None
        self.groups: List[GroupView] = []
        self._workspace: Optional[torch.Tensor] = None
        self._workspace_owner = None

    def workspace(self, n_floats: int) -> torch.Tensor:
        """Float32 scratch that lives until the next request for scratch (one user at a time)."""
        owner = self._workspace_owner
        ws = owner._scratch if owner is not None else self._workspace
        if ws is None or ws.numel() < n_floats:
            ws = torch.empty(max(n_floats, 1 << 16), dtype=torch.float32, device=self.device)
            if owner is not None:
                owner._scratch = ws
            else:
                self._workspace = ws
        return ws


class ModelRunner:
    """A model, its cache, and the step function over both.

    ``max_tokens`` is the number of tokens the page pools hold (rounded up to whole pages);
    ``max_requests`` the number of requests that may be live at once.
    """

    def __init__(self, model_dir: str, dtype: str = "bfloat16", page_size: int = 16, max_tokens: int = 4096,
                 max_requests: int = 64, device: Optional[torch.device] = None):
        self.device = device or K.require_gpu()
        torch_dtype = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
                       "float32": torch.float32, "fp32": torch.float32}.get(dtype)
        if torch_dtype is None:
            raise ValueError(f"dtype {dtype!r} is not one of bfloat16, float32")
        self.dtype = torch_dtype
        self.arch, self.config, self.spec = read_model_folder(model_dir)
        tensors = load_tensors(model_dir, self.spec)
        self.rt = Runtime(torch_dtype, self.device)
        self.model = Model(self.spec, tensors, self.rt)
        del tensors
        self.page_size = int(page_size)
        num_pages = (int(max_tokens) + self.page_size - 1) // self.page_size
        self.cache = KVCacheManager(self.model.cache_needs(), self.page_size, num_pages, max_requests,
                                    dtype=torch_dtype, device=self.device)
        self.vocab_size = self.spec.vocab_size
        self.max_positions = self.model.max_positions
        self.eos_token_ids = tuple(self.spec.eos_token_ids)
        self._done: Dict[Hashable, int] = {}   # tokens of each live request already in the cache
        self._scratch: Optional[torch.Tensor] = None

    # ---------------------------------------------------------------- bookkeeping
    def computed_tokens(self, request: Hashable) -> int:
        return self._done.get(request, 0)

    def release(self, request: Hashable) -> None:
        if request in self._done:
            del self._done[request]
            self.cache.release(request)

    def can_run(self, request: Hashable, n_new: int) -> bool:
        return self.cache.can_reserve(request, self._done.get(request, 0) + n_new)

    # ---------------------------------------------------------------- the step
    def _build_context(self, entries: List[StepEntry]) -> StepContext:
        ctx = StepContext(self.device)
        ctx._workspace_owner = self
        ps = self.page_size
        token_ids: List[int] = []
        positions: List[int] = []
        seq_of_token: List[int] = []
        logit_rows: List[int] = []
        seen = set()
        for e in entries:
            if e.request in seen:
                raise StepError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.request!r} brings no tokens")
            for t in e.tokens:
                if not 0 <= int(t) < self.vocab_size:
                    raise StepError(f"token id {t} of request {e.request!r} is outside the vocabulary "
                                    f"of {self.vocab_size}")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {e.request!r} wants the logits of place {w} among {n} tokens")
            done = self._done.get(e.request, 0)
            if done + n > self.model.max_positions:
                raise StepError(f"request {e.request!r} would reach {done + n} tokens, the model's positions "
                                f"end at {self.model.max_positions}")
        # reserve for all entries, or for none
        totals = [(e.request, self._done.get(e.request, 0) + len(e.tokens)) for e in entries]
        if not self.cache.can_reserve_all(totals):
            raise OutOfPages(f"the step needs more pages or state slots than are free "
                             f"({self.cache.min_free_pages()} pages, {self.cache.slots.num_free} slots free)")
        for request, total in totals:
            if not self.cache.reserve(request, total):
                raise StepError(f"reserving {total} tokens for request {request!r} failed after the check passed")
        row = 0
        for si, e in enumerate(entries):
            n = len(e.tokens)
            done = self._done.get(e.request, 0)
            ctx.requests.append(e.request)
            ctx.q_start.append(row)
            ctx.q_len.append(n)
            ctx.context_len.append(done + n)
            ctx.state_slot.append(self.cache.state_slot(e.request))
            token_ids.extend(int(t) for t in e.tokens)
            positions.extend(range(done, done + n))
            seq_of_token.extend([si] * n)
            logit_rows.extend(row + int(w) for w in e.want)
            row += n
        ctx.n_tokens = row
        ctx.n_seqs = len(entries)
        ctx.max_context = max(ctx.context_len)
        ctx.max_q_len = max(ctx.q_len)
        T, B, R = row, len(entries), len(logit_rows)
        # one upload for all integer tables
        flat: List[int] = token_ids + positions + seq_of_token + logit_rows
        group_meta = []
        for g in self.cache.groups:
            tables = [g.tables[e.request] for e in entries]
            width = max(len(t) for t in tables)
            slot_mapping: List[int] = []
            for e, table in zip(entries, tables):
                done = self._done.get(e.request, 0)
                for p in range(done, done + len(e.tokens)):
                    page = table[p // ps]
                    if page < 0:
                        raise StepError(f"request {e.request!r}: position {p} lies in a page already given back")
                    slot_mapping.append(page * ps + p % ps)
            off_slot = len(flat)
            flat.extend(slot_mapping)
            off_table = len(flat)
            for t in tables:
                flat.extend(t)
                flat.extend([-1] * (width - len(t)))
            group_meta.append((off_slot, off_table, width))
        dev = torch.tensor(flat, dtype=torch.int32).to(self.device, non_blocking=False)
        ctx.token_ids = dev[0:T]
        ctx.positions = dev[T:2 * T]
        ctx.seq_of_token = dev[2 * T:3 * T]
        ctx.logit_rows = dev[3 * T:3 * T + R] if R else None
        for (off_slot, off_table, width) in group_meta:
            ctx.groups.append(GroupView(block_table=dev[off_table:off_table + B * width].view(B, width),
                                        slot_mapping=dev[off_slot:off_slot + T], page_size=ps))
        return ctx

    def _layer_cache(self, ctx: StepContext):
        cache = self.cache

        def get(cache_id: int, writes: bool) -> LayerCache:
            lc = LayerCache(writes=writes, page_size=self.page_size)
            gi = cache.group_of_cache.get(cache_id)
            if gi is not None:
                g = cache.groups[gi]
                view = ctx.groups[gi]
                lc.kpool = g.kpools[cache_id]
                lc.vpool = g.vpools[cache_id]
                lc.block_table = view.block_table
                lc.slot_mapping = view.slot_mapping
            if cache_id in cache.state:
                lc.state = cache.state[cache_id]
            return lc

        return get

    def step(self, entries: Sequence[StepEntry], end: Iterable[Hashable] = ()) -> Optional[torch.Tensor]:
        """Run one batch.  Returns float32 logits ``[wanted, vocab]`` on the device, rows in the
        order of the entries and of each entry's ``want`` (None when nothing is wanted).  Requests
        named in ``end`` give back what they hold after the step."""
        entries = list(entries)
        logits = None
        if entries:
            ctx = self._build_context(entries)
            logits = self.model.forward(ctx, self._layer_cache(ctx))
            for e, total in zip(entries, ctx.context_len):
                self._done[e.request] = total
                self.cache.release_passed(e.request, total)
        for r in end:
            self.release(r)
        return logits
