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

from dataclasses import dataclass
from typing import Dict, Hashable, Iterable, List, Optional, Sequence

import numpy as np
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


@dataclass
class SeqTables:
    """What the step knows of each of its sequences, on the device (int32 [B] each, batch order):
    the first row of its portion, the portion's length, the tokens in the cache after the step, and
    the request's state slot.  A part whose launches may be recorded reads these, never the host lists."""

    q_start: torch.Tensor
    q_len: torch.Tensor
    context_len: torch.Tensor
    state_slot: torch.Tensor


@dataclass
class DrawView:
    """The options of a step's draw on the device, one entry per row in batch order."""

    temperature: torch.Tensor     # float32 [B]
    top_p: torch.Tensor           # float32 [B]
    uniform: torch.Tensor         # float32 [B]: the number each row's draw is taken with
    top_k: torch.Tensor           # int32 [B]


@dataclass
class _Layout:
    """Where the parts of a step's flat integer table lie: per cache group (offset of the slot
    mapping, offset of the block table, table width), and the offset of the per-sequence table
    (four rows of B entries: first row, length, context length, state slot)."""

    groups: list
    seq: int
    draw: Optional[int] = None      # offset of the draw's table (temperature, top_p, uniform as float bits, top_k: B each), if the step has one


_HOST_LISTS = ("requests", "q_start", "q_len", "context_len", "state_slot")


class StepContext:
    """Everything a part may want to know about the step it is running in.

    Device tensors (int32): ``token_ids``, ``positions``, ``seq_of_token`` [T]; ``logit_rows`` [R];
    per cache group a block table [B, pages] and a slot mapping [T].  Host lists, one entry per
    sequence of the step, in batch order: ``requests``, ``q_start`` (first row of its portion),
    ``q_len``, ``context_len`` (tokens in the cache after this step), ``state_slot``.
    ``max_context`` bounds every context length of the step; in a step that is recorded into a
    HIP graph it is a rounded-up bound, and the host lists must not steer the computation.
    """

    def __init__(self, device: torch.device, scratch_owner=None, recording: bool = False):
        self.device = device
        self.n_tokens = 0
        self.n_seqs = 0
        self._host = {name: [] for name in _HOST_LISTS}
        self._sealed = False
        self.max_context = 0
        self.max_q_len = 0
        self.token_ids: torch.Tensor = None
        self.positions: torch.Tensor = None
        self.seq_of_token: torch.Tensor = None
        self.logit_rows: Optional[torch.Tensor] = None
        self.per_seq: Optional[SeqTables] = None
        self.draw: Optional[DrawView] = None
        self.groups: List[GroupView] = []
        self.recording = recording
        self._scratch_owner = scratch_owner
        self._scratch: Optional[torch.Tensor] = None
        self._q_tiles: Dict[int, torch.Tensor] = {}
        self.tile_sizes_asked = set()

    def __getattr__(self, name: str):
        # the host lists: one entry per sequence, in batch order.  While a step is being recorded they
        # are not there to read: the recording would keep what they said at that moment for every replay.
        if name in _HOST_LISTS:
            if self.__dict__.get("_sealed"):
                raise StepError(f"ctx.{name} is a host list, and this step is being recorded: its replays "
                                f"would run with the values of now.  Read ctx.per_seq (the same per sequence, "
                                f"on the device), or declare the part graph_safe = False")
            return self.__dict__["_host"][name]
        raise AttributeError(name)

    def seal(self) -> None:
        """From here on the host lists cannot be read (the runner calls this before it records)."""
        self._sealed = True

    def q_tiles(self, tile_tokens: int) -> Optional[torch.Tensor]:
        """The portions of the step cut into tiles of at most ``tile_tokens`` tokens, int32 [n, 4]
        rows of (sequence, first row, tokens, first position) on the device; built once per step
        and tile size from the host lists.  A recorded step has the tables it was recorded with
        (the runner refills them before every replay) and no others: None then."""
        t = self._q_tiles.get(tile_tokens)
        if t is None:
            self.tile_sizes_asked.add(tile_tokens)
            if self.recording:
                return None
            host = self._host
            flat = K.build_q_tiles(host["q_start"], host["q_len"], host["context_len"], tile_tokens)
            upload = getattr(self._scratch_owner, "_upload", None)
            if upload is not None:       # through the runner's pinned buffers: the host does not wait for the GPU
                t = upload(flat).view(-1, 4)
            else:
                t = torch.tensor(flat, dtype=torch.int32).view(-1, 4).to(self.device)
            self._q_tiles[tile_tokens] = t
        return t

    def workspace(self, n_floats: int) -> torch.Tensor:
        """Float32 scratch that lives until the next request for scratch (one user at a time)."""
        if self.recording or self._scratch_owner is None:
            # a recorded step keeps its scratch in the graph's own memory
            if self._scratch is None or self._scratch.numel() < n_floats:
                self._scratch = torch.empty(n_floats, dtype=torch.float32, device=self.device)
            return self._scratch
        owner = self._scratch_owner
        if owner._scratch is None or owner._scratch.numel() < n_floats:
            owner._scratch = torch.empty(max(n_floats, 1 << 16), dtype=torch.float32, device=self.device)
        return owner._scratch


@dataclass
class _RecordedStep:
    """A decode step of fixed shape recorded into a HIP graph, with the buffers it reads and writes."""

    graph: "torch.cuda.CUDAGraph"
    meta: torch.Tensor            # int32, device: every integer table of the step, fixed layout
    stagings: list                # the same in pinned host memory: a few buffers used in turn, so that the host can
                                  # write the tables of a step while the uploads of the steps before it are still queued
    logits: torch.Tensor
    ctx: StepContext
    copied: list = None                  # per staging buffer: its last upload has read it
    turn: int = 0                        # the staging buffer that holds the tables of the last replay
    layout: list = None                  # per group (offset of slot mapping, offset of table, table width)
    order: tuple = ()                    # requests of the last replay, in batch order
    pages_written: list = None           # per group, per sequence: table entries already in the staging buffer
    tiles: dict = None                   # tile size -> (offset in the tables, number of tiles), for recorded prompt portions
    greedy: torch.Tensor = None          # int32, pinned host: argmax of every row of the logits, copied after a replay
    amax: torch.Tensor = None            # the same on the device, picked by the recording itself; a recorded decode step
                                         # writes it over its own token ids, where its next replay finds them without the host
    replayed: "torch.cuda.Event" = None  # the last replay has finished (and with it the copy into ``greedy``)
    held_bytes: int = 0                  # device memory the recording holds (what the allocator's reserve grew by)


class _Gpu:
    """What recording a step needs from the device besides the model: kept apart so that the
    runner's host side (tables, books, the order of runs while a step is recorded) can be driven
    without a GPU by handing it other services."""

    @staticmethod
    def synchronize() -> None:
        torch.cuda.synchronize()

    @staticmethod
    def pinned(t: torch.Tensor) -> torch.Tensor:
        return t.pin_memory()

    @staticmethod
    def event():
        return torch.cuda.Event()

    @staticmethod
    def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        return K.argmax(logits, out=out)

    @staticmethod
    def reserved_bytes() -> int:
        return int(torch.cuda.memory_reserved())

    @staticmethod
    def draw(logits, work, view: "DrawView", ones, zeros, out, uses_top_k: bool, uses_top_p: bool) -> torch.Tensor:
        """One token per row of ``logits`` into ``out`` by the sampling kernels, without a repetition penalty
        (``ones``: a penalty of 1 per row; ``zeros``: the empty lists of penalised tokens)."""
        R = logits.shape[0]
        return K.sample(logits, work, view.temperature, view.top_k, view.top_p, ones[:R], zeros[:1], zeros[:R + 1],
                        view.uniform, out, uses_top_k=uses_top_k, uses_top_p=uses_top_p)

    @staticmethod
    def capture(run):
        """Record what ``run()`` launches into a HIP graph (nothing is executed meanwhile); returns the
        graph and what ``run`` returned.  Python's cycle collector is held off meanwhile: what it
        finds may be an older runner with recordings of its own, and destroying a graph is one of
        the calls that the runtime refuses while a stream is being captured (the refusal arrives in a
        destructor and ends the process)."""
        import gc
        graph = torch.cuda.CUDAGraph()
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                result = run()
        finally:
            if collecting:
                gc.enable()
        return graph, result


class ModelRunner:
    """A model, its cache, and the step function over both.

    ``max_tokens`` is the number of tokens the page pools hold (rounded up to whole pages);
    ``max_requests`` the number of requests that may be live at once.  With ``use_graphs`` a step
    that consists of single tokens only (decoding), or of one prompt portion of 64 tokens or more,
    is recorded once per shape into a HIP graph and replayed afterwards: the launches of a whole
    step then cost one call.
    """

    GRAPH_MAX_BATCH = 256         # decode steps of more sequences run eagerly
    STAGING_BUFFERS = 4           # pinned copies of a recorded step's tables, used in turn
    HISTORY_ROWS = 16             # decode steps launched back to back before the host reads their tokens
    GRAPH_MIN_PORTION = 64        # a shorter prompt portion is not worth a recording
    GRAPH_MAX_PORTIONS = 24       # recordings of prompt portions kept (each holds its activations)
    GRAPH_MAX_DECODES = 1024      # recordings of decode steps kept (their logits go to one buffer that all share);
                                  # beyond that the one used longest ago is dropped and its shape recorded again if it returns
    GRAPH_PORTION_SIGHTS = 2      # a portion's shape is recorded when it comes this many times: recording costs
                                  # seven runs of the step and gains a few per cent of a run (a lone length never pays)
    GRAPH_MAX_BYTES = 8 << 30     # device memory that all recordings together may hold (their logits, activations and
                                  # tables: what the allocator's reserved memory grew by while each was made);
                                  # beyond that the ones used longest ago are dropped, of either kind

    def __init__(self, model_dir: str, dtype: str = "bfloat16", page_size: int = 16, max_tokens: int = 4096,
                 max_requests: int = 64, device: Optional[torch.device] = None, use_graphs: bool = True,
                 warm_up: bool = True, max_step_tokens: Optional[int] = None, kv_cache_bytes: Optional[int] = None,
                 graph_memory_bytes: Optional[int] = None, one_weight_copy: bool = False):
        arch, config, spec = read_model_folder(model_dir)
        tensors = load_tensors(model_dir, spec)
        self._setup(spec, tensors, dtype, page_size, max_tokens, max_requests, device, use_graphs, warm_up,
                    max_step_tokens, kv_cache_bytes, graph_memory_bytes, arch=arch, config=config,
                    one_weight_copy=one_weight_copy)

    @classmethod
    def from_spec(cls, spec, tensors: Dict[str, torch.Tensor], dtype: str = "bfloat16", page_size: int = 16,
                  max_tokens: int = 4096, max_requests: int = 64, device: Optional[torch.device] = None,
                  use_graphs: bool = True, warm_up: bool = False, max_step_tokens: Optional[int] = None,
                  kv_cache_bytes: Optional[int] = None, graph_memory_bytes: Optional[int] = None,
                  one_weight_copy: bool = False) -> "ModelRunner":
        """A runner over a model given as data (a :class:`~nanoinfer_amd.config.spec.ModelSpec`) and its
        tensors by checkpoint name (CPU tensors), without a folder: the same model, cache manager and
        step function.  The tensors are checked against what the parts of the spec ask for."""
        from ..weights.loader import check_tensors
        self = cls.__new__(cls)
        self._setup(spec, check_tensors(spec, tensors), dtype, page_size, max_tokens, max_requests, device, use_graphs,
                    warm_up, max_step_tokens, kv_cache_bytes, graph_memory_bytes, one_weight_copy=one_weight_copy)
        return self

    def _setup(self, spec, tensors, dtype, page_size, max_tokens, max_requests, device, use_graphs, warm_up,
               max_step_tokens, kv_cache_bytes, graph_memory_bytes, arch=None, config=None, one_weight_copy=False) -> None:
        self.device = device or K.require_gpu()
        torch_dtype = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
                       "float32": torch.float32, "fp32": torch.float32}.get(dtype)
        if torch_dtype is None:
            raise ValueError(f"dtype {dtype!r} is not one of bfloat16, float32")
        self.dtype = torch_dtype
        self.arch, self.config, self.spec = arch, config, spec
        # the products of decode steps stream a re-tiled copy of every layer matrix beside the rows that the
        # library's product of prompt portions reads; ``one_weight_copy`` does without it (a slower decode step)
        self.rt = Runtime(torch_dtype, self.device, tiled=not one_weight_copy)
        el = 2 if torch_dtype == torch.bfloat16 else 4
        self.checkpoint_bytes = sum(t.numel() * (el if t.dim() > 1 else 4) for t in tensors.values())
        self.model = Model(self.spec, tensors, self.rt)
        del tensors
        self.page_size = int(page_size)
        num_pages = (int(max_tokens) + self.page_size - 1) // self.page_size
        if kv_cache_bytes is not None:      # a byte budget for the pools takes the place of the token count
            num_pages = KVCacheManager.pages_for_bytes(self.model.cache_needs(), self.page_size, int(kv_cache_bytes), torch_dtype)
            if num_pages < 1:
                raise ValueError(f"{kv_cache_bytes} bytes do not hold one page of {self.page_size} tokens of this model's cache")
        # with a bound on the tokens one request brings to a step, pools of windowed layers are only as
        # large as their windows need; a longer portion is then refused
        self.max_step_tokens = None if max_step_tokens is None else int(max_step_tokens)
        self.cache = KVCacheManager(self.model.cache_needs(), self.page_size, num_pages, max_requests,
                                    dtype=torch_dtype, device=self.device, max_step_tokens=self.max_step_tokens,
                                    scatter_pages=True)   # requests of equal length would else hold runs at regular distances
        self.vocab_size = self.spec.vocab_size
        self.max_positions = self.model.max_positions
        self.eos_token_ids = tuple(self.spec.eos_token_ids)
        self._done: Dict[Hashable, int] = {}   # tokens of each live request already in the cache
        self._scratch: Optional[torch.Tensor] = None
        if graph_memory_bytes is not None:
            self.GRAPH_MAX_BYTES = int(graph_memory_bytes)
        self._init_graphs(use_graphs)
        if warm_up:
            self._warm_up()

    def memory_report(self) -> Dict[str, int]:
        """Bytes of device memory: the model's tensors, what the checkpoint is in the compute type (matrices; norm
        weights in float32), the key and value pools, and what the recordings hold."""
        return {"weights": self.rt.device_bytes(), "checkpoint": int(self.checkpoint_bytes),
                "kv_pools": self.cache.pool_bytes(),
                "recordings": int(self._recorded_bytes) + (0 if self._logits_buffer is None else self._logits_buffer.numel() * 4)}

    def _warm_up(self) -> None:
        """One short prompt and one decode step of a request of the runner's own, run eagerly and given
        back: the code objects of the kernels and the matrix library's set-up are loaded while the model
        is, not during the first request (on the 1B shape that is 0.2 s of its first step)."""
        n = min(128, self.max_positions - 1, (self.cache.min_free_pages() - 1) * self.page_size,
                self.max_step_tokens or 128)
        if n < 2:
            return
        me = ("warm-up", id(self))
        graphs, self.use_graphs = self.use_graphs, False
        try:
            self.step([StepEntry(me, [0] * n, [n - 1])])
            logits = self.step([StepEntry(me, [0], [0])])
            self.gpu.argmax(logits)
            self.gpu.synchronize()
        finally:
            self.use_graphs = graphs
            self.release(me)

    gpu = _Gpu

    def _init_graphs(self, use_graphs: bool) -> None:
        import os
        self.use_graphs = bool(use_graphs) and self.model.graph_safe() and not os.environ.get("NANOINFER_NO_GRAPHS")
        self._recorded: Dict[tuple, _RecordedStep] = {}      # in the order of their last use
        self._recorded_bytes = 0                             # device memory the recordings hold, as measured when each was made
        self._logits_buffer = None                           # float32 [GRAPH_MAX_BATCH, vocabulary]: where recorded steps leave their logits
        self._work_buffer = None
        self._draw_consts = None
        self._unrecordable = set()
        self._portion_sights: Dict[tuple, int] = {}      # how often a prompt portion's shape has come without a recording
        self._staging = [(None, None)] * 3     # pinned host buffers for the tables of eager steps, and their uploads' events
        self._staging_turn = 0
        self._greedy_of = None                 # (logits returned by the last recorded step, its recording)
        self._history = None                   # pinned host: tokens chosen by decode steps launched back to back
        self._history_done = None
        self.timeline = None                   # a list: every step appends (event before its first launch, event
                                               # behind its last), for whoever measures the GPU's share of a step

    def _upload(self, flat) -> torch.Tensor:
        """The integer tables of an eager step on the device.  They go through one of a few pinned
        host buffers used in turn, so that the copy is asynchronous and the host can prepare and
        launch a step while the one before it still runs."""
        n = len(flat)
        i = self._staging_turn = (self._staging_turn + 1) % len(self._staging)
        buf, done = self._staging[i]
        if done is not None:
            done.synchronize()            # the upload that last used this buffer has read it
        if buf is None or buf.numel() < n:
            buf = self.gpu.pinned(torch.empty(max(n, 4096, 2 * (buf.numel() if buf is not None else 0)), dtype=torch.int32))
        buf.numpy()[:n] = flat
        dev = torch.empty(n, dtype=torch.int32, device=self.device)
        dev.copy_(buf[:n], non_blocking=True)
        done = done or self.gpu.event()
        done.record()
        self._staging[i] = (buf, done)
        return dev

    def greedy_tokens(self, logits: torch.Tensor) -> List[int]:
        """The index of the largest logit of every row (lowest index on ties).  For the logits of a
        recorded step the recording has already computed them and copied them to the host."""
        held = self._greedy_of
        if held is not None and held[0] is logits:
            rec = held[1]
            rec.replayed.synchronize()
            return rec.greedy.tolist()
        return self.gpu.argmax(logits).tolist()

    # ---------------------------------------------------------------- bookkeeping
    def computed_tokens(self, request: Hashable) -> int:
        return self._done.get(request, 0)

    def release(self, request: Hashable) -> None:
        if request in self._done:
            del self._done[request]
            self.cache.release(request)
            for rec in self._recorded.values():     # a later request of the same name starts its tables afresh
                if request in rec.order:
                    rec.order = ()

    def can_run(self, request: Hashable, n_new: int) -> bool:
        return self.cache.can_reserve(request, self._done.get(request, 0) + n_new)

    # ---------------------------------------------------------------- the step
    def _check_and_reserve(self, entries: List[StepEntry]) -> None:
        seen = set()
        vocab = self.vocab_size
        limit = self.model.max_positions
        step_limit = getattr(self, "max_step_tokens", None)
        totals = []
        for e in entries:
            if e.request in seen:
                raise StepError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            toks = e.tokens
            n = len(toks)
            if n == 0:
                raise StepError(f"request {e.request!r} brings no tokens")
            if step_limit is not None and n > step_limit:
                raise StepError(f"request {e.request!r} brings {n} tokens; the pools were sized for at most "
                                f"{step_limit} of one request in a step")
            if not (0 <= min(toks) and max(toks) < vocab):
                bad = next(t for t in toks if not 0 <= int(t) < vocab)
                raise StepError(f"token id {bad} of request {e.request!r} is outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {e.request!r} wants the logits of place {w} among {n} tokens")
            total = self._done.get(e.request, 0) + n
            if total > limit:
                raise StepError(f"request {e.request!r} would reach {total} tokens, the model's positions "
                                f"end at {limit}")
            totals.append((e.request, total))
        # reserve for all entries, or for none
        if not self.cache.reserve_all(totals):
            raise OutOfPages(f"the step needs more pages or state slots than are free "
                             f"({self.cache.min_free_pages()} pages, {self.cache.slots.num_free} slots free)")

    def _describe(self, entries: List[StepEntry], ctx: StepContext, table_width: Optional[int] = None, draw_rows=None):
        """Fill the host side of ``ctx`` and return every integer table of the step as one flat
        int32 array, with the places of its parts: [token ids | positions | sequence of token |
        logit rows | per group: slot mapping, block table | per sequence: first row, length,
        context length, state slot | the draw's table, if ``draw_rows`` (int32 [4 B]) is given]."""
        ps = self.page_size
        i32 = np.int32
        token_ids, positions, seq_of_token = [], [], []
        logit_rows: List[int] = []
        row = 0
        host = ctx._host
        for si, e in enumerate(entries):
            n = len(e.tokens)
            done = self._done.get(e.request, 0)
            host["requests"].append(e.request)
            host["q_start"].append(row)
            host["q_len"].append(n)
            host["context_len"].append(done + n)
            host["state_slot"].append(self.cache.state_slot(e.request))
            token_ids.append(np.asarray(e.tokens, dtype=i32))
            positions.append(np.arange(done, done + n, dtype=i32))
            seq_of_token.append(np.full(n, si, dtype=i32))
            for w in e.want:
                logit_rows.append(row + int(w))
            row += n
        ctx.n_tokens = row
        ctx.n_seqs = len(entries)
        ctx.max_context = max(host["context_len"])
        ctx.max_q_len = max(host["q_len"])
        pieces = token_ids + positions + seq_of_token + [np.asarray(logit_rows, dtype=i32)]
        at = 3 * row + len(logit_rows)
        layout = []
        B = len(entries)
        for g in self.cache.groups:
            tables = [g.tables[e.request] for e in entries]
            width = table_width or max(len(t) for t in tables)
            block_table = np.full((B, width), -1, dtype=i32)
            off_slot = at
            for b, (table, pos) in enumerate(zip(tables, positions)):
                block_table[b, :len(table)] = table
                pages = block_table[b, pos // ps]
                if (pages < 0).any():
                    p = int(pos[int(np.argmax(pages < 0))])
                    raise StepError(f"request {entries[b].request!r}: position {p} lies in a page already given back")
                pieces.append(pages * ps + pos % ps)
            at += row
            pieces.append(block_table.reshape(-1))
            layout.append((off_slot, at, width))
            at += B * width
        pieces.append(np.asarray(host["q_start"] + host["q_len"] + host["context_len"] + host["state_slot"], dtype=i32))
        off_draw = None
        if draw_rows is not None:
            if len(draw_rows) != 4 * B:
                raise StepError(f"a draw's table has four entries a sequence: {len(draw_rows)} for {B} sequences")
            off_draw = at + 4 * B
            pieces.append(np.asarray(draw_rows, dtype=i32))
        return np.concatenate(pieces), _Layout(layout, at, off_draw), len(logit_rows)

    def _bind(self, ctx: StepContext, dev: torch.Tensor, layout, n_rows: int) -> None:
        T, B = ctx.n_tokens, ctx.n_seqs
        ctx.token_ids = dev[0:T]
        ctx.positions = dev[T:2 * T]
        ctx.seq_of_token = dev[2 * T:3 * T]
        ctx.logit_rows = dev[3 * T:3 * T + n_rows] if n_rows else None
        ctx.groups = [GroupView(block_table=dev[off_table:off_table + B * width].view(B, width),
                                slot_mapping=dev[off_slot:off_slot + T], page_size=self.page_size)
                      for (off_slot, off_table, width) in layout.groups]
        at = layout.seq
        ctx.per_seq = SeqTables(dev[at:at + B], dev[at + B:at + 2 * B], dev[at + 2 * B:at + 3 * B], dev[at + 3 * B:at + 4 * B])
        if layout.draw is not None:
            at = layout.draw
            as_float = dev[at:at + 3 * B].view(torch.float32)
            ctx.draw = DrawView(as_float[0:B], as_float[B:2 * B], as_float[2 * B:3 * B], dev[at + 3 * B:at + 4 * B])

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

    # ---------------------------------------------------------------- recorded decode steps
    def _graph_shape(self, entries: List[StepEntry], draw=None):
        """Key of the recorded step that can run these entries, or None when they must run eagerly.
        Two kinds are recorded: single tokens only, each wanting its logits (``("d", batch, ...)``; with
        ``draw``, the (uses top-k, uses top-p) of a draw that the step makes itself, ``("s", batch, ...,
        draw)``), and one prompt portion alone that wants nothing or the logits of its last token
        (``("p", tokens, ..., wanted rows)``).  Table width and context bound are rounded up to
        powers of two so that few recordings serve a growing context."""
        if not self.use_graphs or not 0 < len(entries) <= self.GRAPH_MAX_BATCH:
            return None
        first = entries[0]
        n = len(first.tokens)
        if len(entries) == 1 and n >= self.GRAPH_MIN_PORTION:
            want = list(first.want)
            if want and want != [n - 1]:
                return None
            longest = self._done.get(first.request, 0) + n
            kind, size, rows = "p", n, len(want)
        else:
            if any(len(e.tokens) != 1 or list(e.want) != [0] for e in entries):
                return None
            longest = max(self._done.get(e.request, 0) for e in entries) + 1
            kind, size, rows = "d", len(entries), len(entries)
            if draw is not None:
                kind, rows = "s", (bool(draw[0]), bool(draw[1]))
        pages = max(16, 1 << (self.cache.pages_for(longest) - 1).bit_length())
        bound = max(256, 1 << (longest - 1).bit_length())
        key = (kind, size, pages, bound, rows)
        if key in self._unrecordable:
            return None
        if kind == "p" and key not in self._recorded:
            if sum(1 for k in self._recorded if k[0] == "p") >= self.GRAPH_MAX_PORTIONS:
                return None
            seen = self._portion_sights[key] = self._portion_sights.get(key, 0) + 1
            if seen < self.GRAPH_PORTION_SIGHTS:
                return None
        return key

    def _tables_of(self, entries: List[StepEntry], ctx: StepContext, width: int, tile_sizes, draw_rows=None):
        """Every integer table of a recorded step as one flat list: those of :meth:`_describe`, then
        the attention tiles of each tile size the model asked for."""
        flat, layout, n_rows = self._describe(entries, ctx, table_width=width, draw_rows=draw_rows)
        tiles = {}
        pieces, at = [flat], len(flat)
        for ts in sorted(tile_sizes):
            rows = K.build_q_tiles(ctx._host["q_start"], ctx._host["q_len"], ctx._host["context_len"], ts)
            tiles[ts] = (at, len(rows) // 4)        # where they start, how many
            pieces.append(np.asarray(rows, dtype=np.int32))
            at += len(rows)
        return (np.concatenate(pieces) if len(pieces) > 1 else flat), layout, n_rows, tiles

    def _state_keeper(self):
        """``rewind()``: puts the per-request state of every cache back to what it is now.  A step that
        is being recorded runs several times (once the ordinary way first, then in trial replays beside
        eager runs): keys and values land in the same places with the same values each time, but a
        state that a part updates in place would move on with every run.  For a model whose parts are
        all idempotent ``rewind`` does nothing."""
        if not self.cache.state or self.model.idempotent():
            return lambda: None
        kept = {cid: t.clone() for cid, t in self.cache.state.items()}

        def rewind() -> None:
            for cid, t in kept.items():
                self.cache.state[cid].copy_(t)
        return rewind

    def _record(self, key, entries: List[StepEntry], draw_rows=None) -> Optional[_RecordedStep]:
        kind, size, pages, bound, flags = key
        gpu = self.gpu
        decode = kind in ("d", "s")
        calls_before = K.library_calls()
        rewind = self._state_keeper()
        # run the step once the ordinary way first: code objects get loaded and buffers sized outside
        # the recording, and the model says which attention tiles it wants.  Keys, values and logits
        # are simply written again by later runs; per-request state is put back (``rewind``).
        warm = StepContext(self.device, scratch_owner=self)
        flat_w, layout_w, rows_w = self._describe(entries, warm, draw_rows=draw_rows)
        self._bind(warm, torch.from_numpy(flat_w).to(self.device), layout_w, rows_w)
        warm_logits = self.model.forward(warm, self._layer_cache(warm))
        if warm_logits is not None:
            gpu.argmax(warm_logits)
            if kind == "s":
                gpu.draw(warm_logits, self._shared_work()[:size], warm.draw, *self._draw_constants(),
                         torch.empty(size, dtype=torch.int32, device=self.device), *flags)
        gpu.synchronize()
        rewind()
        held_before = gpu.reserved_bytes()
        ctx = StepContext(self.device, recording=True)
        flat, layout, n_rows, tiles = self._tables_of(entries, ctx, pages, warm.tile_sizes_asked, draw_rows=draw_rows)
        ctx.max_context = bound
        staging = gpu.pinned(torch.from_numpy(flat))
        meta = staging.to(self.device, copy=True)
        self._bind(ctx, meta, layout, n_rows)
        for ts, (off, count) in tiles.items():
            ctx._q_tiles[ts] = meta[off:off + 4 * count].view(-1, 4)
        ctx.seal()
        greedy = gpu.pinned(torch.empty(max(n_rows, 1), dtype=torch.int32))

        def run():
            # the logits of every recording go to one buffer of the runner's: a replay's are copied out before the
            # next replay writes there, so a recording holds its activations only
            logits = self.model.forward(ctx, self._layer_cache(ctx), logits_out=self._shared_logits())
            amax = None
            if logits is not None:
                # greedy decoding needs only this: the recording picks the largest logit of every row, so
                # that one copy brings the ids to the host.  A decode step writes them where its own token
                # ids stand: replayed again for the same requests it decodes on, whether or not the host
                # has looked at the tokens yet.
                if kind == "s":
                    # the step draws by itself: temperature, top-k, top-p and the uniform number of every row come
                    # with the step's tables, and the token drawn lands where the largest logit's would
                    amax = gpu.draw(logits, self._shared_work()[:size], ctx.draw, *self._draw_constants(), meta[0:size], *flags)
                else:
                    amax = gpu.argmax(logits, out=meta[0:size]) if decode else gpu.argmax(logits)
            return logits, amax

        graph, (logits, amax) = gpu.capture(run)
        if ctx.tile_sizes_asked - set(tiles):
            self._unrecordable.add(key)       # the recorded run asked for tiles the eager run did not: not the same step
            return None
        if K.library_calls() != calls_before and not self._replays_faithfully(graph, logits, warm, meta, staging, rewind):
            # a library routine ran inside and its recorded nodes do not reproduce the eager result
            # (some record memory-clearing nodes that misbehave on replay): this shape runs eagerly
            self._unrecordable.add(key)
            return None
        if decode:
            meta.copy_(staging)               # the recording's trial replays have put their own tokens there
        stagings = [staging] + [gpu.pinned(torch.empty_like(staging)) for _ in range(self.STAGING_BUFFERS - 1)]
        rec = _RecordedStep(graph, meta, stagings, logits, ctx, [gpu.event() for _ in stagings])
        rec.greedy, rec.amax, rec.replayed, rec.tiles = greedy, amax, gpu.event(), tiles
        rec.held_bytes = max(0, gpu.reserved_bytes() - held_before) + meta.numel() * 4
        for done in rec.copied:
            done.record()
        self._recorded[key] = rec
        self._recorded_bytes += rec.held_bytes
        return rec

    def _shared_work(self) -> torch.Tensor:
        """Scratch of the sampling kernels of recorded steps, float32 [GRAPH_MAX_BATCH, vocabulary]: like the logits,
        one buffer for all recordings."""
        if self._work_buffer is None:
            self._work_buffer = torch.empty(self.GRAPH_MAX_BATCH, self.vocab_size, dtype=torch.float32, device=self.device)
        return self._work_buffer

    def _draw_constants(self):
        """(a penalty of 1 for every row, zeros: the empty lists of penalised tokens), for draws without a penalty."""
        if self._draw_consts is None:
            self._draw_consts = (torch.ones(self.GRAPH_MAX_BATCH, dtype=torch.float32, device=self.device),
                                 torch.zeros(self.GRAPH_MAX_BATCH + 1, dtype=torch.int32, device=self.device))
        return self._draw_consts

    def _shared_logits(self) -> torch.Tensor:
        if self._logits_buffer is None:
            self._logits_buffer = torch.empty(self.GRAPH_MAX_BATCH, self.vocab_size, dtype=torch.float32, device=self.device)
        return self._logits_buffer

    def _drop_recordings(self) -> None:
        """Keep the recordings within their bounds: decode shapes by number, all of them together by the
        device memory they hold; the ones used longest ago go first (the newest always stays)."""
        decodes = [k for k in self._recorded if k[0] in ("d", "s")]
        for old in decodes[:max(0, len(decodes) - self.GRAPH_MAX_DECODES)]:
            self._recorded_bytes -= self._recorded.pop(old).held_bytes
        for old in list(self._recorded)[:-1]:
            if self._recorded_bytes <= self.GRAPH_MAX_BYTES:
                break
            self._recorded_bytes -= self._recorded.pop(old).held_bytes

    def _written_rows(self, ctx: StepContext) -> torch.Tensor:
        """The keys and values that a step has written, of every cache, gathered into one tensor:
        all that a step which returns no logits leaves behind."""
        parts = []
        ps = self.page_size
        for gi, g in enumerate(self.cache.groups):
            slots = ctx.groups[gi].slot_mapping.long()
            pages, offs = slots // ps, slots % ps
            for cid in g.cache_ids:
                parts.append(g.kpools[cid][pages, :, offs].float().reshape(-1))
                parts.append(g.vpools[cid][pages, :, offs].float().reshape(-1))
        return torch.cat(parts) if parts else torch.zeros(1, device=self.device)

    def _state_rows(self, ctx: StepContext) -> List[torch.Tensor]:
        """The per-request state of the step's sequences, of every cache that holds state."""
        slots = ctx.per_seq.state_slot.long()
        return [t[slots].float().reshape(-1) for _, t in sorted(self.cache.state.items())]

    def _replays_faithfully(self, graph, logits, warm: StepContext, meta: torch.Tensor, staging: torch.Tensor,
                            rewind=lambda: None, rounds: int = 3) -> bool:
        """Replay a fresh recording several times, with the same step run eagerly and a
        synchronisation between the replays, and compare every replay with the eager run: the
        logits, or for a step that returns none the keys and values it wrote; and the per-request
        state it leaves, if the model has any.  Keys and values are simply written again by every
        run; state is put back before each (``rewind``) and at the end.  (The tables are uploaded
        anew each time: a recorded decode step overwrites its token ids with the ones it has chosen.)"""
        gpu = self.gpu

        def left_behind(out):
            parts = [out.reshape(-1)] if out is not None else [self._written_rows(warm)]
            return torch.cat(parts + self._state_rows(warm)).clone()

        ok = True
        for _ in range(rounds):
            meta.copy_(staging)
            rewind()
            graph.replay()
            gpu.synchronize()
            got = left_behind(logits)
            rewind()
            want = left_behind(self.model.forward(warm, self._layer_cache(warm)))
            gpu.synchronize()
            scale = float(want.abs().max())
            if not bool(torch.isfinite(got).all()) or float((got - want).abs().max()) > 1e-3 * max(scale, 1e-30):
                ok = False
                break
        rewind()
        return ok

    def _replay(self, key, entries: List[StepEntry], tokens_from: Optional[_RecordedStep] = None,
                history_row: Optional[int] = None, pick=None, draw_rows=None) -> bool:
        """Run the entries through the recording of their shape (made now if there is none).  False:
        this shape cannot be recorded and the step has not run.  The logits are left in
        ``self._replayed_logits``.

        ``tokens_from``: the token ids of the entries are not known to the host; they are what the
        last replay of that recording (a decode step over the same requests in the same order)
        chose, and are taken from where it left them on the device.  ``history_row``: the tokens
        this replay chooses are also copied to that row of ``self._history`` (pinned host memory),
        and its logits are not kept.  ``pick(logits, out)``: launched behind the replay, it puts other
        tokens than the largest logits where the step leaves its choice.  ``draw_rows``: the table of the
        draw that a step of kind "s" makes itself (int32 [4 B])."""
        rec = self._recorded.pop(key, None)
        if rec is None:
            rec = self._record(key, entries, draw_rows=draw_rows)
            if rec is None:
                return False
            self._drop_recordings()
            # the recording itself has left nothing behind: fall through to the first replay
        else:
            self._recorded[key] = rec          # moved to the end: the most recently used
        kind, B, width = key[0], key[1], key[2]
        decode = kind in ("d", "s")
        if (kind == "s") != (draw_rows is not None):
            raise StepError("a step that draws needs the draw's table, and only such a step takes one")
        ps = self.page_size
        order = tuple(e.request for e in entries)
        if tokens_from is not None and not (decode and order == rec.order):
            # refused before anything is changed: the caller's books and this recording's stay as they were
            raise StepError("tokens can stay on the device only between decode steps over the same requests")
        # the tables are written into the next staging buffer in turn, starting from those of the last replay
        last = rec.stagings[rec.turn]
        rec.turn = (rec.turn + 1) % len(rec.stagings)
        rec.copied[rec.turn].synchronize()          # the upload that last used this buffer has read it
        staging = rec.stagings[rec.turn]
        st = staging.numpy()                        # shares the pinned memory
        totals = []
        if decode and order == rec.order:
            # the same requests in the same places as last time: tokens, positions and slots change,
            # block tables only grow at their ends
            st[:] = last.numpy()
            for b, e in enumerate(entries):
                done = self._done[e.request]
                st[b] = int(e.tokens[0])
                st[B + b] = done
                totals.append(done + 1)
            off_ctx = rec.layout.seq + 2 * B
            st[off_ctx:off_ctx + B] = totals
            if draw_rows is not None:
                st[rec.layout.draw:rec.layout.draw + 4 * B] = draw_rows
            for gi, g in enumerate(self.cache.groups):
                off_slot, off_table, _ = rec.layout.groups[gi]
                written = rec.pages_written[gi]
                for b, e in enumerate(entries):
                    table = g.tables[e.request]
                    n = len(table)
                    if n != written[b]:
                        row = off_table + b * width
                        st[row + written[b]:row + n] = table[written[b]:n]
                        written[b] = n
                    done = totals[b] - 1
                    st[off_slot + b] = table[done // ps] * ps + done % ps
        else:
            ctx = StepContext(self.device)
            flat, layout, _, tiles = self._tables_of(entries, ctx, width, rec.tiles or (), draw_rows=draw_rows)
            if len(flat) != staging.numel() or tiles != (rec.tiles or {}):
                raise StepError("a recorded step was asked to run another shape")
            st[:] = flat
            rec.layout = layout
            rec.order = order if decode else ()
            rec.pages_written = [[len(g.tables[e.request]) for e in entries] for g in self.cache.groups]
            totals = ctx._host["context_len"]
        if tokens_from is None:
            rec.meta.copy_(staging, non_blocking=True)
        else:
            # everything but the token ids, which are on the device already: in this recording's own
            # tables if it ran last, else in the other recording's choice
            rec.meta[B:].copy_(staging[B:], non_blocking=True)
            if tokens_from is not rec:
                rec.meta[0:B].copy_(tokens_from.amax[0:B], non_blocking=True)
        rec.copied[rec.turn].record()
        rec.graph.replay()
        if pick is not None:
            pick(rec.logits, rec.amax[0:B])
        self._last_context_len = totals
        if history_row is not None:
            self._history[history_row, 0:B].copy_(rec.amax[0:B], non_blocking=True)
            self._replayed_logits = None
            return True
        if rec.logits is None:
            self._replayed_logits = None
        else:
            rec.greedy.copy_(rec.amax, non_blocking=True)
            out = rec.logits.clone()      # the graph's own buffer is overwritten by its next replay
            self._greedy_of = (out, rec)
            self._replayed_logits = out
        rec.replayed.record()
        return True

    def _span(self):
        """An event recorded now, and a function that records its partner and notes the pair in
        ``self.timeline``; (None, no-op) when nobody measures."""
        if self.timeline is None:
            return None, lambda: None
        first = torch.cuda.Event(enable_timing=True)
        first.record()

        def close():
            last = torch.cuda.Event(enable_timing=True)
            last.record()
            self.timeline.append((first, last))
        return first, close

    def _book(self, entries: List[StepEntry], totals: Sequence[int]) -> None:
        for e, total in zip(entries, totals):
            self._done[e.request] = total
            self.cache.release_passed(e.request, total)

    def step(self, entries: Sequence[StepEntry], end: Iterable[Hashable] = ()) -> Optional[torch.Tensor]:
        """Run one batch.  Returns float32 logits ``[wanted, vocab]`` on the device, rows in the
        order of the entries and of each entry's ``want`` (None when nothing is wanted).  Requests
        named in ``end`` give back what they hold after the step."""
        entries = list(entries)
        logits = None
        self._greedy_of = None
        if entries:
            self._check_and_reserve(entries)
            key = self._graph_shape(entries)
            totals = None
            _, close = self._span()
            if key is not None and self._replay(key, entries):
                logits = self._replayed_logits
                totals = self._last_context_len
            if totals is None:
                ctx = StepContext(self.device, scratch_owner=self)
                flat, layout, n_rows = self._describe(entries, ctx)
                self._bind(ctx, self._upload(flat), layout, n_rows)
                logits = self.model.forward(ctx, self._layer_cache(ctx))
                totals = ctx._host["context_len"]
            close()
            self._book(entries, totals)
        for r in end:
            self.release(r)
        return logits

    takes_draw_tables = True      # decode_run(..., draw=) exists: recorded decode steps can make the draw themselves

    def _draw_eager(self, logits: torch.Tensor, draw, i: int) -> List[int]:
        """Draw ``i`` of the tables ``draw`` over ``logits``, launched the ordinary way."""
        B = logits.shape[0]
        rows = torch.from_numpy(draw.rows(i)).to(self.device)
        as_float = rows[:3 * B].view(torch.float32)
        view = DrawView(as_float[0:B], as_float[B:2 * B], as_float[2 * B:3 * B], rows[3 * B:4 * B])
        out = torch.empty(B, dtype=torch.int32, device=self.device)
        self.gpu.draw(logits, torch.empty_like(logits), view, *self._draw_constants(), out, *draw.flags)
        return out.tolist()

    def decode_run(self, entries: Sequence[StepEntry], steps: int, pick=None, draw=None) -> List[List[int]]:
        """Decoding of ``steps`` tokens for every entry (one token each, wanting its logits):
        the first step takes the entries' tokens, every later one the tokens that the step before
        chose: the index of the largest logit, lowest index on ties; or with ``pick`` what
        ``pick(i, logits, out)`` launches into ``out`` (int32 [entries], on the device) for step
        ``i`` without waiting for anything; or with ``draw`` (a sampler's
        :class:`~nanoinfer_amd.sampling.sampler.DrawTables`: temperature, top-k, top-p and the uniform
        numbers of every step, no repetition penalty) what the sampling kernels draw, which are then part
        of the recorded step itself.  Returns the chosen tokens,
        ``[step][entry]``: what ``steps`` calls of :meth:`step` with :meth:`greedy_tokens` between
        them return.  Where recordings of the steps' shapes exist, the steps are launched back to
        back, the tokens passing from one to the next on the device, and the host waits once at
        the end: the GPU is not idle while the host reads a token and launches the next step.
        A shape without a recording runs the ordinary way (which records it)."""
        entries = list(entries)
        if any(len(e.tokens) != 1 or list(e.want) != [0] for e in entries):
            raise StepError("decode_run takes entries of one token each that want its logits")
        if pick is not None and draw is not None:
            raise StepError("decode_run takes pick or draw, not both")
        B = len(entries)
        chosen: List[List[int]] = []
        tokens: Optional[List[int]] = [int(e.tokens[0]) for e in entries]     # None: still on the device
        launched = 0                # replays whose tokens the host has not read yet
        last: Optional[_RecordedStep] = None
        self._greedy_of = None
        if self._history is None:
            self._history = self.gpu.pinned(torch.zeros(self.HISTORY_ROWS, self.GRAPH_MAX_BATCH, dtype=torch.int32))
            self._history_done = self.gpu.event()

        def collect() -> None:
            nonlocal launched, tokens
            if launched:
                self._history_done.record()
                self._history_done.synchronize()
                rows = self._history[0:launched, 0:B].tolist()
                chosen.extend(rows)
                tokens = rows[-1]
                launched = 0

        def the_ordinary_way(cur) -> None:
            nonlocal tokens, last
            logits = self.step(cur)
            if draw is not None:
                tokens = self._draw_eager(logits, draw, len(chosen))
            elif pick is None:
                tokens = self.greedy_tokens(logits)
            else:
                out = torch.empty(B, dtype=torch.int32, device=self.device)
                pick(len(chosen), logits, out)
                tokens = out.tolist()
            chosen.append(list(tokens))
            last = None

        order = tuple(e.request for e in entries)
        flags = None if draw is None else draw.flags
        for _ in range(int(steps)):
            cur = [StepEntry(e.request, [tokens[b] if tokens is not None else 0], [0]) for b, e in enumerate(entries)]
            key = self._graph_shape(cur, draw=flags) if B else None
            rec = self._recorded.get(key) if key is not None else None
            # a step that draws by itself is recorded by its first replay here (the ordinary way records the other kind)
            to_record = draw is not None and key is not None and rec is None
            if rec is None or rec.amax is None or launched == self.HISTORY_ROWS or \
                    (tokens is None and rec.order != order):
                # also when the run passes into a recording of another shape (a longer context, a wider
                # table) that last ran other requests: its tables are written anew, from tokens the host knows
                collect()
                cur = [StepEntry(e.request, [tokens[b]], [0]) for b, e in enumerate(entries)]
            if (rec is None and not to_record) or (rec is not None and rec.amax is None):
                the_ordinary_way(cur)
                continue
            self._check_and_reserve(cur)
            at = len(chosen) + launched
            _, close = self._span()
            ran = self._replay(key, cur, tokens_from=last if tokens is None else None, history_row=launched,
                               pick=None if pick is None else (lambda logits, out, at=at: pick(at, logits, out)),
                               draw_rows=None if draw is None else draw.rows(at))
            close()
            if not ran:               # the shape cannot be recorded
                the_ordinary_way(cur)
                continue
            self._book(cur, self._last_context_len)
            launched += 1
            tokens = None
            last = self._recorded[key]
        collect()
        return chosen
