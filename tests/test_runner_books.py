"""The runner's host side without a GPU: the real ``decode_run``, ``_replay``, ``_graph_shape`` and cache
books, over a recording whose graph is a stand-in that "chooses" the next token by a formula.  Every
replay checks the tables it was given against the cache manager's books."""
from types import SimpleNamespace

import pytest
import torch

from nanoinfer_amd.cache.manager import KVCacheManager
from nanoinfer_amd.engine.runner import ModelRunner, StepContext, StepEntry, StepError, _RecordedStep
from nanoinfer_amd.parts.base import CacheNeed, KVNeed, StateNeed

VOCAB = 97


def next_token(token: int, position: int) -> int:
    return (token * 31 + position * 7 + 1) % VOCAB


class _Event:
    def record(self):
        pass

    def synchronize(self):
        pass


class _Graph:
    """Stands for a recorded decode step: reads its tables, checks them, leaves its choice where the
    token ids stood."""

    def __init__(self, runner, rec_of):
        self.runner, self.rec_of, self.replays = runner, rec_of, 0

    def replay(self):
        rec = self.rec_of()
        r, B = self.runner, len(rec.order)
        meta = rec.meta
        (off_slot, off_table, width) = rec.layout.groups[0]
        g = r.cache.groups[0]
        ps = r.page_size
        for b, request in enumerate(rec.order):
            pos = int(meta[B + b])
            assert pos == r._done[request], "position of the replay is the request's next one"
            table = g.tables[request]
            assert int(meta[off_slot + b]) == table[pos // ps] * ps + pos % ps
            row = meta[off_table + b * width: off_table + (b + 1) * width].tolist()
            assert row[:len(table)] == table and all(x == -1 for x in row[len(table):])
            per_seq = meta[rec.layout.seq: rec.layout.seq + 4 * B].view(4, B)[:, b].tolist()
            assert per_seq == [b, 1, pos + 1, r.cache.state_slot(request)], "the per-sequence table of the replay"
            meta[b] = next_token(int(meta[b]), pos)
        rec.logits.zero_()
        for b in range(B):
            rec.logits[b, int(meta[b])] = 1.0
        self.replays += 1


def make_runner(page_size=8, num_pages=200, max_requests=8):
    r = object.__new__(ModelRunner)
    r.device = torch.device("cpu")
    r.page_size = page_size
    r.cache = KVCacheManager({0: CacheNeed(kv=KVNeed(1, 16))}, page_size, num_pages, max_requests, device=None)
    r.vocab_size = VOCAB
    r.model = SimpleNamespace(max_positions=8192, graph_safe=lambda: True)
    r.max_positions = 8192
    r._done = {}
    r._scratch = None
    r._init_graphs(True)
    r._history = torch.zeros(r.HISTORY_ROWS, r.GRAPH_MAX_BATCH, dtype=torch.int32)
    r._history_done = _Event()
    r.recordings_made = []

    def record(key, entries, draw_rows=None):
        kind, size, pages, bound, _ = key
        assert kind == "d" and draw_rows is None
        ctx = StepContext(r.device, recording=True)
        flat, layout, n_rows, tiles = r._tables_of(entries, ctx, pages, ())
        staging = torch.tensor(flat, dtype=torch.int32)
        meta = staging.clone()
        holder = {}
        rec = _RecordedStep(_Graph(r, lambda: holder["rec"]), meta,
                            [staging] + [torch.empty_like(staging) for _ in range(r.STAGING_BUFFERS - 1)],
                            torch.zeros(size, VOCAB), ctx, [_Event() for _ in range(r.STAGING_BUFFERS)])
        rec.greedy = torch.zeros(size, dtype=torch.int32)
        rec.amax, rec.replayed, rec.tiles = meta[0:size], _Event(), tiles
        holder["rec"] = rec
        r._recorded[key] = rec
        r.recordings_made.append(key)
        return rec

    r._record = record
    r.greedy_tokens = lambda logits: logits.argmax(dim=1).tolist()
    return r


def start(r, request, context):
    """A request whose first ``context`` tokens are in the cache already."""
    assert r.cache.reserve(request, context)
    r._done[request] = context


def expected(first_tokens, contexts, steps):
    toks, out = list(first_tokens), []
    for k in range(steps):
        toks = [next_token(t, c + k) for t, c in zip(toks, contexts)]
        out.append(list(toks))
    return out


def run_wave(r, names, context, first_tokens, steps, run):
    got = []
    toks = list(first_tokens)
    left = steps
    while left:
        k = min(run, left)
        rows = r.decode_run([StepEntry(n, [t], [0]) for n, t in zip(names, toks)], k)
        assert len(rows) == k
        got.extend(rows)
        toks = rows[-1]
        left -= k
    assert got == expected(first_tokens, [context] * len(names), steps)
    for n in names:
        assert r._done[n] == context + steps == r.cache.num_tokens(n)


def test_a_second_wave_of_requests_crosses_a_context_bucket_inside_a_run():
    """Two requests decode in runs of eight from context 252: the run passes from the recording
    for contexts up to 256 into the one for up to 512.  A second pair of fresh requests does the
    same afterwards, when both recordings exist and hold the first pair's tables."""
    r = make_runner(page_size=16)
    for wave, names in enumerate((("a", "b"), ("c", "d"), ("e", "f"))):
        for n in names:
            start(r, n, 252)
        run_wave(r, names, 252, [3 + wave, 50 + wave], steps=24, run=8)
        for n in names:
            r.release(n)
        r.cache.check()
    assert len(r.recordings_made) == 2       # one per bucket, made by the first wave only
    assert r.cache.free_pages() == r.cache.num_pages


def test_a_second_wave_crosses_a_page_bucket_inside_a_run():
    """Pages of 8 tokens: the table's width passes from 16 to 32 pages at 128 tokens while the
    context bound stays."""
    r = make_runner(page_size=8)
    for wave, names in enumerate((("a", "b", "c"), ("d", "e", "f"))):
        for n in names:
            start(r, n, 123)
        run_wave(r, names, 123, [1, 2, 3 + wave], steps=16, run=8)
        for n in names:
            r.release(n)
    assert {k[2] for k in r.recordings_made} == {16, 32}


def test_the_same_requests_in_another_order_get_their_tables_written_anew():
    r = make_runner(page_size=16)
    for n in ("a", "b"):
        start(r, n, 40)
    run_wave(r, ("a", "b"), 40, [5, 6], steps=8, run=4)
    got = r.decode_run([StepEntry("b", [9], [0]), StepEntry("a", [11], [0])], 4)
    assert got == expected([9, 11], [48, 48], 4)


def test_tokens_on_the_device_are_refused_before_anything_changes():
    """``_replay`` with ``tokens_from`` for other requests than the recording's last: an error, and
    neither the recording's turn nor the books have moved."""
    r = make_runner(page_size=16)
    for n in ("a", "b", "c", "d"):
        start(r, n, 40)
    run_wave(r, ("a", "b"), 40, [5, 6], steps=2, run=2)
    key = r.recordings_made[0]
    rec = r._recorded[key]
    turn, books = rec.turn, dict(r._done)
    with pytest.raises(StepError):
        r._replay(key, [StepEntry("c", [0], [0]), StepEntry("d", [0], [0])], tokens_from=rec, history_row=0)
    assert rec.turn == turn and r._done == books


def test_decode_recordings_are_kept_up_to_a_limit_and_the_least_recently_used_goes_first():
    r = make_runner(page_size=16)
    r.GRAPH_MAX_DECODES = 2
    for n in ("a", "b"):
        start(r, n, 250)
    run_wave(r, ("a", "b"), 250, [5, 6], steps=8, run=4)            # shapes for contexts up to 256 and up to 512
    first, second = r.recordings_made
    assert list(r._recorded) == [first, second]
    start(r, "c", 10)
    run_wave(r, ("c",), 10, [7], steps=2, run=2)                     # a third shape: the first, used longest ago, goes
    third = r.recordings_made[-1]
    assert list(r._recorded) == [second, third]
    run_wave(r, ("a", "b"), 258, [1, 2], steps=2, run=2)             # the second is used again: now the newest
    assert list(r._recorded) == [third, second]
    for n in ("d", "e"):
        start(r, n, 100)
    run_wave(r, ("d", "e"), 100, [3, 4], steps=2, run=2)             # the first shape comes back: recorded again
    assert r.recordings_made[-1] == first and list(r._recorded) == [second, first]


# ------------------------------------------------------------------ the real recording, over a model with state

class _HostServices:
    """The device services of the runner for a run without a GPU: nothing to wait for, ordinary memory,
    and a "graph" that runs its step anew at every replay (as a HIP graph launches its kernels anew).
    While a step is captured nothing is executed, as on the GPU: the model is told to give its buffers only."""

    def __init__(self, model):
        self.model = model

    synchronize = staticmethod(lambda: None)
    pinned = staticmethod(lambda t: t)
    event = staticmethod(_Event)
    reserved_bytes = staticmethod(lambda: 0)

    @staticmethod
    def argmax(logits, out=None):
        ids = logits.argmax(dim=1).to(torch.int32)
        if out is None:
            return ids
        out.copy_(ids)
        return out

    @staticmethod
    def draw(logits, work, view, ones, zeros, out, uses_top_k, uses_top_p):
        """Stands for the sampling kernels: the largest logit's index moved on by what the row's table says, so
        that a test sees whether every step's own table has reached the step."""
        R = logits.shape[0]
        assert float(ones[:R].min()) == 1.0 and int(zeros[:R + 1].abs().max()) == 0 and not uses_top_p
        shift = (view.uniform * 64).round().to(torch.int32) + view.top_k + (view.temperature * 8).round().to(torch.int32)
        out.copy_((logits.argmax(dim=1).to(torch.int32) + shift) % VOCAB)
        return out

    def capture(self, run):
        self.model.dry = True
        try:
            result = run()
        finally:
            self.model.dry = False
        return SimpleNamespace(replay=run), result


class _CountingModel:
    """Stands for a model with a mixer that updates a per-request state in place: every run of a step
    adds one to the state of each of its sequences, and "chooses" the next token by the formula.  It
    reads its step from the device tables only, and counts as a step with a library product inside,
    so that a fresh recording is tried against eager runs before it is used."""

    max_positions = 8192

    def __init__(self, cache, idempotent_says):
        self.cache, self.dry, self.says = cache, False, idempotent_says
        self.buffers = {}

    def graph_safe(self):
        return True

    def idempotent(self):
        return self.says

    def forward(self, ctx, layer_cache, logits_out=None):
        from nanoinfer_amd import kernels as K
        B = ctx.n_seqs
        logits = self.buffers.setdefault(id(ctx), torch.zeros(B, VOCAB))
        K._library_calls += 1
        if self.dry:
            return logits
        slots = ctx.per_seq.state_slot.long()
        self.cache.state[0][slots] += 1.0
        tokens = (ctx.token_ids[:B].long() * 31 + ctx.positions[:B].long() * 7 + 1) % VOCAB
        logits.zero_()
        logits[torch.arange(B), tokens] = 1.0
        return logits


def make_state_runner(idempotent_says):
    r = object.__new__(ModelRunner)
    r.device = torch.device("cpu")
    r.page_size = 16
    r.max_step_tokens = None
    r.cache = KVCacheManager({0: CacheNeed(kv=KVNeed(1, 16), state=StateNeed((1,)))}, 16, 64, 8, device=r.device)
    r.vocab_size = VOCAB
    r.model = _CountingModel(r.cache, idempotent_says)
    r.gpu = _HostServices(r.model)
    r.max_positions = 8192
    r._done = {}
    r._scratch = None
    r._init_graphs(True)
    return r


def test_a_state_advances_once_for_every_booked_step_also_while_steps_are_recorded():
    """Recording a step runs it several times: once the ordinary way, then in trial replays beside eager
    runs.  A model that says its step is not idempotent finds its per-request state put back in between,
    so that after n booked steps the state has moved n times, whether a step was run eagerly, recorded
    just then, or replayed; and the tokens are those of the formula."""
    r = make_state_runner(idempotent_says=False)
    names, first = ("a", "b", "c"), [3, 50, 7]
    r.step([StepEntry(n, [1] * 5, []) for n in names])                  # prompts: an eager step
    booked = 1
    toks = list(first)
    got = []
    for _ in range(3):                                                  # single steps: the first one records
        toks = r.greedy_tokens(r.step([StepEntry(n, [t], [0]) for n, t in zip(names, toks)]))
        got.append(list(toks))
        booked += 1
        for n in names:
            assert float(r.cache.state[0][r.cache.state_slot(n)]) == booked
    assert len(r._recorded) == 1
    rows = r.decode_run([StepEntry(n, [t], [0]) for n, t in zip(names, toks)], 6)     # and a run of replays
    got.extend(rows)
    booked += 6
    assert got == expected(first, [5, 5, 5], 9)
    for n in names:
        assert float(r.cache.state[0][r.cache.state_slot(n)]) == booked


def test_without_that_declaration_the_recording_would_move_the_state():
    """The same model calling itself idempotent: the runs of the recording all land in the state.  (What
    the test above guards against; here it shows that the stand-in can tell the difference.)"""
    r = make_state_runner(idempotent_says=True)
    r.step([StepEntry("a", [1] * 5, [])])
    r.step([StepEntry("a", [3], [0])])
    assert float(r.cache.state[0][r.cache.state_slot("a")]) > 2


def test_host_lists_cannot_be_read_while_a_step_is_recorded():
    ctx = StepContext(torch.device("cpu"), recording=True)
    ctx._host["q_len"].append(1)
    assert ctx.q_len == [1]
    ctx.seal()
    with pytest.raises(StepError, match="per_seq"):
        ctx.q_len


def test_steps_that_draw_by_themselves_get_their_own_table_every_step():
    """``decode_run(..., draw=tables)``: the draw is part of the recorded step, and what it reads (temperature,
    top-k, top-p, and the uniform number of that very step) travels with the step's tables.  The stand-in draw
    moves the token on by what its table says; the tokens follow, through the first steps that record the
    shapes, a run across a context bound into another recording, and single eager steps when recording is off."""
    from nanoinfer_amd.sampling.params import SamplingParams
    from nanoinfer_amd.sampling.sampler import DrawTables
    params = [SamplingParams(temperature=0.5, top_k=3, seed=11), SamplingParams(temperature=1.0, top_k=0, seed=12)]

    def expect(first, context, generated, steps):
        toks, out = list(first), []
        for k in range(steps):
            nxt = []
            for b, (t, p) in enumerate(zip(toks, params)):
                from nanoinfer_amd.sampling.sampler import uniform_from_counter
                u = uniform_from_counter(p.seed, generated + k)
                shift = round(float(torch.tensor(u, dtype=torch.float32) * 64)) + (p.top_k if p.top_k > 0 else 0) + round(p.temperature * 8)
                nxt.append((next_token(t, context + k) + shift) % VOCAB)
            toks = nxt
            out.append(list(toks))
        return out

    for graphs in (True, False):
        r = make_state_runner(idempotent_says=False)
        r.use_graphs = graphs
        names, first = ("a", "b"), [3, 50]
        r.step([StepEntry(n, [1] * 250, []) for n in names])
        generated = [[] for _ in names]
        toks, got, done = list(first), [], 0
        for k in (3, 8, 5):                    # the second run crosses the bound of 256 tokens
            tables = DrawTables(params, generated, k)
            assert tables.flags == (True, False)
            rows = r.decode_run([StepEntry(n, [t], [0]) for n, t in zip(names, toks)], k, draw=tables)
            assert rows == expect(toks, 250 + done, done, k), (graphs, done)
            for row in rows:
                for g, t in zip(generated, row):
                    g.append(t)
            toks, done = rows[-1], done + k
        assert ({key[0] for key in r._recorded} == {"s"} and len(r._recorded) == 2) if graphs else not r._recorded
        for n in names:                        # and the state moved once a step
            assert float(r.cache.state[0][r.cache.state_slot(n)]) == 1 + done
    with pytest.raises(ValueError, match="repetition penalty"):
        DrawTables([SamplingParams(temperature=1.0, repetition_penalty=1.2)], [[]], 2)
