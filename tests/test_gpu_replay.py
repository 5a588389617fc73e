"""Replay of the same requests cut in different ways, in float32 and bfloat16, against the plain
implementation: whole; most in one step and the last 32 tokens one by one; portions of changing
size down to two tokens; mixed with other requests on so few pages that they are used again.
Driven through ModelRunner.step in-process, and through bin/trace_run as a user would."""
import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

from gpu_common import TOL, assert_close, model_folder, plain_logits, random_tokens
from tiny_configs import ALL

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PAGE = {"A": 16, "B": 8, "C": 4}
LENGTHS = {"A": (7, 19, 33, 70), "B": (1, 40, 77, 130, 200), "C": (2, 50, 65, 97)}


# ------------------------------------------------------------------ traces

def whole(requests):
    return [([(rid, list(toks), list(range(len(toks))))], [rid]) for rid, toks in requests.items()]


def tail_one_by_one(requests, tail=32):
    steps = []
    for rid, toks in requests.items():
        n = len(toks)
        head = max(1, n - tail)
        steps.append(([(rid, list(toks[:head]), list(range(head)))], []))
        for i in range(head, n):
            steps.append(([(rid, [toks[i]], [0])], [rid] if i == n - 1 else []))
        if head == n:
            steps[-1] = (steps[-1][0], [rid])
    return steps


def changing_portions(requests, sizes=(7, 2, 13, 3, 2, 29, 5, 2, 64, 11)):
    steps = []
    for rid, toks in requests.items():
        at, k = 0, 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            if len(toks) - at - n == 1:      # never leave a single token: the smallest portion is two
                n += 1
            k += 1
            steps.append(([(rid, list(toks[at:at + n]), list(range(n)))], [rid] if at + n == len(toks) else []))
            at += n
    return steps


def mixed(requests, seed, max_live=4):
    """Up to ``max_live`` requests at a time: some bring a portion of their prompt (a random first
    part of the request counts as prompt), others single tokens; a request may sit a step out."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}     # rid -> [tokens, done, prompt_len]
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            rid, toks = waiting.pop(0)
            live[rid] = [list(toks), 0, rng.randint(1, len(toks))]
        entries, ended = [], []
        for rid in list(live):
            toks, done, plen = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                      # left out of this step, goes on later
            if done < plen:
                n = min(plen - done, rng.choice([2, 3, 5, 8, 17, 40]))
                if plen - done - n == 1 and done + n + 1 <= len(toks):
                    n += 1
            else:
                n = 1
            want = sorted(rng.sample(range(n), rng.randint(0, n))) if n > 1 else [0]
            entries.append((rid, toks[done:done + n], want))
            live[rid][1] = done + n
            if done + n == len(toks):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append((entries, ended))
    return steps


def max_live_tokens(steps, requests, page):
    """The most tokens live requests hold at once, each rounded up to a multiple of 64."""
    held, worst = {}, 0
    for entries, ended in steps:
        for rid, toks, _ in entries:
            held[rid] = held.get(rid, 0) + len(toks)
        worst = max(worst, sum(-(-n // 64) * 64 for n in held.values()))
        for rid in ended:
            del held[rid]
    return worst


def run_in_process(folder, dtype, page, steps, max_tokens, seen=None, **runner_options):
    """Replay ``steps`` through a runner of its own; ``seen`` (a dict) is told which shapes were recorded."""
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry

    runner = ModelRunner(folder, dtype=dtype, page_size=page, max_tokens=max_tokens, max_requests=4, **runner_options)
    got = {}
    given_back = set()      # pages that some finished request held
    reused = False
    for entries, ended in steps:
        out = runner.step([StepEntry(r, t, w) for r, t, w in entries], end=())
        row = 0
        for r, t, w in entries:
            reused = reused or any(p in given_back for p in runner.cache.block_table(0, r))
            base = runner.computed_tokens(r) - len(t)
            for i in w:
                got[(r, base + i)] = out[row].clone()
                row += 1
        assert (out is None and row == 0) or out.shape[0] == row
        for r in ended:
            given_back.update(runner.cache.block_table(0, r))
            runner.release(r)
    runner.cache.check()
    assert runner.cache.free_pages() == runner.cache.num_pages and not runner.cache.live_requests()
    if seen is not None:
        seen["recorded"], seen["unrecordable"] = list(runner._recorded), set(runner._unrecordable)
        seen["memory"] = runner.memory_report()
    return got, reused


def compare(got, requests, folder, dtype, what):
    assert got, "nothing was compared"
    by_request = {}
    for (rid, pos), row in got.items():
        by_request.setdefault(rid, []).append((pos, row))
    for rid, rows in by_request.items():
        want = plain_logits(folder, tuple(requests[rid]), dtype)
        rows.sort(key=lambda x: x[0])
        idx = [p for p, _ in rows]
        assert_close(torch.stack([r for _, r in rows]), want[idx], dtype, f"{what}, request {rid}, positions {idx[0]}..{idx[-1]}")


def make_requests(name, seed=0):
    vocab = ALL[name]["vocab_size"]
    return {f"r{i}": random_tokens(vocab, n, seed * 100 + i) for i, n in enumerate(LENGTHS[name])}


# ------------------------------------------------------------------ tests

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_each_request_alone_and_whole(name, dtype):
    folder, requests = model_folder(name), make_requests(name)
    steps = whole(requests)
    got, _ = run_in_process(folder, dtype, PAGE[name], steps, max_live_tokens(steps, requests, PAGE[name]))
    assert len(got) == sum(len(t) for t in requests.values())
    compare(got, requests, folder, dtype, f"{name} whole")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_last_32_tokens_one_by_one(name, dtype):
    folder, requests = model_folder(name), make_requests(name)
    steps = tail_one_by_one(requests)
    got, _ = run_in_process(folder, dtype, PAGE[name], steps, max_live_tokens(steps, requests, PAGE[name]))
    assert len(got) == sum(len(t) for t in requests.values())
    compare(got, requests, folder, dtype, f"{name} tail")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_portions_of_changing_size(name, dtype):
    folder, requests = model_folder(name), make_requests(name)
    steps = changing_portions(requests)
    assert min(len(t) for e, _ in steps for _, t, _ in e if len(t) > 1) == 2
    got, _ = run_in_process(folder, dtype, PAGE[name], steps, max_live_tokens(steps, requests, PAGE[name]))
    compare(got, requests, folder, dtype, f"{name} portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_requests_on_few_pages(name, dtype):
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    lengths = list(LENGTHS[name]) + [23, 64, 5, 48, 100]
    requests = {f"m{i}": random_tokens(vocab, n, 500 + i) for i, n in enumerate(lengths)}
    steps = mixed(requests, seed=11)
    assert max(len(e) for e, _ in steps) == 4                          # four live at once did happen
    assert any(len(e) > 1 and any(len(t) > 1 for _, t, _ in e) and any(len(t) == 1 for _, t, _ in e) for e, _ in steps)
    got, reused = run_in_process(folder, dtype, PAGE[name], steps, max_live_tokens(steps, requests, PAGE[name]))
    assert reused, "the pool was large enough that no page was used twice"
    compare(got, requests, folder, dtype, f"{name} mixed")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("B", 12), ("C", 5), ("A", 1)])
def test_pages_whose_size_is_no_power_of_two(name, page, dtype):
    """The mixed trace again with pages of 12, 5 and 1 slots: page and slot of a position come from
    a division, not a shift, in the cache books and in every kernel that walks a block table."""
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    requests = {f"p{i}": random_tokens(vocab, n, 900 + i) for i, n in enumerate([37, 70, 9, 25, 61])}
    steps = mixed(requests, seed=5)
    got, reused = run_in_process(folder, dtype, page, steps, max_live_tokens(steps, requests, page))
    assert reused
    compare(got, requests, folder, dtype, f"{name} pages of {page}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype, monkeypatch):
    """A short prompt, then some four hundred tokens one at a time: positions far beyond the prompt,
    many page boundaries, the split key range of the decode path."""
    name = "B"
    folder = model_folder(name)
    toks = random_tokens(ALL[name]["vocab_size"], 420, 77)
    steps = [([("long", list(toks[:3]), [0, 1, 2])], [])]
    steps += [([("long", [t], [0])], []) for t in toks[3:]]
    steps[-1] = (steps[-1][0], ["long"])
    from nanoinfer_amd import kernels as K
    merged, original = [], K.skinny_gemm_merged
    monkeypatch.setattr(K, "skinny_gemm_merged", lambda *a, **kw: (merged.append(a[1]), original(*a, **kw))[1])
    got, _ = run_in_process(folder, dtype, PAGE[name], steps, 448)
    compare(got, {"long": toks}, folder, dtype, "long decoding")
    # in bfloat16 the output product of a lone token merges the key runs itself once there are two of them
    assert (dtype == "bfloat16") == bool(merged) and set(merged) <= {2}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_of_a_sequence(name, dtype):
    """Position 0 alone, then 1, then 2: a context of one key, the first page's first slots."""
    folder = model_folder(name)
    toks = random_tokens(ALL[name]["vocab_size"], 4, 5)
    steps = [([("f", [t], [0])], []) for t in toks]
    got, _ = run_in_process(folder, dtype, PAGE[name], steps + [([], ["f"])], 64)
    compare(got, {"f": toks}, folder, dtype, "first tokens")
    steps = [([("g", list(toks[:1]), [0]), ("h", list(toks[:2]), [0, 1])], ["g", "h"])]
    got, _ = run_in_process(folder, dtype, PAGE[name], steps, 128)
    compare(got, {"g": toks[:1], "h": toks[:2]}, folder, dtype, "two short requests")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_copy_of_every_matrix_gives_the_same_logits(dtype):
    """``one_weight_copy``: no layer matrix gets the re-tiled copy that the products of decode steps stream; they
    read the rows as stored, and norms and residual sums run as kernels of their own.  Device memory then holds
    the checkpoint once (by default nearly twice); the logits of every way of cutting stay the plain ones."""
    name = "B"
    folder, requests = model_folder(name), make_requests(name)
    memory = {}
    for one_copy in (True, False):
        seen = {}
        for steps in (tail_one_by_one(requests), mixed(requests, seed=4)):
            got, _ = run_in_process(folder, dtype, PAGE[name], steps, max_live_tokens(steps, requests, PAGE[name]), seen=seen,
                                    one_weight_copy=one_copy)
            compare(got, requests, folder, dtype, f"{name}, one copy of the matrices: {one_copy}")
        memory[one_copy] = seen["memory"]
    assert memory[True]["weights"] <= 1.02 * memory[True]["checkpoint"] + (1 << 20)      # the rotation tables are the rest
    assert memory[False]["weights"] >= 1.5 * memory[False]["checkpoint"]


def test_stored_bfloat16_weights_give_the_same_logits_in_both_stores():
    """A folder stored in bfloat16 and run in float32 uses exactly the stored values."""
    folder = model_folder("A", stored="bfloat16")
    requests = {"x": random_tokens(256, 40, 3)}
    for dtype in ("float32", "bfloat16"):
        got, _ = run_in_process(folder, dtype, 16, whole(requests), 64)
        compare(got, requests, folder, dtype, f"stored bf16 run {dtype}")


# ------------------------------------------------------------------ the program, as a user runs it

def run_trace_program(folder, dtype, steps, max_tokens, out_dir, extra=()):
    lines = [json.dumps({"step": i, "entries": [{"id": r, "tokens": list(t), "want": list(w)} for r, t, w in entries],
                         "end": ended}) for i, (entries, ended) in enumerate(steps)]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out_dir,
           "--max-tokens", str(max_tokens), *extra]
    proc = subprocess.run(cmd, input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(steps))]
    return proc


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(dtype, tmp_path):
    name = "B"
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    requests = {f"t{i}": random_tokens(vocab, n, 900 + i) for i, n in enumerate((30, 64, 90, 12, 57, 101))}
    steps = mixed(requests, seed=5)
    out_dir = str(tmp_path / "out")
    run_trace_program(folder, dtype, steps, max_live_tokens(steps, requests, 16), out_dir)
    held, got = {}, {}
    for i, (entries, ended) in enumerate(steps):
        n_want = sum(len(w) for _, _, w in entries)
        path = os.path.join(out_dir, f"{i}.f32")
        if n_want == 0:
            assert not os.path.exists(path)
        else:
            data = np.fromfile(path, dtype="<f4").reshape(n_want, vocab)
        row = 0
        for r, t, w in entries:
            base = held.get(r, 0)
            for j in w:
                got[(r, base + j)] = torch.from_numpy(data[row].copy())
                row += 1
            held[r] = base + len(t)
    compare(got, requests, folder, dtype, "trace_run mixed")


# ------------------------------------------------------------------ recorded (HIP graph) decode steps

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_decode_steps_equal_eager_ones(dtype):
    """Decode steps are recorded once per shape and replayed.  Every replay is checked against a
    runner that records nothing, with eager work (prompt portions of other requests, requests
    coming and going, a changing batch size) and synchronisations between the replays."""
    from nanoinfer_amd import kernels as K
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry
    name = "B"
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    recorded = ModelRunner(folder, dtype=dtype, page_size=8, max_tokens=1024, max_requests=4)
    eager = ModelRunner(folder, dtype=dtype, page_size=8, max_tokens=1024, max_requests=4, use_graphs=False)
    assert recorded.use_graphs and not eager.use_graphs
    reqs = {f"g{i}": random_tokens(vocab, n, 300 + i) for i, n in enumerate((150, 90, 120))}
    done = {k: 0 for k in reqs}
    got = {}

    def both(entries, end=()):
        a = recorded.step([StepEntry(*e) for e in entries], end=end)
        b = eager.step([StepEntry(*e) for e in entries], end=end)
        torch.cuda.synchronize()
        assert (a is None) == (b is None)
        if a is not None:
            assert float((a - b).abs().max()) <= TOL[dtype] * float(b.abs().max()) * 0.1
            # the tokens a recording brings to the host itself are the argmax of the logits it returns,
            # replay after replay (asked for twice: the answer is kept until the next step)
            assert recorded.greedy_tokens(a) == K.argmax(a).tolist() == recorded.greedy_tokens(a)
            assert eager.greedy_tokens(b) == K.argmax(b).tolist()
            row = 0
            for rid, toks, want in entries:
                for w in want:
                    got[(rid, done[rid] + w)] = a[row].clone()
                    row += 1
        for rid, toks, _ in entries:
            done[rid] += len(toks)

    def dec(rid):
        return (rid, [reqs[rid][done[rid]]], [0])

    both([("g0", list(reqs["g0"][:40]), [39])])
    for _ in range(30):
        both([dec("g0")])                                        # batch 1, replayed
    both([("g1", list(reqs["g1"][:33]), []), dec("g0")])          # eager: a prompt portion beside a token
    for _ in range(25):
        both([dec("g0"), dec("g1")])                              # batch 2
    both([("g2", list(reqs["g2"][:64]), [0, 63])])
    for i in range(30):
        both([dec("g1"), dec("g2"), dec("g0")] if i % 3 else [dec("g2"), dec("g0")])
    while done["g1"] < len(reqs["g1"]):
        both([dec("g1")], end=["g1"] if done["g1"] == len(reqs["g1"]) - 1 else ())
    both([dec("g0"), dec("g2")])
    assert len(recorded._recorded) >= 3 and not eager._recorded
    # every recording leaves its logits in the runner's one buffer (they are copied out after a replay), so a
    # recording holds its activations only, not batch x vocabulary floats of its own
    shared = recorded._logits_buffer
    assert shared.shape == (recorded.GRAPH_MAX_BATCH, vocab)
    assert all(rec.logits.data_ptr() == shared.data_ptr() for rec in recorded._recorded.values())
    compare(got, reqs, folder, dtype, "recorded decode")


@pytest.mark.parametrize("verdict", ["as it comes", "refused", "accepted"])
def test_recorded_steps_with_library_products_are_checked_before_use(verdict, monkeypatch):
    """More than 16 rows go to the library's matrix product.  A recording that contains one is
    replayed against eager runs before it is trusted.  The check's answer is also forced both ways:
    a refused shape is noted and runs eagerly from then on, an accepted one is replayed; either way
    the logits of every step equal those of a runner that records nothing."""
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry
    folder = model_folder("A", stored="bfloat16")
    asked, said = [], []
    check = ModelRunner._replays_faithfully
    if verdict != "as it comes":
        monkeypatch.setattr(ModelRunner, "_replays_faithfully",
                            lambda self, *a, **kw: (asked.append(1), verdict == "accepted")[1])
    else:       # the check itself, looked over the shoulder
        monkeypatch.setattr(ModelRunner, "_replays_faithfully",
                            lambda self, *a, **kw: (asked.append(1), said.append(check(self, *a, **kw)), said[-1])[2])
    recorded = ModelRunner(folder, dtype="bfloat16", page_size=16, max_tokens=2048, max_requests=24)
    eager = ModelRunner(folder, dtype="bfloat16", page_size=16, max_tokens=2048, max_requests=24, use_graphs=False)
    n = 20
    prompts = [list(random_tokens(256, 5 + i, 700 + i)) for i in range(n)]
    for i, p in enumerate(prompts):
        a = recorded.step([StepEntry(i, p, [len(p) - 1])])
        b = eager.step([StepEntry(i, p, [len(p) - 1])])
        assert float((a - b).abs().max()) <= 1e-3 * float(b.abs().max())
    toks = [7 * i % 256 for i in range(n)]
    for step in range(6):
        a = recorded.step([StepEntry(i, [toks[i]], [0]) for i in range(n)])
        b = eager.step([StepEntry(i, [toks[i]], [0]) for i in range(n)])
        torch.cuda.synchronize()
        assert float((a - b).abs().max()) <= 2e-3 * float(b.abs().max()), step
        toks = a.argmax(-1).tolist()
    assert len(recorded._recorded) + len(recorded._unrecordable) == 1
    if verdict == "as it comes":
        # asked once, and the shape went where the answer sent it; a shape that was accepted passes the same
        # check again now, after the steps that have replayed it
        assert asked == [1] and len(said) == 1
        assert len(recorded._recorded) == (1 if said[0] else 0) and len(recorded._unrecordable) == (0 if said[0] else 1)
        if said[0]:
            from nanoinfer_amd.engine.runner import StepContext
            (key, rec), = recorded._recorded.items()
            entries = [StepEntry(i, [toks[i]], [0]) for i in range(n)]
            recorded._check_and_reserve(entries)
            warm = StepContext(recorded.device, scratch_owner=recorded)
            flat, layout, rows = recorded._describe(entries, warm)
            recorded._bind(warm, torch.from_numpy(flat).to(recorded.device), layout, rows)
            staging = rec.stagings[0]
            staging.numpy()[:] = recorded._tables_of(entries, StepContext(recorded.device), key[2], ())[0]
            assert check(recorded, rec.graph, rec.logits, warm, rec.meta, staging)
    if verdict == "refused":
        assert asked == [1] and len(recorded._unrecordable) == 1 and not recorded._recorded      # asked once, never recorded again
    if verdict == "accepted":
        assert asked == [1] and len(recorded._recorded) == 1


def test_a_recording_whose_replays_differ_from_the_eager_step_is_refused():
    """The check itself: a graph whose replays leave other logits than the eager step (here: a
    stand-in that spoils the logits after every replay, as a misbehaving recorded node would) is not
    trusted; the same graph unspoiled is."""
    from nanoinfer_amd.engine.runner import ModelRunner, StepContext, StepEntry
    folder = model_folder("A")
    runner = ModelRunner(folder, dtype="float32", page_size=16, max_tokens=512, max_requests=4)
    for i in range(2):
        runner.step([StepEntry(i, list(random_tokens(256, 9 + i, 30 + i)), [])])
    entries = [StepEntry(i, [3 + i], [0]) for i in range(2)]
    runner._check_and_reserve(entries)
    key = runner._graph_shape(entries)
    rec = runner._record(key, entries)
    assert rec is not None
    warm = StepContext(runner.device, scratch_owner=runner)
    flat, layout, rows = runner._describe(entries, warm)
    runner._bind(warm, torch.from_numpy(flat).to(runner.device), layout, rows)

    class Spoiled:
        def __init__(self, graph, logits, by):
            self.graph, self.logits, self.by = graph, logits, by

        def replay(self):
            self.graph.replay()
            self.logits.add_(self.by)

    staging = rec.stagings[0]
    assert runner._replays_faithfully(Spoiled(rec.graph, rec.logits, 0.0), rec.logits, warm, rec.meta, staging)
    assert not runner._replays_faithfully(Spoiled(rec.graph, rec.logits, 0.5), rec.logits, warm, rec.meta, staging)
    rec.logits.fill_(float("nan"))
    assert not runner._replays_faithfully(Spoiled(rec.graph, rec.logits, float("nan")), rec.logits, warm, rec.meta, staging)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_prompt_portions_equal_eager_ones(dtype):
    """A prompt portion of 64 tokens or more that stands alone in its step is recorded per shape
    and replayed at other positions and for other requests; every replay is checked against a
    runner that records nothing, with decode steps and shorter portions between them, and the
    whole against the plain implementation."""
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry
    name = "B"
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    recorded = ModelRunner(folder, dtype=dtype, page_size=8, max_tokens=2048, max_requests=4)
    assert recorded.GRAPH_PORTION_SIGHTS == 2        # by default a shape is recorded when it comes the second time
    recorded.GRAPH_PORTION_SIGHTS = 1                # here: at once
    eager = ModelRunner(folder, dtype=dtype, page_size=8, max_tokens=2048, max_requests=4, use_graphs=False)
    reqs = {f"q{i}": random_tokens(vocab, n, 700 + i) for i, n in enumerate((300, 214, 129))}
    done = {k: 0 for k in reqs}
    got = {}

    def both(entries, end=()):
        a = recorded.step([StepEntry(*e) for e in entries], end=end)
        b = eager.step([StepEntry(*e) for e in entries], end=end)
        torch.cuda.synchronize()
        assert (a is None) == (b is None)
        if a is not None:
            assert float((a - b).abs().max()) <= TOL[dtype] * float(b.abs().max()) * 0.1
            row = 0
            for rid, toks, want in entries:
                for w in want:
                    got[(rid, done[rid] + w)] = a[row].clone()
                    row += 1
        for rid, toks, _ in entries:
            done[rid] += len(toks)

    def portion(rid, n, want_last):
        return (rid, list(reqs[rid][done[rid]:done[rid] + n]), [n - 1] if want_last else [])

    both([portion("q0", 64, False)])                 # recorded now, no logits: judged by the keys and values it writes
    both([portion("q0", 64, True)])                  # another recording: one row of logits
    both([portion("q1", 64, False)])                 # replay for another request at position 0
    both([portion("q0", 64, True)])                  # replay further on in q0 (same bucket of context)
    both([portion("q1", 64, True), portion("q2", 64, False)])      # two portions in one step: not recorded, eager
    both([portion("q0", 3, True)])                   # a short portion: eager
    for _ in range(5):
        both([("q0", [reqs["q0"][done["q0"]]], [0]), ("q1", [reqs["q1"][done["q1"]]], [0])])     # recorded decode steps between
    both([portion("q0", 64, True)])                  # context now beyond 256: a new bucket, a new recording
    both([portion("q1", 64, True)])
    both([portion("q2", 64, True)])
    both([portion("q0", 100 - 64, True)])
    keys = list(recorded._recorded)
    assert sum(1 for k in keys if k[0] == "p") >= 3 and sum(1 for k in keys if k[0] == "d") >= 1, keys
    assert not eager._recorded
    by_request = {}
    for (rid, pos), row in got.items():
        by_request.setdefault(rid, []).append((pos, row))
    for rid, rows in by_request.items():
        want = plain_logits(folder, tuple(reqs[rid]), dtype)
        rows.sort(key=lambda x: x[0])
        idx = [p for p, _ in rows]
        assert_close(torch.stack([r for _, r in rows]), want[idx], dtype, f"recorded portions, request {rid}")


def test_a_portion_shape_is_recorded_when_it_comes_again():
    """A recording costs several runs of its step: a prompt portion's shape that has come once runs
    the ordinary way, the second time it is recorded, from then on replayed."""
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry
    folder = model_folder("B")
    vocab = ALL["B"]["vocab_size"]
    runner = ModelRunner(folder, dtype="float32", page_size=8, max_tokens=1024, max_requests=4)
    eager = ModelRunner(folder, dtype="float32", page_size=8, max_tokens=1024, max_requests=4, use_graphs=False)
    portions = lambda: sum(1 for k in runner._recorded if k[0] == "p")
    for i, (n, recorded_after) in enumerate(((80, 0), (96, 0), (80, 1), (80, 1), (96, 2), (70, 2))):
        toks = random_tokens(vocab, n, 900 + i)
        a = runner.step([StepEntry(i, toks, [n - 1])], end=[i])
        b = eager.step([StepEntry(i, toks, [n - 1])], end=[i])
        assert float((a - b).abs().max()) <= 1e-4 * float(b.abs().max()), (i, n)
        assert portions() == recorded_after, (i, n)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_runs_equal_single_steps(dtype):
    """Runs of decode steps launched back to back, the tokens passing from step to step on the
    device, choose the tokens that single steps with the host between them choose.  The runs
    cross page edges, the context bounds at which another recording takes over (256), the number
    of steps whose tokens the host collects at once, and start before any recording exists; the
    cache they leave gives the same logits afterwards.  Both runners replay the same recordings, so
    their tokens are equal bit for bit.  A runner without recordings decodes in runs too, step by
    step; its attention cuts the keys elsewhere, which may turn a tie of two logits the other way,
    so its tokens are compared in float32 only, where ties are not met."""
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry
    name = "B"
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    runs = ModelRunner(folder, dtype=dtype, page_size=8, max_tokens=2048, max_requests=4)
    single = ModelRunner(folder, dtype=dtype, page_size=8, max_tokens=2048, max_requests=4)
    eager = ModelRunner(folder, dtype=dtype, page_size=8, max_tokens=2048, max_requests=4, use_graphs=False)
    prompts = {f"r{i}": list(random_tokens(vocab, n, 900 + i)) for i, n in enumerate((236, 150, 61))}
    tokens = {}
    with_eager = dtype == "float32"
    for rid, p in prompts.items():
        firsts = []
        for runner in (runs, single, eager) if with_eager else (runs, single):
            logits = runner.step([StepEntry(rid, p, [len(p) - 1])])
            firsts.append(runner.greedy_tokens(logits)[0])
        assert len(set(firsts)) == 1
        tokens[rid] = firsts[0]
    ids = list(prompts)
    for k in (1, 3, 8, 20, 2, 33):
        entries = [StepEntry(rid, [tokens[rid]], [0]) for rid in ids]
        got = runs.decode_run(entries, k)
        want = []
        toks = [tokens[rid] for rid in ids]
        for _ in range(k):
            toks = single.greedy_tokens(single.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, toks)]))
            want.append(list(toks))
        assert got == want, k
        if with_eager:
            assert eager.decode_run([StepEntry(rid, [tokens[rid]], [0]) for rid in ids], k) == want, k
        assert all(runs.computed_tokens(rid) == single.computed_tokens(rid) for rid in ids)
        tokens = dict(zip(ids, want[-1]))
    assert runs.computed_tokens("r0") == 236 + 67 > 256                  # the longest request has passed a bound
    probe = [StepEntry(rid, [tokens[rid]], [0]) for rid in ids]
    a, b = runs.step(probe), single.step(probe)
    assert float((a - b).abs().max()) <= TOL[dtype] * float(b.abs().max()) * 0.1
    # a batch of another make-up after a run: the tables are written anew
    a, b = runs.step(probe[:2]), single.step(probe[:2])
    assert float((a - b).abs().max()) <= TOL[dtype] * float(b.abs().max()) * 0.1
    with pytest.raises(Exception):
        runs.decode_run([StepEntry("r0", [1, 2], [1])], 2)


@pytest.mark.parametrize("page, prompt_len", [(16, 250), (8, 121)])
def test_a_later_wave_of_requests_decodes_in_runs_across_a_recording_s_bounds(page, prompt_len):
    """Waves of fresh requests of one batch size, each decoding in runs of eight: the runs pass,
    in their middle, from one recording into the next (the context bound of 256, or with pages of
    8 tokens the table width of 16 pages at 128 tokens).  From the second wave on both recordings
    exist and hold the tables of requests that are gone.  Tokens equal those of single steps."""
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry
    name = "B"
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    runs = ModelRunner(folder, dtype="float32", page_size=page, max_tokens=1024, max_requests=4)
    single = ModelRunner(folder, dtype="float32", page_size=page, max_tokens=1024, max_requests=4)
    for wave in range(3):
        ids = [f"w{wave}r{i}" for i in range(2)]
        toks = []
        for i, rid in enumerate(ids):
            p = list(random_tokens(vocab, prompt_len + i, 70 + 10 * wave + i))
            a = runs.greedy_tokens(runs.step([StepEntry(rid, p, [len(p) - 1])]))[0]
            b = single.greedy_tokens(single.step([StepEntry(rid, p, [len(p) - 1])]))[0]
            assert a == b
            toks.append(a)
        for _ in range(3):
            got = runs.decode_run([StepEntry(rid, [t], [0]) for rid, t in zip(ids, toks)], 8)
            want = []
            for _ in range(8):
                toks = single.greedy_tokens(single.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, toks)]))
                want.append(list(toks))
            assert got == want, wave
        assert runs.computed_tokens(ids[0]) == prompt_len + 24
        for rid in ids:
            runs.release(rid)
            single.release(rid)
        runs.cache.check()
    assert runs.cache.free_pages() == runs.cache.num_pages


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_long_sequences_reach_the_larger_tiles_and_the_key_runs_of_prompt_attention(dtype, monkeypatch):
    """Configuration D (32 query heads on 8): a prompt of 4,200 tokens in one step takes the tiles
    of two blocks a wavefront; a lone portion of 512 tokens that starts 1,100 tokens into its
    sequence takes two-block tiles with its keys cut into runs.  What the attention was asked for is
    noted, so that the test fails if these paths are no longer the ones taken (bfloat16; the float32
    kernel has one tile size and cuts keys for few tiles only)."""
    from nanoinfer_amd import kernels as K
    name = "D"
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    asked, original = [], K.mfma_attention
    monkeypatch.setattr(K, "mfma_attention", lambda *a, **kw: (asked.append((a[0].shape[0], a[11], a[13])), original(*a, **kw))[1])
    small = K.mfma_tile_tokens(32, 4, dtype=torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    long_prompt = random_tokens(vocab, 4200, 41)
    deep = random_tokens(vocab, 1100 + 512 + 30, 42)
    steps = [([("long", list(long_prompt), [0, 1, 2047, 2048, 4095, 4199])], ["long"]),
             ([("deep", list(deep[:1100]), [1099])], []),
             ([("deep", list(deep[1100:1612]), [0, 255, 511])], []),
             ([("deep", list(deep[1612:]), list(range(30)))], ["deep"])]
    got, _ = run_in_process(folder, dtype, 16, steps, 4200 + 64)
    compare(got, {"long": long_prompt, "deep": deep}, folder, dtype, "configuration D")
    by_tokens = {t: (nsplit, tile) for t, nsplit, tile in asked}
    if dtype == "bfloat16":
        assert by_tokens[4200] == (1, 2 * small)
        assert by_tokens[512] == (4, 2 * small)
    else:
        assert by_tokens[4200][1] == small


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("name", ["E64", "E128"])
def test_the_family_s_head_sizes_reach_the_larger_tiles_and_the_key_runs_through_the_engine(name, dtype, monkeypatch):
    """Head sizes 64 (32 query heads on 8) and 128 (24 on 8) on one narrow layer: a prompt of 2,300 tokens
    in one step (at head size 64 the tiles of two blocks a wavefront), a lone portion of 512 tokens
    1,100 tokens into its sequence (two-block tiles with the keys cut into runs at head size 64), a
    lone portion of 128 tokens there (few tiles: key runs at either head size), then tokens one by
    one.  What the attention was asked for is noted, so that the test fails if these paths are no
    longer the ones taken."""
    from nanoinfer_amd import kernels as K
    folder = model_folder(name)
    cfg = ALL[name]
    vocab, hd, group = cfg["vocab_size"], cfg["head_dim"], cfg["num_attention_heads"] // cfg["num_key_value_heads"]
    asked, original = [], K.mfma_attention
    monkeypatch.setattr(K, "mfma_attention", lambda *a, **kw: (asked.append((a[0].shape[0], a[11], a[13])), original(*a, **kw))[1])
    small = K.mfma_tile_tokens(hd, group, dtype=torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    long_prompt = random_tokens(vocab, 2300, 51)
    deep = random_tokens(vocab, 1100 + 512 + 128 + 20, 52)
    steps = [([("long", list(long_prompt), [0, 1, 1023, 1024, 2047, 2048, 2299])], ["long"]),
             ([("deep", list(deep[:1100]), [1099])], []),
             ([("deep", list(deep[1100:1612]), [0, 255, 511])], []),
             ([("deep", list(deep[1612:1740]), [0, 64, 127])], [])]
    steps += [([("deep", [t], [0])], []) for t in deep[1740:]]
    steps[-1] = (steps[-1][0], ["deep"])
    got, _ = run_in_process(folder, dtype, 16, steps, 2304 + 64)
    compare(got, {"long": long_prompt, "deep": deep}, folder, dtype, f"configuration {name}")
    by_tokens = {t: (nsplit, tile) for t, nsplit, tile in asked}
    if dtype == "bfloat16" and hd == 64:
        assert by_tokens[2300] == (1, 2 * small) and by_tokens[512] == (4, 2 * small)
    if dtype == "bfloat16":
        assert by_tokens[128][0] > 1 and by_tokens[128][1] == small
    else:
        assert by_tokens[2300][1] == small


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_a_sequence_longer_than_one_segment_of_the_block_table(dtype):
    """Configuration F (two heads on one, one layer) past 16,384 tokens at pages of 16: the block table
    of the sequence no longer fits one segment of the table that the attention kernels keep in LDS.
    The prompt goes in portions of 2,048, the last ones ending a little before the seam; then a
    portion of 96 tokens across it, tokens one by one beyond it, and a portion of 40 further on.
    Query and key matrices are drawn ten times larger than the others, so that a row's attention
    rests on a handful of keys anywhere in the sequence and not on the mean of all of them."""
    name = "F"
    folder = model_folder(name, overrides=((".q_proj.weight", 0.0, 0.25), (".k_proj.weight", 0.0, 0.25)))
    vocab = ALL[name]["vocab_size"]
    n = 16384 + 200
    toks = random_tokens(vocab, n, 61)
    steps, at = [], 0
    while at + 2048 <= 16384 - 64:
        steps.append(([("s", list(toks[at:at + 2048]), [0, 2047])], []))
        at += 2048
    head = 16384 - 40 - at
    steps.append(([("s", list(toks[at:at + head]), [head - 1])], []))           # up to 40 tokens before the seam
    at += head
    steps.append(([("s", list(toks[at:at + 96]), list(range(0, 96, 5)) + [95])], []))     # across it
    at += 96
    for t in toks[at:at + 24]:
        steps.append(([("s", [t], [0])], []))                                        # single tokens beyond it
    at += 24
    steps.append(([("s", list(toks[at:at + 40]), list(range(40)))], []))
    at += 40
    for t in toks[at:]:
        steps.append(([("s", [t], [0])], []))
    steps[-1] = (steps[-1][0], ["s"])
    got, _ = run_in_process(folder, dtype, 16, steps, n + 64)
    assert max(p for _, p in got) == n - 1 and any(16300 < p < 16384 for _, p in got)
    compare(got, {"s": toks}, folder, dtype, "past one table segment")
    # the attention does rest on few keys: the largest softmax weight of a late row is far above 1 / context
    config, tensors = P_read(folder)
    assert peak_weight(config, tensors, toks, row=n - 1) > 50.0 / n


def P_read(folder):
    import plain_llama as P
    return P.read_model_folder(folder)


def peak_weight(config, tensors, toks, row):
    """The largest softmax weight that head 0 of the (only) layer gives any key at ``row``."""
    import math

    import plain_llama as P
    H, KVH, hd = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    T = len(toks)
    x = P.rmsnorm(P.embedding(tensors["model.embed_tokens.weight"], toks), tensors["model.layers.0.input_layernorm.weight"],
                  config["rms_norm_eps"])
    sin, cos = P.rope_tables(range(T), P.rope_frequencies(hd, config["rope_theta"], config.get("rope_scaling")))
    q = P.rope_interleaved(P.linear(x, P.permute_reverse(tensors["model.layers.0.self_attn.q_proj.weight"], H)).reshape(T, H, hd), sin, cos)
    k = P.rope_interleaved(P.linear(x, P.permute_reverse(tensors["model.layers.0.self_attn.k_proj.weight"], KVH)).reshape(T, KVH, hd), sin, cos)
    scores = (k[:row + 1, 0] @ q[row, 0]) / math.sqrt(hd)
    return float(torch.softmax(scores, 0).max())
