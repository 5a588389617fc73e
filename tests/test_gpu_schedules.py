"""Schedules that the other files do not reach: steps of more than 64 sequences (past the
largest recorded batch and the skinny products' 64 rows), and bfloat16 under random scheduling
with preemptions, judged by logits and not by tokens."""
import random

import pytest
import torch

import plain_llama as P
from gpu_common import assert_close, model_folder, plain_logits, random_tokens
from tiny_configs import ALL

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------ more than 64 sequences in a step

@pytest.mark.parametrize("recorded_up_to", [64, 256])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_of_more_than_64_sequences(dtype, recorded_up_to):
    """A hundred live requests of configuration B: their prompts in one step of a hundred portions, a
    pure decode step of a hundred tokens, a step of seventy tokens beside thirty portions of two, and
    the rest token by token, a hundred a step (the last steps shrink below 64 as requests end).
    Every row of every step is compared with the plain implementation.  More than 64 rows are past
    what the skinny products take: such a decode step runs on the library's products and the kernels
    between them, eagerly (``recorded_up_to`` 64) or as a recorded step."""
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry
    name, n = "B", 100
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    requests = {i: random_tokens(vocab, 14 + (i * 7) % 29, 4000 + i) for i in range(n)}
    runner = ModelRunner(folder, dtype=dtype, page_size=8, max_tokens=n * 48, max_requests=128)
    assert runner.GRAPH_MAX_BATCH == 256
    runner.GRAPH_MAX_BATCH = recorded_up_to
    done = {i: 0 for i in requests}
    got = {}

    def step(counts):
        entries = [StepEntry(i, list(requests[i][done[i]:done[i] + c]), list(range(c))) for i, c in counts.items()]
        out = runner.step(entries, end=[i for i, c in counts.items() if done[i] + c == len(requests[i])])
        assert out.shape[0] == sum(counts.values())
        row = 0
        for i, c in counts.items():
            for j in range(c):
                got[(i, done[i] + j)] = out[row].clone()
                row += 1
            done[i] += c

    step({i: len(requests[i]) - 3 - i % 9 for i in requests})          # a hundred prompt portions (3 to 11 tokens are left)
    step({i: 1 for i in requests})                                     # a hundred single tokens
    step({i: (2 if i % 10 < 3 else 1) for i in requests})              # seventy tokens beside thirty portions
    sizes = []
    while any(done[i] < len(requests[i]) for i in requests):
        live = {i: 1 for i in requests if done[i] < len(requests[i])}
        sizes.append(len(live))
        step(live)
    assert max(sizes) > 64 > min(sizes)                                # both sides of the recorded steps' limit
    assert not runner.cache.live_requests() and runner.cache.free_pages() == runner.cache.num_pages
    assert (max(key[1] for key in runner._recorded if key[0] == "d") > 64) == (recorded_up_to > 64)
    for i, toks in requests.items():
        want = plain_logits(folder, tuple(toks), dtype)
        assert_close(torch.stack([got[(i, p)] for p in range(len(toks))]), want, dtype, f"request {i} of {n}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_with_more_than_64_requests_at_once(dtype):
    """A hundred requests through the entry point with ``max_batch_size`` 128: greedy tokens in
    float32 are the plain implementation's; in bfloat16 they are wherever the plain margin between the
    two largest logits is clear."""
    from nanoinfer_amd.engine.llm import Engine
    from nanoinfer_amd.engine.scheduler import EngineConfig
    from nanoinfer_amd.sampling.params import SamplingParams
    name, n, new = "B", 100, 5
    folder = model_folder(name, stored="bfloat16")
    vocab = ALL[name]["vocab_size"]
    prompts = [list(random_tokens(vocab, 3 + (i * 5) % 23, 6000 + i)) for i in range(n)]
    eng = Engine(folder, EngineConfig(dtype=dtype, block_size=8, num_cache_blocks=n * 5, max_sequences=128, max_batch_size=128,
                                      max_num_batched_tokens=4096), ignore_eos=True)
    batches = []
    step = eng.runner.step
    eng.runner.step = lambda entries, end=(): (batches.append(len(entries)), step(entries, end))[1]
    results = eng.generate(prompts, max_new_tokens=new, params=SamplingParams.greedy())
    assert max(batches) == n, "the hundred requests never ran in one step"
    config, tensors = P.read_model_folder(folder)
    clear = 0
    for prompt, res in zip(prompts, results):
        toks = list(prompt)
        for t in res.tokens:
            row = P.forward(config, tensors, toks)[-1]
            top = torch.topk(row, 2).values
            if dtype == "float32" or float(top[0] - top[1]) > 0.05 * float(row.abs().max()):
                assert t == int(row.argmax()), (len(prompt), len(toks))
                clear += 1
            toks.append(t)
    assert clear >= (n * new if dtype == "float32" else n * new // 3)


# ------------------------------------------------------------------ bfloat16 under random scheduling

class ScriptedSampler:
    """Stands where the engine's sampler stands.  It gives every request the next token of a script
    written beforehand (so that the tokens do not depend on close calls between two logits) and
    keeps the logits it was shown: row (request, tokens generated so far).  Requests are told apart
    by the seed of their sampling options.  It plans runs of decode steps like the real one."""

    def __init__(self, scripts):
        self.scripts = scripts          # seed -> the tokens the request is to "generate"
        self.seen = {}

    def _note(self, logits, params, counts):
        rows = logits.float().cpu()
        for r, (p, c) in enumerate(zip(params, counts)):
            assert (p.seed, c) not in self.seen, "a request was asked for the same token twice"
            self.seen[(p.seed, c)] = rows[r].clone()

    def sample(self, logits, params, generated, counters, greedy=None):
        self._note(logits, params, counters)
        return [self.scripts[p.seed][c] for p, c in zip(params, counters)]

    def plan(self, params, generated, steps):
        sampler, start = self, [len(g) for g in generated]

        class Plan:
            def launch(self, i, logits, out):
                sampler._note(logits, params, [s + i for s in start])
                out.copy_(torch.tensor([sampler.scripts[p.seed][s + i] for p, s in zip(params, start)], dtype=torch.int32))
        return Plan()


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_random_scheduling_settings_do_not_change_the_logits(name, dtype, monkeypatch):
    """Generation under random settings of pool, page, portion, token budget, sequences at once, decode
    run and recorded steps on or off (most of them preempt and compute requests again), with the
    tokens given by a script: the logits from which every token of every request would have been
    chosen are those of the plain implementation over the request's whole sequence, row by row."""
    from nanoinfer_amd.engine.llm import Engine
    from nanoinfer_amd.engine.scheduler import EngineConfig
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder(name)
    vocab, maxpos = ALL[name]["vocab_size"], ALL[name]["max_position_embeddings"]
    preempted = runs = 0
    for seed in range(8):
        rng = random.Random(seed * 17 + len(name))
        new = rng.randint(5, 40)
        prompts = [list(random_tokens(vocab, rng.randint(1, min(120, maxpos - new - 1)), seed * 100 + i))
                   for i in range(rng.randint(2, 7))]
        scripts = {i: list(random_tokens(vocab, new, 9000 + seed * 10 + i)) for i in range(len(prompts))}
        page = rng.choice([4, 8, 16])
        need = sum(-(-(len(p) + new) // page) for p in prompts)
        longest = max(-(-(len(p) + new) // page) for p in prompts)
        if rng.random() < 0.3:
            monkeypatch.setenv("NANOINFER_NO_GRAPHS", "1")
        else:
            monkeypatch.delenv("NANOINFER_NO_GRAPHS", raising=False)
        sampler = ScriptedSampler(scripts)
        eng = Engine(folder, EngineConfig(dtype=dtype, block_size=page, num_cache_blocks=rng.randint(longest + 1, max(longest + 2, need)),
                                          max_sequences=rng.randint(1, 8), prefill_chunk_size=rng.choice([2, 5, 16, 64, 512]),
                                          max_num_batched_tokens=rng.choice([8, 33, 256, 2048]),
                                          max_decode_run=rng.choice([1, 2, 8])), sampler=sampler, ignore_eos=True)
        planned = []
        decode_run = eng.runner.decode_run
        eng.runner.decode_run = lambda entries, steps, pick=None, draw=None: (planned.append(steps), decode_run(entries, steps, pick, draw))[1]
        ids = [eng.add_request(p, new, SamplingParams(temperature=1.0, seed=i)) for i, p in enumerate(prompts)]
        eng.run()
        preempted += eng.scheduler.num_preemptions > 0
        runs += any(s > 1 for s in planned)
        eng.runner.cache.check()
        assert eng.runner.cache.free_pages() == eng.runner.cache.num_pages
        for i, (rid, prompt) in enumerate(zip(ids, prompts)):
            assert eng.get_request(rid).generated == scripts[i]
            want = plain_logits(folder, tuple(prompt + scripts[i][:-1]), dtype)
            rows = torch.stack([sampler.seen[(i, c)] for c in range(new)])
            assert_close(rows, want[len(prompt) - 1:], dtype, f"{name} setting {seed} request {i} ({eng.config})")
    assert preempted >= 3 and runs >= 1
