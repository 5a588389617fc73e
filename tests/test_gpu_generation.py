"""Generation through the entry points: greedy and seeded sampling against the plain
implementation, continuous batching on a pool so small that requests are preempted, the command
line, and the smoke test of the driver."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_llama as P
from gpu_common import model_folder, random_tokens
from tiny_configs import ALL

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def plain_greedy(folder, prompt, n_new, stop=()):
    config, tensors = P.read_model_folder(folder)
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(P.argmax(P.forward(config, tensors, toks)[-1]))
        if toks[-1] in stop:
            break
    return toks[len(prompt):]


def engine(folder, **kw):
    from nanoinfer_amd.engine.llm import Engine
    from nanoinfer_amd.engine.scheduler import EngineConfig
    ignore_eos = kw.pop("ignore_eos", True)
    return Engine(folder, EngineConfig(**kw), ignore_eos=ignore_eos)


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_equals_plain(name):
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder(name)
    vocab = ALL[name]["vocab_size"]
    prompts = [list(random_tokens(vocab, n, 40 + n)) for n in (7, 19, 33)]
    eng = engine(folder, dtype="float32", block_size=16, num_cache_blocks=16, max_sequences=4, prefill_chunk_size=8,
                 max_num_batched_tokens=24)
    results = eng.generate(prompts, max_new_tokens=16, params=SamplingParams.greedy())
    for prompt, res in zip(prompts, results):
        assert res.tokens == plain_greedy(folder, prompt, 16), f"prompt of {len(prompt)}"
        assert res.finish_reason == "length"
    assert eng.runner.cache.free_pages() == 16


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_runs_do_not_change_the_tokens(dtype):
    """Greedy requests decode in runs of steps on one scheduling decision (max_decode_run); the
    tokens are those of an engine that decides before every step, also when requests end at
    different times, join later and draw from a pool that runs short."""
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder("B")
    prompts = [list(random_tokens(1000, n, 80 + n)) for n in (9, 40, 23, 3)]
    outs = []
    for run in (1, 8):
        eng = engine(folder, dtype=dtype, block_size=8, num_cache_blocks=24, max_sequences=3, max_decode_run=run)
        ids = [eng.add_request(p, n, SamplingParams.greedy()) for p, n in zip(prompts, (30, 11, 50, 17))]
        eng.run()
        outs.append([eng.get_request(i).generated for i in ids])
        assert eng.runner.cache.free_pages() == 24
        assert all(eng.get_request(i).finish_reason == "length" for i in ids)
    assert outs[0] == outs[1]
    assert [len(t) for t in outs[1]] == [30, 11, 50, 17]


def test_decode_runs_with_planned_draws_give_the_tokens_of_single_steps():
    """Requests that draw (temperature, top-k, top-p, repetition penalty) decode in runs too: the
    uniform numbers of their draws are known ahead, every step's draw is launched behind the step,
    and the tokens that a penalty looks at grow on the device.  Float32, so that the two ways see
    the same logits to the last bit but for the attention's key runs."""
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder("B")
    prompts = [list(random_tokens(1000, n, 60 + n)) for n in (9, 40, 23, 3)]
    options = [SamplingParams(temperature=0.8, seed=5), SamplingParams(temperature=1.3, top_k=40, top_p=0.9, seed=6),
               SamplingParams.greedy(), SamplingParams(temperature=0.9, top_p=0.8, repetition_penalty=1.6, seed=7)]
    outs, runs = [], []
    for run in (1, 8):
        eng = engine(folder, dtype="float32", block_size=8, num_cache_blocks=24, max_sequences=3, max_decode_run=run)
        asked, original = [], eng.runner.decode_run
        eng.runner.decode_run = lambda entries, steps, pick=None, draw=None: (asked.append((steps, pick is not None)), original(entries, steps, pick, draw))[1]
        ids = [eng.add_request(p, n, o) for p, n, o in zip(prompts, (30, 11, 50, 17), options)]
        eng.run()
        outs.append([eng.get_request(i).generated for i in ids])
        runs.append(asked)
        assert eng.runner.cache.free_pages() == 24
    assert outs[0] == outs[1]
    assert [len(t) for t in outs[1]] == [30, 11, 50, 17]
    assert not runs[0] and any(steps == 8 and draws for steps, draws in runs[1])
    assert len({tuple(t) for t in outs[1]}) == 4 and outs[1][2] != outs[1][0]
    # the penalty changed what was drawn, and a greedy request with a penalty runs through the same plan
    other = engine(folder, dtype="float32", block_size=8, num_cache_blocks=24, max_decode_run=8)
    plain = other.generate([prompts[3]], 17, SamplingParams(temperature=0.9, top_p=0.8, seed=7))[0].tokens
    assert plain != outs[1][3]
    greedy = []
    for run in (1, 8):
        eng = engine(folder, dtype="float32", block_size=8, num_cache_blocks=24, max_decode_run=run)
        greedy.append(eng.generate([prompts[0]], 24, SamplingParams(temperature=0.0, repetition_penalty=1.5))[0].tokens)
    assert greedy[0] == greedy[1] and greedy[0] != outs[1][2][:24]


def test_decode_runs_whose_steps_draw_by_themselves_give_the_tokens_of_single_steps(dtype="float32"):
    """Requests that draw with temperature, top-k and top-p but without a repetition penalty decode in runs whose
    recorded steps make the draw themselves (no kernel is launched between a step and the next): the tokens are
    those of an engine that decides before every step and draws through the sampler.  Float32, so that the two
    ways see the same logits but for the last bits (their batches differ where a request ends inside a run)."""
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder("B")
    prompts = [list(random_tokens(1000, n, 60 + n)) for n in (9, 40, 23, 3)]
    options = [SamplingParams(temperature=0.8, seed=5), SamplingParams(temperature=1.3, top_k=40, top_p=0.9, seed=6),
               SamplingParams.greedy(), SamplingParams(temperature=0.9, top_p=0.8, seed=7)]
    outs, runs = [], []
    for run in (1, 8):
        eng = engine(folder, dtype=dtype, block_size=8, num_cache_blocks=24, max_sequences=3, max_decode_run=run)
        asked, original = [], eng.runner.decode_run
        eng.runner.decode_run = lambda entries, steps, pick=None, draw=None: (
            asked.append((steps, pick is not None, draw is not None)), original(entries, steps, pick, draw))[1]
        ids = [eng.add_request(p, n, o) for p, n, o in zip(prompts, (30, 11, 50, 17), options)]
        eng.run()
        outs.append([eng.get_request(i).generated for i in ids])
        runs.append((asked, {key[0] for key in eng.runner._recorded}))
        assert eng.runner.cache.free_pages() == 24
    assert outs[0] == outs[1]
    assert [len(t) for t in outs[1]] == [30, 11, 50, 17] and len({tuple(t) for t in outs[1]}) == 4
    assert not runs[0][0] and "s" not in runs[0][1]
    assert any(steps == 8 and draws and not picks for steps, picks, draws in runs[1][0]) and "s" in runs[1][1]
    # and a seeded request alone draws the same tokens as in company
    alone = engine(folder, dtype=dtype, block_size=8, num_cache_blocks=24, max_decode_run=8)
    assert alone.generate([prompts[1]], 11, options[1])[0].tokens == outs[1][1]


def test_stop_token_from_the_configuration():
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder("B")
    prompt = list(random_tokens(1000, 12, 3))
    free_run = plain_greedy(folder, prompt, 12)
    # make the fifth generated token a stop token by writing it into a copy of the configuration
    import shutil
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        shutil.copy(os.path.join(folder, "model.safetensors"), d)
        cfg = json.load(open(os.path.join(folder, "config.json")))
        cfg["eos_token_id"] = [free_run[4], 999]
        json.dump(cfg, open(os.path.join(d, "config.json"), "w"))
        eng = engine(d, dtype="float32", num_cache_blocks=8, ignore_eos=False)
        res = eng.generate([prompt], max_new_tokens=12, params=SamplingParams.greedy())[0]
        first = free_run.index(free_run[4])
        assert res.tokens == free_run[:first + 1] and res.finish_reason == "stop"


def test_preemption_does_not_change_the_tokens():
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder("A")
    prompts = [list(random_tokens(256, n, 60 + n)) for n in (20, 25, 30, 18)]
    roomy = engine(folder, dtype="float32", block_size=4, num_cache_blocks=64, max_sequences=4)
    want = [r.tokens for r in roomy.generate(prompts, max_new_tokens=24, params=SamplingParams.greedy())]
    assert roomy.scheduler.num_preemptions == 0
    tight = engine(folder, dtype="float32", block_size=4, num_cache_blocks=30, max_sequences=4)   # 120 tokens for 189
    got = tight.generate(prompts, max_new_tokens=24, params=SamplingParams.greedy())
    assert tight.scheduler.num_preemptions > 0 and any(r.preemptions for r in got)
    assert [r.tokens for r in got] == want
    assert tight.runner.cache.free_pages() == 30


@pytest.mark.parametrize("name", ["A", "D"])
def test_random_scheduling_settings_do_not_change_the_tokens(name, monkeypatch):
    """Float32 generation, greedy or with seeded draws, under a dozen random settings of pool, page, portion,
    token budget, sequences at once, decode run and recorded steps on or off (most of them preempt): the tokens
    are those of an engine with room for everything."""
    import random
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder(name)
    vocab, maxpos = ALL[name]["vocab_size"], ALL[name]["max_position_embeddings"]
    preempted = 0
    for seed in range(12):
        rng = random.Random(seed * 31 + len(name))
        new = rng.randint(5, 40)
        prompts = [list(random_tokens(vocab, rng.randint(1, min(120, maxpos - new - 1)), seed * 100 + i))
                   for i in range(rng.randint(2, 7))]
        page = rng.choice([4, 8, 16])
        need = sum(-(-(len(p) + new) // page) for p in prompts)
        params = SamplingParams.greedy() if seed % 2 else SamplingParams(
            temperature=rng.choice([0.5, 0.8, 1.3]), top_k=rng.choice([0, 5, 50]), top_p=rng.choice([1.0, 0.9, 0.5]),
            repetition_penalty=rng.choice([1.0, 1.2]), seed=seed)
        roomy = engine(folder, dtype="float32", block_size=page, num_cache_blocks=need + 8, max_sequences=8)
        want = [r.tokens for r in roomy.generate(prompts, max_new_tokens=new, params=params)]
        longest = max(-(-(len(p) + new) // page) for p in prompts)
        if rng.random() < 0.3:
            monkeypatch.setenv("NANOINFER_NO_GRAPHS", "1")
        else:
            monkeypatch.delenv("NANOINFER_NO_GRAPHS", raising=False)
        tight = engine(folder, dtype="float32", block_size=page, num_cache_blocks=rng.randint(longest + 1, max(longest + 2, need)),
                       max_sequences=rng.randint(1, 8), prefill_chunk_size=rng.choice([2, 5, 16, 64, 512]),
                       max_num_batched_tokens=rng.choice([8, 33, 256, 2048]), max_decode_run=rng.choice([1, 2, 8]))
        got = [r.tokens for r in tight.generate(prompts, max_new_tokens=new, params=params)]
        assert got == want, (seed, tight.config)
        preempted += tight.scheduler.num_preemptions > 0
        tight.runner.cache.check()
        assert tight.runner.cache.free_pages() == tight.runner.cache.num_pages
    assert preempted >= 3


def test_seeded_sampling_is_reproducible_and_follows_the_plain_pipeline():
    from nanoinfer_amd.sampling.params import SamplingParams
    from nanoinfer_amd.sampling.sampler import uniform_from_counter
    folder = model_folder("B")
    prompts = [list(random_tokens(1000, n, 80 + n)) for n in (1, 40, 77)]
    params = SamplingParams(temperature=0.8, top_k=50, top_p=0.95, repetition_penalty=1.1, seed=1234)
    runs = []
    for chunk in (32, 512):
        eng = engine(folder, dtype="float32", block_size=8, num_cache_blocks=64, prefill_chunk_size=chunk)
        runs.append([r.tokens for r in eng.generate(prompts, max_new_tokens=10, params=params)])
    assert runs[0] == runs[1]                       # the cut of the prompt does not change a seeded draw
    other = engine(folder, dtype="float32", block_size=8, num_cache_blocks=64)
    alone = other.generate(prompts[1:2], max_new_tokens=10, params=params)[0].tokens
    assert alone == runs[0][1]                      # nor does the company in the batch
    # step by step against the plain pipeline with the same uniform numbers
    config, tensors = P.read_model_folder(folder)
    toks, gen = list(prompts[1]), []
    for step in range(10):
        l = P.forward(config, tensors, toks)[-1]
        l = P.repetition_penalty(l, gen, 1.1)
        probs = P.filtered_distribution(P.temperature_scale(l, 0.8), 50, 0.95)
        u = uniform_from_counter(1234, step)
        pick = P.inverse_cdf(probs, u)
        if pick != alone[step]:
            cum = torch.cumsum(probs, 0)
            lo = min(pick, alone[step])
            assert probs[alone[step]] > 0 and abs(float(cum[lo]) - u) < 1e-5, (step, pick, alone[step])
        gen.append(alone[step])
        toks.append(alone[step])
    different = engine(folder, dtype="float32", block_size=8, num_cache_blocks=64)
    p2 = SamplingParams(temperature=0.8, top_k=50, top_p=0.95, repetition_penalty=1.1, seed=99)
    assert different.generate(prompts[1:2], max_new_tokens=10, params=p2)[0].tokens != alone


def test_bfloat16_generation_runs_and_agrees_on_clear_choices():
    """bfloat16 may pick another token where two logits are close; where the plain margin is
    clear it must pick the same."""
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder("A", stored="bfloat16")
    prompt = list(random_tokens(256, 30, 9))
    eng = engine(folder, dtype="bfloat16", num_cache_blocks=8)
    got = eng.generate([prompt], max_new_tokens=8, params=SamplingParams.greedy())[0].tokens
    config, tensors = P.read_model_folder(folder)
    toks = list(prompt)
    compared = 0
    for t in got:
        l = P.forward(config, tensors, toks)[-1]
        top = torch.topk(l, 2).values
        if float(top[0] - top[1]) > 0.05 * float(l.abs().max()):
            assert t == int(l.argmax())
            compared += 1
        toks.append(t)
    assert compared >= 6, f"only {compared} of {len(got)} choices were clear enough to compare"


def test_command_line(tmp_path):
    folder = model_folder("A")
    prompt = list(random_tokens(256, 9, 2))
    cmd = [sys.executable, os.path.join(ROOT, "bin", "nanoinfer"), "--model", folder, "--dtype", "fp32",
           "--prompt-ids", ",".join(map(str, prompt)), "--prompt-len", "21", "--max-tokens", "6", "--ignore-eos",
           "--num-cache-blocks", "16", "--json"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rows = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    assert len(rows) == 2 and rows[0]["tokens"] == plain_greedy(folder, prompt, 6) and rows[1]["prompt_len"] == 21
    assert "Prefill:" in proc.stdout and "Decode:" in proc.stdout and "tok/s" in proc.stdout
    # temperature with a seed: two runs agree
    sampled = []
    for _ in range(2):
        p = subprocess.run(cmd[:-1] + ["--temperature", "0.9", "--top-k", "20", "--seed", "5", "--json"],
                           capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-2000:]
        sampled.append([json.loads(l)["tokens"] for l in p.stdout.splitlines() if l.startswith("{")])
    assert sampled[0] == sampled[1]
    # random-weights mode writes a folder and generates from it
    cfg_path = tmp_path / "cfg.json"
    cfg_path.write_text(json.dumps(ALL["C"]))
    out_dir = tmp_path / "made"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "nanoinfer"), "--random-config", str(cfg_path),
                        "--random-seed", "3", "--save-random-model", str(out_dir), "--max-tokens", "4", "--ignore-eos"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert (out_dir / "config.json").exists() and (out_dir / "model.safetensors").exists()


def test_the_pool_can_be_sized_by_a_byte_budget():
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = model_folder("A")
    # configuration A: 2 layers x (keys + values) x 2 kv heads x 16 dims x 4 bytes = 512 bytes a token, 8 KiB a page of 16
    eng = engine(folder, dtype="float32", block_size=16, kv_cache_bytes=5 * 8192 + 100, max_sequences=2)
    assert eng.runner.cache.num_pages == 5 and eng.runner.cache.pool_bytes() == 5 * 8192
    prompt = list(random_tokens(256, 30, 4))
    got = eng.generate([prompt], max_new_tokens=8, params=SamplingParams.greedy())[0].tokens
    assert got == plain_greedy(folder, prompt, 8)
    with pytest.raises(ValueError, match="do not hold one page"):
        engine(folder, dtype="float32", block_size=16, kv_cache_bytes=100)


def test_smoke_entry():
    sys.path.insert(0, ROOT)
    import __graft_entry__
    __graft_entry__.smoke()
