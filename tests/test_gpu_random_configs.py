"""Configurations drawn at random (head counts and groups, head sizes in steps of 16, widths, feed-forward
sizes and vocabularies that are multiples of nothing, pages of any size) through the engine, against the
plain implementation: a size that the configuration allows is computed right or refused with an error that
names it.  The seeds here are a sample; the same generator was run once over 1,100 more."""
import json
import os
import random
import shutil
import tempfile

import pytest
import torch

import gpu_common as G
from test_gpu_replay import changing_portions, max_live_tokens, mixed, run_in_process, tail_one_by_one

pytestmark = pytest.mark.gpu

HEAD_SIZES = (16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 256)


def random_config(rng, head_sizes=HEAD_SIZES):
    heads = rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 20])
    kv_heads = rng.choice([d for d in range(1, heads + 1) if heads % d == 0])
    scaling = None
    if rng.random() < 0.6:
        low = rng.choice([1.0, 0.5, 2.0])
        scaling = {"rope_type": "llama3", "factor": rng.choice([2.0, 4.0, 8.0, 32.0]), "low_freq_factor": low,
                   "high_freq_factor": low * rng.choice([2.0, 4.0, 8.0]),
                   "original_max_position_embeddings": rng.choice([16, 64, 256, 8192])}
    return {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": rng.choice([rng.randint(8, 400), rng.choice([64, 128, 192, 256, 320, 512, 1024]), rng.randint(8, 50) * 8]),
        "num_hidden_layers": rng.randint(1, 3), "num_attention_heads": heads, "num_key_value_heads": kv_heads,
        "head_dim": rng.choice(head_sizes),
        "intermediate_size": rng.choice([rng.randint(8, 700), rng.choice([64, 128, 256, 512, 1024, 2048]), rng.randint(2, 90) * 16]),
        "vocab_size": rng.choice([rng.randint(3, 3000), rng.choice([256, 1024, 4096]), rng.randint(30000, 40000)]),
        "rms_norm_eps": rng.choice([1e-5, 1e-6, 3e-6, 1e-4]), "rope_theta": rng.choice([10000.0, 500000.0, 25000.0, 1e6]),
        "rope_scaling": scaling, "max_position_embeddings": 1024, "tie_word_embeddings": rng.random() < 0.5,
        "hidden_act": "silu",
    }


@pytest.fixture
def folder_of():
    made = []

    def make(config, seed):
        from nanoinfer_amd.weights.loader import make_random_model
        root = tempfile.mkdtemp(prefix="nanoinfer-random-config-")
        made.append(root)
        return make_random_model(os.path.join(root, "model"), config, seed, dtype="float32")

    yield make
    for root in made:
        shutil.rmtree(root, ignore_errors=True)


@pytest.mark.parametrize("seed", [3, 14, 27, 101, 158, 222, 340, 481])
def test_a_configuration_drawn_at_random_gives_the_plain_logits(seed, folder_of):
    rng = random.Random(seed)
    config = random_config(rng)
    page = rng.choice([1, 3, 4, 8, 16, 16, 32, 12])
    folder = folder_of(config, seed)
    lengths = [rng.randint(1, 140) for _ in range(5)] + [rng.randint(150, 400)]
    requests = {f"q{i}": G.random_tokens(config["vocab_size"], n, seed * 10 + i) for i, n in enumerate(lengths)}
    what = f"seed {seed}, pages of {page}, " + json.dumps({k: config[k] for k in (
        "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size",
        "vocab_size", "tie_word_embeddings")})
    for dtype in ("float32", "bfloat16"):
        for steps in (mixed(requests, seed=seed), tail_one_by_one(requests), changing_portions(requests)):
            got, _ = run_in_process(folder, dtype, page, steps, max_live_tokens(steps, requests, page))
            by_request = {}
            for (rid, pos), row in got.items():
                by_request.setdefault(rid, []).append((pos, row))
            for rid, rows in by_request.items():
                want = G.plain_logits(folder, tuple(requests[rid]), dtype)
                rows.sort(key=lambda x: x[0])
                at = [p for p, _ in rows]
                G.assert_close(torch.stack([r for _, r in rows]), want[at], dtype, f"{what}; {dtype}, request {rid}")


@pytest.mark.parametrize("head_dim", [24, 40, 6])
def test_a_head_size_outside_the_steps_of_16_is_refused_by_name(head_dim, folder_of):
    from nanoinfer_amd.engine.runner import ModelRunner
    config = dict(random_config(random.Random(1)), head_dim=head_dim)
    folder = folder_of(config, 1)
    with pytest.raises(Exception, match=f"head size {head_dim} is not supported"):
        ModelRunner(folder, dtype="float32", page_size=16, max_tokens=256, max_requests=2)
