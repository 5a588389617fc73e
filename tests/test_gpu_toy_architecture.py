"""Another architecture, added from outside the package: a typed configuration, a ``build_spec`` and
two toy parts, registered here and nowhere else.  Its model folder is written by the random-weights
mode, read back by ``config.json``'s architecture name, and replayed through the same runner,
cache and kernels in the four ways of cutting, against a plain forward written here from the plain
implementation's functions.  Nothing under ``nanoinfer_amd/`` knows of it.

The toy parts are no model of anyone's: an embedding that adds a learned vector per position (it
needs the step's positions, and a second tensor), and a rotary position encoding whose
frequencies are stored in the checkpoint (a position part that asks for a tensor).  They are
written with library tensor operations: they show what the framework hosts, not how fast.
"""
import json
import os
from dataclasses import asdict, dataclass

import pytest
import torch

import plain_llama as P
from gpu_common import assert_close, random_tokens
from test_gpu_replay import changing_portions, max_live_tokens, mixed, run_in_process, tail_one_by_one, whole

pytestmark = pytest.mark.gpu

TOY_CONFIG = {
    "architectures": ["ToyLearnedPositionsLM"], "width": 80, "layers": 2, "heads": 5, "kv_heads": 5, "head_size": 16,
    "inner": 96, "vocab": 211, "eps": 1e-5, "positions": 160,
}


@dataclass
class ToyConfig:
    width: int
    layers: int
    heads: int
    kv_heads: int
    head_size: int
    inner: int
    vocab: int
    eps: float
    positions: int

    @classmethod
    def from_dict(cls, d):
        return cls(**{k: d[k] for k in cls.__dataclass_fields__})

    def to_dict(self):
        return dict(asdict(self), architectures=["ToyLearnedPositionsLM"])


def toy_spec(cfg: ToyConfig):
    from nanoinfer_amd.config.spec import BlockSpec, LayerRun, ModelSpec, PartSpec
    d = cfg.width
    blocks = []
    for i in range(cfg.layers):
        pre = f"toy.{i}."
        position = PartSpec("toy_stored_rotation", {"rotary_dim": cfg.head_size, "max_positions": cfg.positions},
                            {"freqs": pre + "rotation"})
        blocks.append(BlockSpec("prenorm", dict(
            mixer_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.eps}, {"weight": pre + "n1"}),
            mixer=PartSpec("attention", {"hidden_size": d, "num_heads": cfg.heads, "num_kv_heads": cfg.kv_heads,
                                         "head_dim": cfg.head_size, "scale": None, "window": None, "position": position},
                           {"q": pre + "q", "k": pre + "k", "v": pre + "v", "o": pre + "o"}),
            ffn_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.eps}, {"weight": pre + "n2"}),
            ffn=PartSpec("swiglu", {"hidden_size": d, "intermediate_size": cfg.inner},
                         {"gate": pre + "g", "up": pre + "u", "down": pre + "d"}))))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=d, max_positions=cfg.positions,
        embedding=PartSpec("toy_learned_positions", {"vocab_size": cfg.vocab, "hidden_size": d, "positions": cfg.positions},
                           {"weight": "toy.tokens", "positions": "toy.positions"}),
        blocks=blocks, order=[LayerRun(i, i) for i in range(cfg.layers)],
        final_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.eps}, {"weight": "toy.norm"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d}, {"weight": "toy.head"}))


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    from nanoinfer_amd import kernels as K
    from nanoinfer_amd.parts.base import Part, WeightRequest
    from nanoinfer_amd.registry import Architecture, register_architecture, register_part
    from nanoinfer_amd.weights.loader import make_random_model
    from nanoinfer_amd.weights.random_init import InitRule

    @register_part("embedding", "toy_learned_positions")
    class LearnedPositionsEmbedding(Part):
        graph_safe = True

        @classmethod
        def weight_requests(cls, spec):
            p = spec.params
            return [WeightRequest(spec.weights["weight"], (p["vocab_size"], p["hidden_size"])),
                    WeightRequest(spec.weights["positions"], (p["positions"], p["hidden_size"]))]

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            self.weight = rt.matrix(spec.weights["weight"], weights["weight"])
            self.positions = rt.matrix(spec.weights["positions"], weights["positions"])     # in the compute type, like every matrix

        def forward(self, token_ids, ctx):
            out = torch.empty(token_ids.shape[0], self.weight.shape[1], dtype=torch.float32, device=self.rt.device)
            K.embedding(token_ids, self.weight, out)
            return out.add_(self.positions.index_select(0, ctx.positions).float())

    @register_part("position", "toy_stored_rotation")
    class StoredRotation(Part):
        graph_safe = True

        @classmethod
        def weight_requests(cls, spec):
            return [WeightRequest(spec.weights["freqs"], (spec.params["rotary_dim"] // 2,))]

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            freqs = weights["freqs"].to(device=rt.device, dtype=torch.float32).contiguous()
            self.cos, self.sin = K.rope_table(freqs, int(spec.params["max_positions"]))

        def tables(self):
            return self.cos, self.sin

    register_architecture(Architecture(
        name="ToyLearnedPositionsLM", config_from_dict=ToyConfig.from_dict, build_spec=toy_spec,
        # stored frequencies around 0.3, learned position vectors as large as the token vectors
        init=InitRule(matrix_std=0.08, overrides=((".rotation", 0.3, 0.1), ("toy.positions", 0.0, 0.08)))))
    folder = str(tmp_path_factory.mktemp("toy") / "model")
    return make_random_model(folder, TOY_CONFIG, seed=12, dtype="float32")


def plain_toy_forward(folder, tokens, as_bf16=False):
    """The toy model by the plain implementation's functions, whole sequence, float64; ``as_bf16``:
    with the matrices rounded to bfloat16 first, as a bfloat16 engine holds them."""
    config, tensors = P.read_model_folder(folder)
    if as_bf16:
        tensors = P.round_to_bfloat16(tensors)
    cfg = ToyConfig.from_dict(config)
    t = {k: v.double() for k, v in tensors.items()}
    T = len(tokens)
    h = P.embedding(t["toy.tokens"], tokens) + t["toy.positions"][:T]
    for i in range(cfg.layers):
        pre = f"toy.{i}."
        x = P.rmsnorm(h, t[pre + "n1"], cfg.eps)
        q = P.linear(x, P.permute_reverse(t[pre + "q"], cfg.heads)).reshape(T, cfg.heads, cfg.head_size)
        k = P.linear(x, P.permute_reverse(t[pre + "k"], cfg.kv_heads)).reshape(T, cfg.kv_heads, cfg.head_size)
        v = P.linear(x, t[pre + "v"]).reshape(T, cfg.kv_heads, cfg.head_size)
        sin, cos = P.rope_tables(range(T), tensors[pre + "rotation"].to(torch.float32).numpy())      # stored, not rounded
        q, k = P.rope_interleaved(q, sin, cos), P.rope_interleaved(k, sin, cos)
        a = P.causal_attention(q, k, v, range(T)).reshape(T, cfg.heads * cfg.head_size)
        h = h + P.linear(a, t[pre + "o"])
        x = P.rmsnorm(h, t[pre + "n2"], cfg.eps)
        h = h + P.linear(P.swiglu(P.linear(x, t[pre + "g"]), P.linear(x, t[pre + "u"])), t[pre + "d"])
    return P.linear(P.rmsnorm(h, t["toy.norm"], cfg.eps), t["toy.head"])


def test_the_folder_is_what_the_parts_and_the_rule_say(toy_folder):
    from nanoinfer_amd.weights.loader import expected_tensors, load_tensors, read_model_folder
    arch, cfg, spec = read_model_folder(toy_folder)
    assert arch.name == "ToyLearnedPositionsLM" and isinstance(cfg, ToyConfig) and cfg.heads == 5
    assert json.load(open(os.path.join(toy_folder, "config.json")))["architectures"] == ["ToyLearnedPositionsLM"]
    tensors = load_tensors(toy_folder, spec)
    assert set(tensors) == set(expected_tensors(spec))
    assert tensors["toy.positions"].shape == (160, 80) and tensors["toy.1.rotation"].shape == (8,)
    assert abs(float(tensors["toy.0.rotation"].mean()) - 0.3) < 0.15          # the rule's override for that name
    assert abs(float(tensors["toy.0.n1"].mean()) - 1.0) < 0.1                  # the rule for tensors of one dimension


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_the_toy_architecture_replays_like_any_other(toy_folder, mode, dtype):
    vocab = TOY_CONFIG["vocab"]
    requests = {f"r{i}": random_tokens(vocab, n, 300 + i) for i, n in enumerate((3, 41, 77, 150))}
    steps = {"whole": whole, "tail": tail_one_by_one, "portions": changing_portions,
             "mixed": lambda r: mixed(r, seed=8)}[mode](requests)
    page = 8
    got, reused = run_in_process(toy_folder, dtype, page, steps, max_live_tokens(steps, requests, page))
    assert got and (reused or mode != "mixed")
    plain = {rid: plain_toy_forward(toy_folder, list(toks), as_bf16=dtype == "bfloat16") for rid, toks in requests.items()}
    for rid in requests:
        rows = sorted((pos, row) for (r, pos), row in got.items() if r == rid)
        assert_close(torch.stack([row for _, row in rows]), plain[rid][[pos for pos, _ in rows]], dtype, f"toy {mode} {rid}")


def test_the_toy_architecture_generates_through_the_entry_point(toy_folder):
    from nanoinfer_amd.engine.llm import Engine
    from nanoinfer_amd.engine.scheduler import EngineConfig
    from nanoinfer_amd.sampling.params import SamplingParams
    prompts = [list(random_tokens(TOY_CONFIG["vocab"], n, 50 + n)) for n in (9, 30)]
    eng = Engine(toy_folder, EngineConfig(dtype="float32", block_size=8, num_cache_blocks=32, max_sequences=2))
    results = eng.generate(prompts, max_new_tokens=6, params=SamplingParams.greedy())
    for prompt, res in zip(prompts, results):
        toks = list(prompt)
        for _ in range(6):
            toks.append(int(plain_toy_forward(toy_folder, toks)[-1].argmax()))
        assert res.tokens == toks[len(prompt):]
