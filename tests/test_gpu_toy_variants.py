"""Variants of the parts that the framework hosts without a change to its files, in one toy
architecture registered here: a block of another arrangement (norms before AND after mixer and
feed-forward), an attention whose query heads are normalised between projection and rotation (it
replaces one stage of the attention part and keeps the others), and a mixer with a per-request
state of fixed size that reads its step from the device tables, so that its decode steps are
recorded into HIP graphs and replayed like any other.

The model folder is written by the random-weights mode; the model is replayed in the four ways of
cutting in both precisions against a plain forward written here, and generated from through the
entry point with so few pages that requests are preempted and computed again.  The toy parts are
no model of anyone's and are written with library tensor operations: they show what the framework
hosts, not how fast.
"""
from dataclasses import asdict, dataclass

import pytest
import torch

import plain_llama as P
from gpu_common import assert_close, random_tokens
from test_gpu_replay import changing_portions, max_live_tokens, mixed, run_in_process, tail_one_by_one, whole

pytestmark = pytest.mark.gpu

NAME = "ToyVariantsLM"
TOY_CONFIG = {"architectures": [NAME], "width": 96, "layers": 3, "heads": 6, "kv_heads": 2, "head_size": 32,
              "inner": 112, "state": 40, "vocab": 197, "eps": 1e-5, "positions": 192, "decay": 0.5}


@dataclass
class ToyConfig:
    width: int
    layers: int
    heads: int
    kv_heads: int
    head_size: int
    inner: int
    state: int
    vocab: int
    eps: float
    positions: int
    decay: float

    @classmethod
    def from_dict(cls, d):
        return cls(**{k: d[k] for k in cls.__dataclass_fields__})

    def to_dict(self):
        return dict(asdict(self), architectures=[NAME])


def layer_kinds(cfg):
    """Layer i: (block kind, mixer kind).  0: the sandwich block around the q-normed attention; 1: the
    usual block around the state mixer; 2: the usual block around the usual attention; and so on."""
    return [(("toy_sandwich", "toy_qnorm_attention"), ("prenorm", "toy_decay_tables"), ("prenorm", "attention"))[i % 3]
            for i in range(cfg.layers)]


def toy_spec(cfg: ToyConfig):
    from nanoinfer_amd.config.spec import BlockSpec, LayerRun, ModelSpec, PartSpec
    d = cfg.width

    def norm(name):
        return PartSpec("rmsnorm", {"size": d, "eps": cfg.eps}, {"weight": name})

    position = PartSpec("rope", {"rotary_dim": cfg.head_size, "theta": 10000.0, "scaling": None, "max_positions": cfg.positions})
    blocks = []
    for i, (block_kind, mixer_kind) in enumerate(layer_kinds(cfg)):
        pre = f"toy.{i}."
        if mixer_kind == "toy_decay_tables":
            mixer = PartSpec(mixer_kind, {"hidden_size": d, "state_size": cfg.state, "decay": cfg.decay},
                             {"inp": pre + "inp", "out": pre + "out"})
        else:
            names = {"q": pre + "q", "k": pre + "k", "v": pre + "v", "o": pre + "o"}
            if mixer_kind == "toy_qnorm_attention":
                names["q_norm"] = pre + "qn"
            mixer = PartSpec(mixer_kind, {"hidden_size": d, "num_heads": cfg.heads, "num_kv_heads": cfg.kv_heads,
                                          "head_dim": cfg.head_size, "scale": None, "window": None, "position": position,
                                          "q_norm_eps": cfg.eps}, names)
        parts = {"mixer_norm": norm(pre + "n1"), "mixer": mixer, "ffn_norm": norm(pre + "n2"),
                 "ffn": PartSpec("swiglu", {"hidden_size": d, "intermediate_size": cfg.inner},
                                 {"gate": pre + "g", "up": pre + "u", "down": pre + "d"})}
        if block_kind == "toy_sandwich":
            parts["mixer_post_norm"] = norm(pre + "p1")
            parts["ffn_post_norm"] = norm(pre + "p2")
        blocks.append(BlockSpec(block_kind, parts))
    return ModelSpec(vocab_size=cfg.vocab, hidden_size=d, max_positions=cfg.positions,
                     embedding=PartSpec("table", {"vocab_size": cfg.vocab, "hidden_size": d}, {"weight": "toy.tokens"}),
                     blocks=blocks, order=[LayerRun(i, i) for i in range(cfg.layers)], final_norm=norm("toy.norm"),
                     head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d}, {"weight": "toy.tokens"}))


def register_variants():
    from nanoinfer_amd import kernels as K
    from nanoinfer_amd.parts.base import Block, CacheNeed, Part, StateNeed, WeightRequest, pending_for
    from nanoinfer_amd.parts.standard import Attention
    from nanoinfer_amd.registry import Architecture, register_architecture, register_part
    from nanoinfer_amd.weights.random_init import InitRule

    @register_part("block", "toy_sandwich")
    class SandwichBlock(Block):
        """``h += post1(mixer(pre1(h))); h += post2(ffn(pre2(h)))``: four norms instead of two.  Only the
        roles and the arrangement are written here; tensors, building, cache need and the yes/no
        answers of the whole block come from the base."""

        ROLES = {"mixer_norm": "norm", "mixer": "mixer", "mixer_post_norm": "norm",
                 "ffn_norm": "norm", "ffn": "feed_forward", "ffn_post_norm": "norm"}

        def forward(self, h, pending, ctx, cache):
            x = self.mixer_norm.forward(h, pending_for(self.mixer_norm, pending, self.rt.dtype))   # adds what was pending
            a = self.mixer_post_norm.forward(self.mixer.forward(x, ctx, cache).float(), None)
            x = self.ffn_norm.forward(h, a)                                                          # h += a, then the norm
            f = self.ffn_post_norm.forward(self.ffn.forward(x, ctx).float(), None)
            return h, f

    @register_part("mixer", "toy_qnorm_attention")
    class QNormAttention(Attention):
        """The framework's attention with every query head brought to unit root-mean-square and scaled by
        a learned vector, between projection and rotation: the ``project`` stage is replaced, rotation,
        cache write, attention over the pages and the output product are the framework's."""

        @classmethod
        def weight_requests(cls, spec):
            return super().weight_requests(spec) + [WeightRequest(spec.weights["q_norm"], (spec.params["head_dim"],))]

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            self.q_norm = rt.vector32(spec.weights["q_norm"], weights["q_norm"])
            self.q_norm_eps = float(spec.params["q_norm_eps"])

        def project(self, x, ctx):
            qkv = super().project(x, ctx)
            T, width = qkv.shape[0], self.H * self.hd
            q = qkv[:, :width].float().view(T, self.H, self.hd)
            q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + self.q_norm_eps) * self.q_norm
            qkv[:, :width] = q.view(T, width).to(qkv.dtype)
            return qkv

    @register_part("mixer", "toy_decay_tables")
    class DecayMixer(Part):
        """``y_t = out(s_t)``, ``s_t = decay * s_(t-1) + inp(x_t)``: a state of fixed size per request, kept
        in the request's state slot between steps.  Everything it needs to know about the step it reads
        from the device (``ctx.per_seq``, ``ctx.seq_of_token``), so its launches are the same for every
        step of a shape and a decode step with it can be recorded and replayed; since it moves its state
        forward in place, it says that running a step twice is not running it once."""

        graph_safe = True
        idempotent = False

        @classmethod
        def weight_requests(cls, spec):
            d, n = spec.params["hidden_size"], spec.params["state_size"]
            return [WeightRequest(spec.weights["inp"], (n, d)), WeightRequest(spec.weights["out"], (d, n))]

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            self.n = int(spec.params["state_size"])
            self.decay = float(spec.params["decay"])
            self.inp = rt.matrix(spec.weights["inp"], weights["inp"])
            self.out = rt.matrix(spec.weights["out"], weights["out"])

        def cache_need(self):
            return CacheNeed(state=StateNeed((self.n,), torch.float32))

        def forward(self, x, ctx, cache):
            T = x.shape[0]
            per = ctx.per_seq
            u = K.linear(x, self.inp).float()                                    # [T, n]
            seq = ctx.seq_of_token.long()
            row = torch.arange(T, device=x.device)
            # s_i = sum over the rows j <= i of the same sequence of decay^(i-j) u_j, plus the state the
            # sequence brought into the step, decayed once for every row up to i
            apart = row[:, None] - row[None, :]
            weight = torch.where((seq[:, None] == seq[None, :]) & (apart >= 0),
                                 torch.pow(self.decay, apart.clamp(min=0).float()), 0.0)
            brought = cache.state[per.state_slot.long()]                          # [B, n]; zero for a request's first step
            since = (row - per.q_start.long()[seq] + 1).float()
            K.note_library_call()
            states = weight @ u + torch.pow(self.decay, since)[:, None] * brought[seq]
            last = (per.q_start + per.q_len - 1).long()
            cache.state.index_copy_(0, per.state_slot.long(), states[last])
            return K.linear(states.to(x.dtype), self.out)

    register_architecture(Architecture(name=NAME, config_from_dict=ToyConfig.from_dict, build_spec=toy_spec,
                                       init=InitRule(matrix_std=0.08, vector_mean=1.0, vector_std=0.1)))


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    from nanoinfer_amd.weights.loader import make_random_model
    register_variants()
    return make_random_model(str(tmp_path_factory.mktemp("variants") / "model"), TOY_CONFIG, seed=21, dtype="float32")


def plain_forward(folder, tokens, as_bf16=False):
    """The toy model by the plain implementation's functions: whole sequence, no cache, float64."""
    config, tensors = P.read_model_folder(folder)
    if as_bf16:
        tensors = P.round_to_bfloat16(tensors)
    cfg = ToyConfig.from_dict(config)
    t = {k: v.double() for k, v in tensors.items()}
    T, H, KVH, hd = len(tokens), cfg.heads, cfg.kv_heads, cfg.head_size
    sin, cos = P.rope_tables(range(T), P.rope_frequencies(hd, 10000.0, None))
    h = P.embedding(t["toy.tokens"], tokens)
    for i, (block_kind, mixer_kind) in enumerate(layer_kinds(cfg)):
        pre = f"toy.{i}."
        x = P.rmsnorm(h, t[pre + "n1"], cfg.eps)
        if mixer_kind == "toy_decay_tables":
            u = P.linear(x, t[pre + "inp"])
            s, rows = torch.zeros(cfg.state, dtype=torch.float64), []
            for j in range(T):
                s = cfg.decay * s + u[j]
                rows.append(s.clone())
            a = P.linear(torch.stack(rows), t[pre + "out"])
        else:
            q = P.linear(x, P.permute_reverse(t[pre + "q"], H)).reshape(T, H, hd)
            k = P.linear(x, P.permute_reverse(t[pre + "k"], KVH)).reshape(T, KVH, hd)
            v = P.linear(x, t[pre + "v"]).reshape(T, KVH, hd)
            if mixer_kind == "toy_qnorm_attention":
                # the learned vector is stored in the checkpoint's order of a head's dimensions (first half, second
                # half); the plain implementation holds a head with its rotated pairs side by side
                w = t[pre + "qn"]
                w_pairs = torch.stack([w[:hd // 2], w[hd // 2:]], dim=1).reshape(hd)
                q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + cfg.eps) * w_pairs
            q, k = P.rope_interleaved(q, sin, cos), P.rope_interleaved(k, sin, cos)
            a = P.linear(P.causal_attention(q, k, v, range(T)).reshape(T, H * hd), t[pre + "o"])
        if block_kind == "toy_sandwich":
            a = P.rmsnorm(a, t[pre + "p1"], cfg.eps)
        h = h + a
        x = P.rmsnorm(h, t[pre + "n2"], cfg.eps)
        f = P.linear(P.swiglu(P.linear(x, t[pre + "g"]), P.linear(x, t[pre + "u"])), t[pre + "d"])
        if block_kind == "toy_sandwich":
            f = P.rmsnorm(f, t[pre + "p2"], cfg.eps)
        h = h + f
    return P.linear(P.rmsnorm(h, t["toy.norm"], cfg.eps), t["toy.tokens"])


def test_the_variants_are_built_from_their_specs(toy_folder):
    from nanoinfer_amd.engine.runner import ModelRunner
    from nanoinfer_amd.weights.loader import expected_tensors, read_model_folder
    _, _, spec = read_model_folder(toy_folder)
    names = set(expected_tensors(spec))
    assert {"toy.0.p1", "toy.0.p2", "toy.0.qn", "toy.1.inp", "toy.1.out", "toy.2.q"} <= names and "toy.2.p1" not in names
    runner = ModelRunner(toy_folder, dtype="float32", page_size=8, max_tokens=256, max_requests=4)
    kinds = [(type(b).kind, type(b.mixer).kind) for b in runner.model.blocks]
    assert kinds == [("toy_sandwich", "toy_qnorm_attention"), ("prenorm", "toy_decay_tables"), ("prenorm", "attention")]
    assert runner.model.graph_safe() and not runner.model.idempotent() and runner.use_graphs
    assert list(runner.cache.state) == [1] and tuple(runner.cache.state[1].shape) == (4, TOY_CONFIG["state"])
    # a block that is given a part it has no role for, or lacks one, says so
    from nanoinfer_amd.config.spec import BlockSpec
    from nanoinfer_amd.registry import get_part
    bad = BlockSpec("prenorm", dict(spec.blocks[0].parts))
    with pytest.raises(ValueError, match="not known.*mixer_post_norm"):
        get_part("block", "prenorm").weight_requests(bad)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_the_variants_replay_in_the_four_ways(toy_folder, mode, dtype):
    vocab = TOY_CONFIG["vocab"]
    requests = {f"r{i}": random_tokens(vocab, n, 700 + i) for i, n in enumerate((3, 41, 77, 150, 64, 9))}
    steps = {"whole": whole, "tail": tail_one_by_one, "portions": changing_portions,
             "mixed": lambda r: mixed(r, seed=3)}[mode](requests)
    page = 8
    seen = {}
    got, reused = run_in_process(toy_folder, dtype, page, steps, max_live_tokens(steps, requests, page), seen=seen)
    assert got and (reused or mode != "mixed")
    if mode == "tail":
        # the single tokens ran as replays of recorded steps, state mixer and all
        assert any(key[0] == "d" for key in seen["recorded"]) and not seen["unrecordable"]
    for rid, toks in requests.items():
        plain = plain_forward(toy_folder, list(toks), as_bf16=dtype == "bfloat16")
        rows = sorted((pos, row) for (r, pos), row in got.items() if r == rid)
        assert_close(torch.stack([row for _, row in rows]), plain[[pos for pos, _ in rows]], dtype, f"variants {mode} {rid}")


def plain_greedy(folder, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(plain_forward(folder, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("decode_run", [1, 8])
def test_preempted_requests_of_the_variants_are_computed_again_with_a_fresh_state(toy_folder, decode_run):
    """Generation through the entry point with so few pages that requests are preempted: a preempted
    request gives its state slot back and starts again from an empty one.  Greedy tokens in float32 are
    those of the plain forward; decode steps run as replays (in runs of eight, the tokens passing from
    step to step on the device), each advancing the state once."""
    from nanoinfer_amd.engine.llm import Engine
    from nanoinfer_amd.engine.scheduler import EngineConfig
    from nanoinfer_amd.sampling.params import SamplingParams
    prompts = [list(random_tokens(TOY_CONFIG["vocab"], n, 40 + n)) for n in (20, 25, 30, 18)]
    want = [plain_greedy(toy_folder, p, 24) for p in prompts]
    for blocks in (64, 30):
        eng = Engine(toy_folder, EngineConfig(dtype="float32", block_size=4, num_cache_blocks=blocks, max_sequences=4,
                                              max_decode_run=decode_run), ignore_eos=True)
        got = eng.generate(prompts, max_new_tokens=24, params=SamplingParams.greedy())
        assert [r.tokens for r in got] == want, blocks
        assert (eng.scheduler.num_preemptions > 0) == (blocks == 30)
        assert any(key[0] == "d" for key in eng.runner._recorded)
        assert eng.runner.cache.free_pages() == blocks and eng.runner.cache.slots.num_free == 4
