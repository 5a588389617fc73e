"""Each part alone, built from a spec as the model builds it, against the plain functions; the
order of layers as data; and toy parts that are registered, built and stepped from here without a
change to the framework's files: a mixer with state of its own, a feed-forward with routing beside
a dense one, another position encoding."""
import math

import pytest
import torch

import plain_llama as P
from gpu_common import TOL, model_folder, random_tokens
from tiny_configs import ALL, TINY_B

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def rel(got, want):
    return float((got.double().cpu() - want.double()).abs().max() / float(want.double().abs().max()))


def runtime(dtype):
    from nanoinfer_amd.parts.base import Runtime
    return Runtime(DT[dtype], torch.device("cuda", 0))


def test_parts_fail_loudly_without_their_sizes():
    from nanoinfer_amd.config.spec import PartSpec
    from nanoinfer_amd.parts.standard import Attention
    spec = PartSpec("attention", {"hidden_size": 64, "num_heads": 4, "num_kv_heads": 2, "head_dim": 24,
                                  "position": PartSpec("none")}, {"q": "q", "k": "k", "v": "v", "o": "o"})
    w = {"q": torch.zeros(96, 64), "k": torch.zeros(48, 64), "v": torch.zeros(48, 64), "o": torch.zeros(64, 96)}
    with pytest.raises(Exception) as e:
        Attention(spec, w, runtime("float32"))
    assert "multiple of 16" in str(e.value)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_embedding_head_feed_forward(dtype):
    from nanoinfer_amd.config.spec import PartSpec
    from nanoinfer_amd.parts.standard import build_part
    rt = runtime(dtype)
    g = torch.Generator().manual_seed(0)
    d, I, V, T = 100, 136, 777, 13
    tensors = {"n": 1 + 0.1 * torch.randn(d, generator=g), "e": 0.1 * torch.randn(V, d, generator=g),
               "g": 0.1 * torch.randn(I, d, generator=g), "u": 0.1 * torch.randn(I, d, generator=g),
               "d": 0.1 * torch.randn(d, I, generator=g)}
    rounded = {k: (v.to(DT[dtype]).double() if v.dim() == 2 else v.double()) for k, v in tensors.items()}
    norm = build_part("norm", PartSpec("rmsnorm", {"size": d, "eps": 1e-3}, {"weight": "n"}), tensors, rt)
    h = torch.randn(T, d, generator=g)
    x = norm.forward(h.cuda(), None)
    assert x.dtype == DT[dtype] and rel(x, P.rmsnorm(h, tensors["n"], 1e-3)) < TOL[dtype]
    emb = build_part("embedding", PartSpec("table", {"vocab_size": V, "hidden_size": d}, {"weight": "e"}), tensors, rt)
    ids = torch.randint(0, V, (T,), generator=g).to(torch.int32)
    assert torch.equal(emb.forward(ids.cuda()).double().cpu(), rounded["e"][ids.long()])
    head = build_part("head", PartSpec("linear", {"vocab_size": V, "hidden_size": d}, {"weight": "e"}), tensors, rt)
    assert head.weight.data_ptr() == emb.weight.data_ptr()                    # tied: one buffer on the device
    xin = x
    logits = head.forward(xin)
    assert logits.dtype == torch.float32 and rel(logits, P.linear(xin.double().cpu(), rounded["e"])) < TOL[dtype]
    ffn = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": d, "intermediate_size": I},
                                              {"gate": "g", "up": "u", "down": "d"}), tensors, rt)
    y = ffn.forward(xin, None)
    xd = xin.double().cpu()
    want = P.linear(P.swiglu(P.linear(xd, rounded["g"]), P.linear(xd, rounded["u"])), rounded["d"])
    assert rel(y, want) < TOL[dtype]


def test_position_part_shares_one_table():
    from nanoinfer_amd.config.spec import PartSpec
    from nanoinfer_amd.parts.standard import build_part
    rt = runtime("float32")
    sc = dict(TINY_B["rope_scaling"])
    sc["kind"] = sc.pop("rope_type")
    spec = PartSpec("rope", {"rotary_dim": 32, "theta": 500000.0, "scaling": sc, "max_positions": 300})
    a = build_part("position", spec, {}, rt)
    b = build_part("position", spec, {}, rt)
    assert a.tables()[0].data_ptr() == b.tables()[0].data_ptr()
    s, c = P.rope_tables(range(300), P.rope_frequencies(32, 500000.0, sc))
    assert float((a.tables()[1].double().cpu() - s).abs().max()) < 2e-6
    assert float((a.tables()[0].double().cpu() - c).abs().max()) < 2e-6
    assert build_part("position", PartSpec("none"), {}, rt).tables() is None


# ------------------------------------------------------------------ a model from a spec written here

def tiny_spec(mixer_kinds, order, d=64, H=4, KVH=2, hd=16, I=96, V=128, window=None, position="rope", state_size=None,
              ffn_kinds=None, experts=3, norm_kinds=None):
    from nanoinfer_amd.config.spec import BlockSpec, LayerRun, ModelSpec, PartSpec
    if position == "rope":
        pos = PartSpec("rope", {"rotary_dim": hd, "theta": 10000.0, "scaling": None, "max_positions": 256})
    elif position == "none":
        pos = PartSpec("none")
    else:       # a position encoding registered by a test: the same constants, its own kind
        pos = PartSpec(position, {"rotary_dim": hd, "theta": 10000.0, "max_positions": 256})
    blocks = []
    for i, kind in enumerate(mixer_kinds):
        pre = f"L{i}."
        if kind == "attention":
            mixer = PartSpec("attention", {"hidden_size": d, "num_heads": H, "num_kv_heads": KVH, "head_dim": hd,
                                           "scale": None, "window": window[i] if window else None, "position": pos},
                             {"q": pre + "q", "k": pre + "k", "v": pre + "v", "o": pre + "o"})
        else:
            mixer = PartSpec(kind, {"hidden_size": d, "state_size": state_size}, {"inp": pre + "inp", "out": pre + "out"})
        if ffn_kinds is None or ffn_kinds[i] == "swiglu":
            ffn = PartSpec("swiglu", {"hidden_size": d, "intermediate_size": I},
                           {"gate": pre + "g", "up": pre + "u", "down": pre + "d"})
        else:
            ffn = PartSpec(ffn_kinds[i], {"hidden_size": d, "intermediate_size": I, "experts": experts},
                           {"router": pre + "router", "w1": pre + "w1", "w2": pre + "w2"})
        def norm(name):
            if norm_kinds is None or norm_kinds[i] == "rmsnorm":
                return PartSpec("rmsnorm", {"size": d, "eps": 1e-5}, {"weight": pre + name})
            return PartSpec(norm_kinds[i], {"size": d, "eps": 1e-5}, {"weight": pre + name, "bias": pre + name + "b"})
        blocks.append(BlockSpec("prenorm", {"mixer_norm": norm("n1"), "mixer": mixer, "ffn_norm": norm("n2"), "ffn": ffn}))
    return ModelSpec(V, d, 256, PartSpec("table", {"vocab_size": V, "hidden_size": d}, {"weight": "emb"}), blocks,
                     [LayerRun(*o) for o in order], PartSpec("rmsnorm", {"size": d, "eps": 1e-5}, {"weight": "nf"}),
                     PartSpec("linear", {"vocab_size": V, "hidden_size": d}, {"weight": "emb"}))


def random_tensors(spec, seed):
    from nanoinfer_amd.weights.loader import expected_tensors
    g = torch.Generator().manual_seed(seed)
    return {n: (1 + 0.05 * torch.randn(s, generator=g)) if len(s) == 1 else 0.08 * torch.randn(s, generator=g)
            for n, s in expected_tensors(spec).items()}


def SpecRunner(spec, tensors, dtype, page_size=8, max_tokens=512, max_step_tokens=None):
    """A runner over a spec and tensors given directly (no folder): the same model, cache manager and
    step function, through the runner's own constructor for models given as data."""
    from nanoinfer_amd.engine.runner import ModelRunner
    return ModelRunner.from_spec(spec, tensors, dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_requests=4,
                                 max_step_tokens=max_step_tokens)


def plain_spec_forward(spec, tensors, tokens, extra_mixers=None, extra_ffns=None, extra_positions=None, extra_norms=None):
    """The plain implementation applied to a spec: same functions, parts chosen by the spec."""
    T = len(tokens)
    t64 = {k: v.double() for k, v in tensors.items()}
    h = P.embedding(t64[spec.embedding.weights["weight"]], tokens)
    kv = {}

    def normed(part, h):
        if part.kind == "rmsnorm":
            return P.rmsnorm(h, t64[part.weights["weight"]], part.params["eps"])
        return extra_norms[part.kind](h, t64, part)
    for run in spec.order:
        b = spec.blocks[run.block]
        x = normed(b.mixer_norm, h)
        m = b.mixer
        if m.kind == "attention":
            p = m.params
            H, KVH, hd = p["num_heads"], p["num_kv_heads"], p["head_dim"]
            q = P.linear(x, P.permute_reverse(t64[m.weights["q"]], H)).reshape(T, H, hd)
            if run.writes_cache:
                k = P.linear(x, P.permute_reverse(t64[m.weights["k"]], KVH)).reshape(T, KVH, hd)
                v = P.linear(x, t64[m.weights["v"]]).reshape(T, KVH, hd)
            if p["position"].kind == "rope":
                pp = p["position"].params
                s, c = P.rope_tables(range(T), P.rope_frequencies(pp["rotary_dim"], pp["theta"], pp["scaling"]))
                q = P.rope_interleaved(q, s, c)
                if run.writes_cache:
                    k = P.rope_interleaved(k, s, c)
            elif p["position"].kind != "none":
                s, c = extra_positions[p["position"].kind](T, p["position"].params)
                q = P.rope_interleaved(q, s, c)
                if run.writes_cache:
                    k = P.rope_interleaved(k, s, c)
            if run.writes_cache:
                kv[run.cache] = (k, v)
            k, v = kv[run.cache]
            a = P.linear(P.causal_attention(q, k, v, range(T), window=p["window"]).reshape(T, H * hd), t64[m.weights["o"]])
        else:
            a = extra_mixers[m.kind](x, t64, m)
        h = h + a
        x = normed(b.ffn_norm, h)
        f = b.ffn
        if f.kind == "swiglu":
            h = h + P.linear(P.swiglu(P.linear(x, t64[f.weights["gate"]]), P.linear(x, t64[f.weights["up"]])), t64[f.weights["down"]])
        else:
            h = h + extra_ffns[f.kind](x, t64, f)
    return P.linear(P.rmsnorm(h, t64[spec.final_norm.weights["weight"]], spec.final_norm.params["eps"]),
                    t64[spec.head.weights["weight"]])


def step_in_portions(runner, tokens, sizes, rid="s"):
    from nanoinfer_amd.engine.runner import StepEntry
    outs, at, k = [], 0, 0
    while at < len(tokens):
        n = min(sizes[k % len(sizes)], len(tokens) - at)
        outs.append(runner.step([StepEntry(rid, tokens[at:at + n], list(range(n)))]))
        at, k = at + n, k + 1
    runner.release(rid)
    return torch.cat(outs)


def test_order_of_layers_is_data():
    """A block run twice on caches of its own, a layer that reads another layer's cache, a layer
    with a window and one without position encoding: all from one list, no new code."""
    tokens = list(random_tokens(128, 60, 1))
    cases = {
        "plain order": (["attention", "attention"], [(0, 0), (1, 1)], None, "rope"),
        "block 0 twice": (["attention", "attention"], [(0, 0), (1, 1), (0, 2)], None, "rope"),
        "layer 1 reads layer 0's cache": (["attention", "attention"], [(0, 0, True), (1, 0, False)], None, "rope"),
        "window on layer 1": (["attention", "attention"], [(0, 0), (1, 1)], [None, 9], "rope"),
        "no position encoding": (["attention"], [(0, 0)], None, "none"),
    }
    for what, (kinds, order, window, position) in cases.items():
        spec = tiny_spec(kinds, order, window=window, position=position)
        tensors = random_tensors(spec, 3)
        want = plain_spec_forward(spec, tensors, tokens)
        runner = SpecRunner(spec, tensors, "float32")
        if what == "window on layer 1":
            assert len(runner.cache.groups) == 2            # a window is another need: pages of its own
        for sizes in ([60], [7, 2, 13, 1, 1, 1]):
            got = step_in_portions(runner, tokens, sizes)
            assert rel(got, want) < TOL["float32"], (what, sizes)
        runner.cache.check()
        assert all(g.pages.num_free == g.pages.num_pages for g in runner.cache.groups)
    with pytest.raises(ValueError):
        from nanoinfer_amd.engine.model import Model
        bad = tiny_spec(["attention", "attention"], [(0, 0, False), (1, 0, True)])
        Model(bad, random_tensors(bad, 0), runtime("float32"))     # reads a cache nobody has written yet


def test_windowed_layer_gives_pages_back_while_running():
    from nanoinfer_amd.engine.runner import StepEntry
    spec = tiny_spec(["attention", "attention"], [(0, 0), (1, 1)], window=[None, 9])
    tensors = random_tensors(spec, 4)
    runner = SpecRunner(spec, tensors, "float32", page_size=4, max_tokens=256)
    tokens = list(random_tokens(128, 100, 2))
    want = plain_spec_forward(spec, tensors, tokens)
    outs = [runner.step([StepEntry("w", tokens[:20], list(range(20)))])]
    windowed = next(g for g in runner.cache.groups if g.need.window == 9)
    full = next(g for g in runner.cache.groups if g.need.window is None)
    for t in tokens[20:]:
        outs.append(runner.step([StepEntry("w", [t], [0])]))
        assert windowed.pages.num_taken <= 4                       # 9 keys span at most 3 pages, plus the new one
    assert full.pages.num_taken == 25 and windowed.tables["w"][:20] == [-1] * 20
    assert rel(torch.cat(outs), want) < TOL["float32"]
    runner.release("w")


def test_a_windowed_layer_s_pool_is_as_small_as_its_window_allows():
    """With a bound on the tokens a request brings to a step, the windowed layer's pool holds four
    requests' windows and steps, not their contexts: two requests run far past what that pool could
    hold of whole contexts, and a portion longer than the bound is refused before anything is reserved."""
    from nanoinfer_amd.engine.runner import StepEntry, StepError
    spec = tiny_spec(["attention", "attention"], [(0, 0), (1, 1)], window=[None, 9])
    tensors = random_tensors(spec, 5)
    runner = SpecRunner(spec, tensors, "float32", page_size=4, max_tokens=512, max_step_tokens=12)
    windowed = next(g for g in runner.cache.groups if g.need.window == 9)
    full = next(g for g in runner.cache.groups if g.need.window is None)
    assert full.pages.num_pages == 128 and windowed.pages.num_pages == 4 * (-(-(9 + 12) // 4) + 1) == 28
    assert all(g.kpools[c].shape[0] == g.pages.num_pages for g in runner.cache.groups for c in g.cache_ids)
    tokens = {r: list(random_tokens(128, 150, 20 + i)) for i, r in enumerate("ab")}
    want = {r: plain_spec_forward(spec, tensors, t) for r, t in tokens.items()}
    at = {r: 0 for r in tokens}
    sizes = [12, 1, 5, 1, 1, 9, 2]
    k = 0
    while any(at[r] < 150 for r in tokens):
        entries = []
        for r in tokens:
            n = min(sizes[k % len(sizes)], 150 - at[r])
            k += 1
            if n:
                entries.append(StepEntry(r, tokens[r][at[r]:at[r] + n], list(range(n))))
        out = runner.step(entries)
        row = 0
        for e in entries:
            n = len(e.tokens)
            assert rel(out[row:row + n], want[e.request][at[e.request]:at[e.request] + n]) < TOL["float32"], (e.request, at[e.request])
            row += n
            at[e.request] += n
        assert windowed.pages.num_taken <= 2 * 6
    with pytest.raises(StepError, match="sized for at most"):
        runner.step([StepEntry("c", [1] * 13, [])])
    assert not runner.cache.has("c")
    for r in tokens:
        runner.release(r)
    runner.cache.check()


# ------------------------------------------------------------------ a toy mixer with state

def register_toy_mixer():
    from nanoinfer_amd.parts.base import CacheNeed, Part, StateNeed, WeightRequest
    from nanoinfer_amd.registry import register_part

    @register_part("mixer", "toy_decay")
    class ToyDecayMixer(Part):
        """y_t = out(s_t), s_t = 0.5 * s_{t-1} + inp(x_t): a running state of fixed size per request,
        kept in a state slot between steps.  Written with library tensor operations: it shows the
        interface, it is no product kernel."""

        @classmethod
        def weight_requests(cls, spec):
            d, n = spec.params["hidden_size"], spec.params["state_size"]
            return [WeightRequest(spec.weights["inp"], (n, d)), WeightRequest(spec.weights["out"], (d, n))]

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            self.n = spec.params["state_size"]
            self.inp = rt.matrix(spec.weights["inp"], weights["inp"])
            self.out = rt.matrix(spec.weights["out"], weights["out"])

        def cache_need(self):
            return CacheNeed(state=StateNeed((self.n,), torch.float32))

        def forward(self, x, ctx, cache):
            u = (x @ self.inp.t()).float()
            states = torch.empty_like(u)
            for start, length, total, slot in zip(ctx.q_start, ctx.q_len, ctx.context_len, ctx.state_slot):
                s = cache.state[slot]
                if total == length:           # the request's first tokens: start from nothing
                    s = torch.zeros_like(s)
                for i in range(start, start + length):
                    s = 0.5 * s + u[i]
                    states[i] = s
                cache.state[slot] = s
            return states.to(x.dtype) @ self.out.t()

    return ToyDecayMixer


def plain_toy(x, t64, m):
    u = P.linear(x, t64[m.weights["inp"]])
    s = torch.zeros(u.shape[1], dtype=torch.float64)
    rows = []
    for i in range(u.shape[0]):
        s = 0.5 * s + u[i]
        rows.append(s.clone())
    return P.linear(torch.stack(rows), t64[m.weights["out"]])


def test_toy_mixer_with_state_is_registered_built_and_stepped():
    from nanoinfer_amd.engine.runner import StepEntry
    register_toy_mixer()
    spec = tiny_spec(["attention", "toy_decay", "attention"], [(0, 0), (1, 1), (2, 2)], state_size=24)
    tensors = random_tensors(spec, 5)
    runner = SpecRunner(spec, tensors, "float32", page_size=8, max_tokens=512)
    assert len(runner.cache.groups) == 1 and runner.cache.groups[0].cache_ids == [0, 2]
    assert list(runner.cache.state) == [1] and tuple(runner.cache.state[1].shape) == (4, 24)
    reqs = {"p": list(random_tokens(128, 41, 6)), "q": list(random_tokens(128, 29, 7)), "r": list(random_tokens(128, 17, 8))}
    want = {k: plain_spec_forward(spec, tensors, v, {"toy_decay": plain_toy}) for k, v in reqs.items()}
    got = {k: [] for k in reqs}
    done = {k: 0 for k in reqs}
    plan = [{"p": 5}, {"p": 3, "q": 9}, {"q": 1, "p": 1}, {"p": 20, "q": 1, "r": 17}, {"q": 18, "p": 12}]
    for stepplan in plan:
        entries = [StepEntry(k, reqs[k][done[k]:done[k] + n], list(range(n))) for k, n in stepplan.items()]
        out = runner.step(entries, end=[k for k, n in stepplan.items() if done[k] + n == len(reqs[k])])
        row = 0
        for k, n in stepplan.items():
            got[k].append(out[row:row + n])
            row += n
            done[k] += n
    for k in reqs:
        assert done[k] == len(reqs[k]) and rel(torch.cat(got[k]), want[k]) < TOL["float32"], k
    # the slot of a finished request is handed out again and starts from nothing
    out = runner.step([StepEntry("again", reqs["r"], list(range(17)))], end=["again"])
    assert rel(out, want["r"]) < TOL["float32"]
    runner.cache.check()
    assert runner.cache.slots.num_free == 4


# ------------------------------------------------------------------ a toy feed-forward with routing

def register_toy_routed_ffn():
    from nanoinfer_amd.parts.base import Part, WeightRequest
    from nanoinfer_amd.registry import register_part

    @register_part("feed_forward", "toy_routed")
    class ToyRoutedFeedForward(Part):
        """Every token goes to the one expert whose router logit (float32) is largest and is scaled by
        the softmax weight of that logit: y = p_e * W2_e relu(W1_e x).  Library tensor operations: it
        shows that a feed-forward with routing fits the interface, it is no product kernel."""

        @classmethod
        def weight_requests(cls, spec):
            d, i, e = spec.params["hidden_size"], spec.params["intermediate_size"], spec.params["experts"]
            return [WeightRequest(spec.weights["router"], (e, d)), WeightRequest(spec.weights["w1"], (e * i, d)),
                    WeightRequest(spec.weights["w2"], (e * d, i))]

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            p = spec.params
            self.d, self.i, self.e = p["hidden_size"], p["intermediate_size"], p["experts"]
            self.router = rt.vector32(spec.weights["router"], weights["router"].reshape(-1)).view(self.e, self.d)
            self.w1 = rt.matrix(spec.weights["w1"], weights["w1"]).view(self.e, self.i, self.d)
            self.w2 = rt.matrix(spec.weights["w2"], weights["w2"]).view(self.e, self.d, self.i)

        def forward(self, x, ctx):
            logits = x.float() @ self.router.t()
            prob = torch.softmax(logits, dim=-1)
            choice = logits.argmax(dim=-1)
            y = torch.zeros(x.shape[0], self.d, dtype=torch.float32, device=x.device)
            for e in range(self.e):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    hidden = torch.relu(x[rows] @ self.w1[e].t())
                    y[rows] = (hidden @ self.w2[e].t()).float() * prob[rows, e:e + 1]
            return y.to(x.dtype)

    return ToyRoutedFeedForward


def plain_routed(x, t64, f):
    p = f.params
    d, i, e = p["hidden_size"], p["intermediate_size"], p["experts"]
    router, w1, w2 = t64[f.weights["router"]], t64[f.weights["w1"]].view(e, i, d), t64[f.weights["w2"]].view(e, d, i)
    logits = P.linear(x, router)
    prob = torch.softmax(logits, dim=-1)
    rows = []
    for t in range(x.shape[0]):
        c = int(logits[t].argmax())
        rows.append(P.linear(torch.relu(P.linear(x[t:t + 1], w1[c])), w2[c])[0] * prob[t, c])
    return torch.stack(rows)


def test_toy_feed_forward_with_routing_beside_a_dense_one():
    """One model whose first layer has a routed feed-forward defined here and whose second has the
    framework's dense one: chosen per layer by the spec, stepped in portions and token by token
    through the framework's step function without a change to its files."""
    register_toy_routed_ffn()
    spec = tiny_spec(["attention", "attention"], [(0, 0), (1, 1)], ffn_kinds=["toy_routed", "swiglu"], experts=3)
    tensors = random_tensors(spec, 9)
    tensors["L0.router"] = tensors["L0.router"] * 8          # decided choices: no token sits on a tie
    tokens = list(random_tokens(128, 50, 4))
    want = plain_spec_forward(spec, tensors, tokens, extra_ffns={"toy_routed": plain_routed})
    choices = P.linear(P.rmsnorm(P.embedding(tensors["emb"].double(), tokens), tensors["L0.n1"].double(), 1e-5),
                       tensors["L0.router"].double()).argmax(-1)
    runner = SpecRunner(spec, tensors, "float32")
    assert not runner.use_graphs                           # a part that does not declare itself graph-safe keeps the steps eager
    for sizes in ([50], [9, 2, 1, 1, 17, 1]):
        got = step_in_portions(runner, tokens, sizes)
        assert rel(got, want) < TOL["float32"], sizes
    assert len(set(choices.tolist())) >= 2                  # the tokens do go to different experts
    runner.cache.check()


# ------------------------------------------------------------------ a toy norm

def register_toy_norm():
    from nanoinfer_amd.parts.base import Part, WeightRequest
    from nanoinfer_amd.registry import register_part

    @register_part("norm", "toy_centered")
    class ToyCenteredNorm(Part):
        """``(x - mean(x)) / sqrt(var(x) + eps) * w + b`` in float32, by library tensor operations: a norm with the
        family's interface and none of the optional abilities (no prologue, no addends, no half-done input): the
        block sums what is pending for it and runs it as a step of its own."""

        @classmethod
        def weight_requests(cls, spec):
            return [WeightRequest(spec.weights["weight"], (spec.params["size"],)),
                    WeightRequest(spec.weights["bias"], (spec.params["size"],))]

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            self.eps = float(spec.params["eps"])
            self.weight = rt.vector32(spec.weights["weight"], weights["weight"])
            self.bias = rt.vector32(spec.weights["bias"], weights["bias"])

        def forward(self, h, pending, rows=None):
            if rows is None and pending is not None:
                h += pending.float()                     # the residual sum, in float32, in place
            x = h if rows is None else h[rows.long()]
            mean = x.mean(dim=-1, keepdim=True)
            var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
            return (((x - mean) / torch.sqrt(var + self.eps)) * self.weight + self.bias).to(self.rt.dtype)

    return ToyCenteredNorm


def plain_centered(h, t64, part):
    mean = h.mean(dim=-1, keepdim=True)
    var = ((h - mean) ** 2).mean(dim=-1, keepdim=True)
    return (h - mean) / torch.sqrt(var + part.params["eps"]) * t64[part.weights["weight"]] + t64[part.weights["bias"]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kinds", [("toy_centered", "rmsnorm"), ("rmsnorm", "toy_centered"), ("rmsnorm", "toy_centered", "rmsnorm")])
def test_toy_norm_beside_the_frameworks_own(kinds, dtype, monkeypatch):
    """Layers whose norms are a toy norm defined here beside layers with the framework's RMSNorm, in both orders.
    Around the framework's norm the products do the norm in two halves (the one before it leaves ``h * w`` and the
    sums of squares, the one behind it divides), and where such a layer follows one with the toy norm the toy
    layer's last product leaves them for it; around the toy norm, which offers nothing of the kind, the block adds
    what is pending and runs the norm as a step of its own.  Portions, single tokens and steps of a few rows."""
    from nanoinfer_amd import kernels
    register_toy_norm()
    n = len(kinds)
    spec = tiny_spec(["attention"] * n, [(i, i) for i in range(n)], norm_kinds=list(kinds))
    tensors = random_tensors(spec, 21)
    tokens = list(random_tokens(128, 70, 6))
    if dtype == "bfloat16":
        tensors = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v) for k, v in tensors.items()}
    want = plain_spec_forward(spec, tensors, tokens, extra_norms={"toy_centered": plain_centered})
    left = []
    gemm = kernels.skinny_gemm
    monkeypatch.setattr(kernels, "skinny_gemm", lambda x, w, out, *a, **kw: (
        lambda r: (left.append(tuple(out.shape)) if isinstance(r, kernels.ScaledInput) else None, r)[1])(gemm(x, w, out, *a, **kw)))
    runner = SpecRunner(spec, tensors, dtype)
    for sizes in ([70], [9, 2, 1, 1, 17, 1, 5]):
        got = step_in_portions(runner, tokens, sizes)
        assert rel(got, want) < TOL[dtype], (kinds, sizes)
    # per step of few rows: the product before every RMSNorm that stands inside the model left its input half done
    # (the o product where the layer's norms are the framework's, the down product where the next layer's are)
    inner = sum(k == "rmsnorm" for k in kinds) + sum(k == "rmsnorm" for k in kinds[1:])
    assert len([shape for shape in left if shape[0] == 1]) % inner == 0 and any(shape[0] == 1 for shape in left)
    assert not any(shape[0] == 70 for shape in left)
    runner.cache.check()


# ------------------------------------------------------------------ a toy position encoding

def register_toy_position():
    from nanoinfer_amd.parts.base import Part
    from nanoinfer_amd.registry import register_part

    @register_part("position", "toy_sqrt")
    class SquareRootPosition(Part):
        """Rotation by sqrt(pos) * f_p instead of pos * f_p: another position encoding of the rotating
        kind, given to the attention part as tables of its own."""

        graph_safe = True

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            p = spec.params
            self.max_positions = int(p["max_positions"])
            half = p["rotary_dim"] // 2
            freq = torch.tensor([p["theta"] ** (-2.0 * j / p["rotary_dim"]) for j in range(half)], dtype=torch.float64)
            angle = torch.arange(self.max_positions, dtype=torch.float64).sqrt()[:, None] * freq[None]
            self.cos = angle.cos().float().to(rt.device).contiguous()
            self.sin = angle.sin().float().to(rt.device).contiguous()

        def tables(self):
            return self.cos, self.sin

    return SquareRootPosition


def plain_sqrt_tables(T, params):
    half = params["rotary_dim"] // 2
    freq = torch.tensor([params["theta"] ** (-2.0 * j / params["rotary_dim"]) for j in range(half)], dtype=torch.float64)
    angle = torch.arange(T, dtype=torch.float64).sqrt()[:, None] * freq[None]
    return angle.sin(), angle.cos()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_position_encoding_feeds_the_attention_part(dtype):
    """A position encoding registered here (angles sqrt(pos) * f) drives the framework's attention
    part, its fused rotation epilogue and its recorded decode steps unchanged: only tables differ."""
    from nanoinfer_amd.engine.runner import StepEntry
    register_toy_position()
    spec = tiny_spec(["attention", "attention"], [(0, 0), (1, 1)], hd=32, H=2, KVH=1, position="toy_sqrt")
    tensors = random_tensors(spec, 12)
    if dtype == "bfloat16":
        tensors = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v) for k, v in tensors.items()}
    tokens = list(random_tokens(128, 40, 5))
    want = plain_spec_forward(spec, tensors, tokens, extra_positions={"toy_sqrt": plain_sqrt_tables})
    runner = SpecRunner(spec, tensors, dtype)
    assert runner.use_graphs
    outs = [runner.step([StepEntry("s", tokens[:25], list(range(25)))])]
    for t in tokens[25:]:
        outs.append(runner.step([StepEntry("s", [t], [0])]).clone())
    runner.release("s")
    assert rel(torch.cat(outs), want) < TOL[dtype]
    # and it is no rope in disguise: the framework's own rotation gives other logits
    other = tiny_spec(["attention", "attention"], [(0, 0), (1, 1)], hd=32, H=2, KVH=1, position="rope")
    assert rel(plain_spec_forward(other, tensors, tokens), want) > 10 * TOL[dtype]
