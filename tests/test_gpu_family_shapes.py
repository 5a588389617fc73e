"""The layer sizes of the Llama 3 family (two layers each, random weights) through the engine's
step function against the plain implementation: a prompt in one portion and in two, then single
tokens one by one (recorded steps), in float32 and bfloat16.  These are the hidden widths, head
sizes and groups at which the kernels' other code paths run: head size 128, rows of 3,072 and
4,096 elements (too long for the norm prologue in bfloat16, so the separate norm kernel runs),
three query heads per kv head, an intermediate size of 14,336, the family's vocabulary; and
portions of 17 to 64 tokens, whose output and down products are cut along K in bfloat16."""
import pytest
import torch

from gpu_common import assert_close, model_folder, plain_logits, random_tokens
from tiny_configs import ALL

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["1B", "3B", "8B"])
def test_family_layer_sizes(name, dtype):
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry

    folder = model_folder(name, stored="bfloat16" if dtype == "bfloat16" else "float32")
    vocab = ALL[name]["vocab_size"]
    a = random_tokens(vocab, 75, 11)
    b = random_tokens(vocab, 41, 12)
    runner = ModelRunner(folder, dtype=dtype, page_size=16, max_tokens=256, max_requests=4)
    got_a, got_b = {}, {}
    # a: 60 tokens as one portion; b: 20 + 13 tokens in two steps, the second beside single tokens of a
    out = runner.step([StepEntry("a", a[:60], list(range(60))), StepEntry("b", b[:20], [0, 19])])
    for i in range(60):
        got_a[i] = out[i]
    got_b[0], got_b[19] = out[60], out[61]
    out = runner.step([StepEntry("a", [a[60]], [0]), StepEntry("b", b[20:33], list(range(13)))])
    got_a[60] = out[0]
    for i in range(13):
        got_b[20 + i] = out[1 + i]
    # then both one token at a time, in the same batch: recorded decode steps
    for i in range(8):
        out = runner.step([StepEntry("a", [a[61 + i]], [0]), StepEntry("b", [b[33 + i]], [0])])
        got_a[61 + i], got_b[33 + i] = out[0].clone(), out[1].clone()
    # a alone to its end
    for i in range(69, 75):
        out = runner.step([StepEntry("a", [a[i]], [0])])
        got_a[i] = out[0].clone()
    # c: portions of 40 and 24 tokens, steps of 17 to 64 rows (in bfloat16 the products onto the residual
    # stream are cut along K there and the norms add their shares)
    c = random_tokens(vocab, 64, 13)
    got_c = {}
    out = runner.step([StepEntry("c", c[:40], list(range(40)))])
    for i in range(40):
        got_c[i] = out[i].clone()
    out = runner.step([StepEntry("c", c[40:], list(range(24)))])
    for i in range(24):
        got_c[40 + i] = out[i].clone()
    runner.release("a"), runner.release("b"), runner.release("c")
    runner.cache.check()
    for tokens, got, rid in ((a, got_a, "a"), (b[:41], got_b, "b"), (c, got_c, "c")):
        want = plain_logits(folder, tuple(tokens), dtype)
        idx = sorted(got)
        assert_close(torch.stack([got[i] for i in idx]), want[idx], dtype, f"{name} {dtype} request {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_whose_cut_products_are_added_by_the_next_layer(dtype, monkeypatch):
    """At the 1B sizes a decode step's down product goes in two shares of K where no product leaves the next
    norm's input half done (here switched off; in use it is the last layer's, before the final norm).  Up to
    eight rows the next layer's first product adds them to its rows in its normalising prologue and its output
    product brings them into the residual stream (no kernel sums them); the last layer's go to the final norm.
    Steps of eight, three and one token, recorded and not, against the plain implementation."""
    from nanoinfer_amd import kernels
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry
    from nanoinfer_amd.parts import standard

    monkeypatch.setattr(kernels, "DEFER_NORMS", False)
    folder = model_folder("1B", stored="bfloat16" if dtype == "bfloat16" else "float32")
    vocab = ALL["1B"]["vocab_size"]
    prompts = [random_tokens(vocab, 30 + 7 * i, 40 + i) for i in range(8)]
    carried = []
    carries = standard.Attention.carries_addends

    def spy(self, T, addends):
        carried.append((T, addends, carries(self, T, addends)))
        return carried[-1][2]
    monkeypatch.setattr(standard.Attention, "carries_addends", spy)
    for graphs in (False, True):
        runner = ModelRunner(folder, dtype=dtype, page_size=16, max_tokens=1024, max_requests=8, use_graphs=graphs)
        for i, p in enumerate(prompts):
            runner.step([StepEntry(i, p[:-4], [])])
        got = {}
        for k, live in ((4, 8), (3, 8), (2, 3), (1, 1)):        # the eight twice: the second time as a recorded step
            out = runner.step([StepEntry(i, [prompts[i][-k]], [0]) for i in range(live)])
            for i in range(live):
                got[(i, len(prompts[i]) - k)] = out[i].clone()
        for i in range(8):
            runner.release(i)
        runner.cache.check()
        for i, p in enumerate(prompts):
            want = plain_logits(folder, tuple(p), dtype)
            at = sorted(pos for (r, pos) in got if r == i)
            assert_close(torch.stack([got[(i, pos)] for pos in at]), want[at], dtype, f"1B {dtype} request {i} graphs {graphs}")
    assert {(T, S) for T, S, _ in carried} == {(8, 2), (3, 2), (1, 2)} and all(ok for _, _, ok in carried)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["1B", "3B", "8B"])
def test_decode_steps_whose_norms_are_done_in_two_halves(name, dtype, monkeypatch):
    """Steps of few tokens at the family's layer sizes: the o and down products leave ``h * w`` and the sums of
    squares behind, the gate/up product and the next layer's q/k/v product divide in their epilogues, and no norm
    kernel runs between the first layer's and the last one's.  Steps of 1, 3, 8, 16 tokens (and 21: only the o
    product leaves there), recorded and not, against the plain implementation."""
    from nanoinfer_amd import kernels
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry

    folder = model_folder(name, stored="bfloat16" if dtype == "bfloat16" else "float32")
    vocab = ALL[name]["vocab_size"]
    prompts = [random_tokens(vocab, 20 + 3 * i, 70 + i) for i in range(24)]
    left, taken, norms = [], [], []
    gemm, rope, norm = kernels.skinny_gemm, kernels.skinny_qkv_rope, kernels.add_rmsnorm

    def spy_gemm(x, weight, out, *a, **kw):
        result = gemm(x, weight, out, *a, **kw)
        if isinstance(result, kernels.ScaledInput):
            left.append(x.shape[0])
        if isinstance(x, kernels.ScaledInput):
            taken.append(x.shape[0])
        return result

    def spy_rope(x, *a, **kw):
        if isinstance(x, kernels.ScaledInput):
            taken.append(x.shape[0])
        return rope(x, *a, **kw)

    def spy_norm(h, *a, **kw):
        norms.append(h.shape[0])
        return norm(h, *a, **kw)
    monkeypatch.setattr(kernels, "skinny_gemm", spy_gemm)
    monkeypatch.setattr(kernels, "skinny_qkv_rope", spy_rope)
    monkeypatch.setattr(kernels, "add_rmsnorm", spy_norm)
    for graphs in (False, True):
        runner = ModelRunner(folder, dtype=dtype, page_size=16, max_tokens=4096, max_requests=24, use_graphs=graphs)
        for i, p in enumerate(prompts):
            runner.step([StepEntry(i, p[:-5], [])])
        got = {}
        del left[:], taken[:], norms[:]
        for k, live in ((5, 16), (4, 16), (3, 8), (2, 3), (1, 1)):      # the sixteen twice: the second time as a recorded step
            out = runner.step([StepEntry(i, [prompts[i][-k]], [0]) for i in range(live)])
            for i in range(live):
                got[(i, len(prompts[i]) - k)] = out[i].clone()
        if not graphs:
            # two layers: o and down of the first, o of the second leave; gate/up twice and the second q/k/v take
            # (at the 1B sizes in float32 the down product is cut along K to fill the chip and leaves nothing; in
            # bfloat16 it runs whole on halved tiles from five rows on)
            n = 2 if (name, dtype) == ("1B", "float32") else 3
            assert sorted(set(left)) == [1, 3, 8, 16] and left.count(8) == n and taken.count(8) == n, (left, taken)
            assert left.count(3) == (2 if name == "1B" else 3)
            assert norms.count(8) <= 2, "the first layer's first norm at most, and the last norm on the wanted rows"
        rows = [(i, 5) for i in range(16, 24)] + [(i, 3) for i in range(8, 16)] + [(i, 2) for i in range(3, 8)]      # 21 rows
        out = runner.step([StepEntry(i, [prompts[i][-k]], [0]) for i, k in rows])
        for j, (i, k) in enumerate(rows):
            got[(i, len(prompts[i]) - k)] = out[j].clone()
        for i in range(24):
            runner.release(i)
        runner.cache.check()
        for i, p in enumerate(prompts):
            want = plain_logits(folder, tuple(p), dtype)
            at = sorted(pos for (r, pos) in got if r == i)
            if at:
                assert_close(torch.stack([got[(i, pos)] for pos in at]), want[at], dtype, f"{name} {dtype} request {i} graphs {graphs}")
