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
    """At the 1B sizes a decode step's down product goes in two shares of K.  Up to eight rows the next
    layer's first product adds them to its rows in its normalising prologue and its output product brings
    them into the residual stream (no kernel sums them); the last layer's go to the final norm.  Steps of
    eight, three and one token, recorded and not, against the plain implementation."""
    from nanoinfer_amd.engine.runner import ModelRunner, StepEntry
    from nanoinfer_amd.parts import standard

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
