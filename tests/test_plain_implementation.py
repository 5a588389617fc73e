"""Pins of the plain implementation (tests/plain_llama.py) by what fixes it beside the text of
the reference: vectors the reference's own tests hold, special cases that reduce to a library
routine, and invariants.  Each is chosen so that a plausible mistake fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_llama as P
from tiny_configs import TINY, TINY_A, TINY_B

F64 = torch.float64


# ------------------------------------------------------------------ RMSNorm

def test_rmsnorm_reference_vector():
    # test/test_op/test_layer_rmsnorm.cpp:112-136: input [1..dim], weight 1 -> i / sqrt(mean(i^2) + 1e-5)
    dim = 8
    x = torch.arange(1, dim + 1, dtype=F64)[None]
    want = x / math.sqrt(float((x * x).mean()) + 1e-5)
    assert torch.allclose(P.rmsnorm(x, torch.ones(dim), 1e-5), want, atol=1e-12)


def test_rmsnorm_unit_rms_and_weight_after_normalisation():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 33, generator=g, dtype=F64) * 7
    y = P.rmsnorm(x, torch.ones(33), 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=F64), atol=1e-12)
    w = torch.randn(33, generator=g, dtype=F64)
    assert torch.allclose(P.rmsnorm(x, w, 0.0), y * w, atol=1e-12)       # weight multiplies, is not added
    assert torch.allclose(P.rmsnorm(3 * x, w, 0.0), P.rmsnorm(x, w, 0.0), atol=1e-12)  # scale invariance
    # eps is inside the root, added to the mean (not to the sum, not outside the root)
    x1 = torch.tensor([[3.0, 4.0]], dtype=F64)
    assert torch.allclose(P.rmsnorm(x1, torch.ones(2), 2.5), x1 / math.sqrt(12.5 + 2.5))


# ------------------------------------------------------------------ linear

def test_linear_reference_vector():
    # test/test_cuda_kernel/test_matmul_kernel.cpp:30-99: ones x 0.5, K = 128 -> 64
    out = P.linear(torch.ones(3, 128), torch.full((7, 128), 0.5))
    assert out.shape == (3, 7) and torch.all(out == 64.0)


def test_linear_is_x_times_w_transposed():
    g = torch.Generator().manual_seed(1)
    x, w = torch.randn(4, 6, generator=g, dtype=F64), torch.randn(5, 6, generator=g, dtype=F64)
    assert torch.allclose(P.linear(x, w), F.linear(x, w))


# ------------------------------------------------------------------ rotation

def test_rope_table_golden_loop():
    # test/test_cuda_kernel/test_rope_kernel.cpp:146-168: freq = 1 / 10000^((i/2*2)/hd), val = pos * freq
    hd, n = 16, 9
    freqs = P.rope_frequencies(hd, 10000.0, None)
    sin, cos = P.rope_tables(range(n), freqs)
    for pos in range(n):
        for p in range(hd // 2):
            val = np.float32(pos) * np.float32(1.0 / np.power(np.float32(10000.0), np.float32(2 * p) / np.float32(hd)))
            assert abs(float(sin[pos, p]) - math.sin(float(val))) < 1e-6
            assert abs(float(cos[pos, p]) - math.cos(float(val))) < 1e-6
    assert torch.all(sin[0] == 0) and torch.all(cos[0] == 1)


def test_rope_quarter_turn_reference_vector():
    # test/test_cuda_kernel/test_rope_kernel.cpp:20-118: sin = 1, cos = 0 turns the pair (2, 2) into (-2, 2)
    x = torch.tensor([[[2.0, 2.0], [2.0, 2.0]]], dtype=F64)          # one token, two heads of size 2
    out = P.rope_interleaved(x, torch.ones(1, 1, dtype=F64), torch.zeros(1, 1, dtype=F64))
    assert torch.allclose(out, torch.tensor([[[-2.0, 2.0], [-2.0, 2.0]]], dtype=F64))


def test_rope_llama3_scaling_branches():
    s = TINY_B["rope_scaling"]
    hd, theta = TINY_B["head_dim"], TINY_B["rope_theta"]
    base = P.rope_frequencies(hd, theta, None)
    scaled = P.rope_frequencies(hd, theta, s)
    wl = 2 * math.pi / base
    lo, hi = s["original_max_position_embeddings"] / s["low_freq_factor"], \
        s["original_max_position_embeddings"] / s["high_freq_factor"]
    kinds = set()
    for p in range(hd // 2):
        if wl[p] >= lo:
            kinds.add("long")
            assert scaled[p] == pytest.approx(base[p] / s["factor"], rel=1e-6)
        elif wl[p] > hi:
            kinds.add("middle")
            assert base[p] / s["factor"] < scaled[p] < base[p]
        else:
            kinds.add("short")
            assert scaled[p] == base[p]
    assert kinds == {"long", "middle", "short"}      # the tiny configuration reaches all three
    # the blend is continuous at both ends of the middle band
    one = dict(s, factor=1.0)
    assert np.allclose(P.rope_frequencies(hd, theta, one), base, rtol=1e-6)
    # test_rope_kernel.cpp:233-239: with the 1B constants the slowest pair barely turns at position 1
    f = P.rope_frequencies(64, 500000.0, {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                          "original_max_position_embeddings": 8192})
    assert abs(math.sin(float(f[-1]))) < 0.1 and f[-1] == pytest.approx(1 / 500000 ** (62 / 64) / 32, rel=1e-5)


def test_rope_llama3_frequencies_as_numbers():
    """The three bands, and above all the blend of the middle one, against numbers worked out from
    the rule independently (tests/rope_literals.py): a blend the other way round, a band edge
    moved to the other constant or a factor applied twice all miss them by far more than 1e-5."""
    from rope_literals import CASES
    for hd, theta, scaling, pairs in CASES:
        f = P.rope_frequencies(hd, theta, scaling)
        assert f.dtype == np.float32 and f.shape == (hd // 2,)
        for p, (band, value) in pairs.items():
            assert float(f[p]) == pytest.approx(value, rel=1e-5), (hd, p, band)
    assert {band for _, _, _, pairs in CASES for band, _ in pairs.values()} == {"short", "middle", "long"}


def test_rope_llama3_blend_meets_both_neighbours_at_the_band_edges():
    """With a factor other than 1: a pair whose wavelength lies a hair inside the middle band has
    nearly the frequency of a pair a hair outside it, at the long edge (f / factor) and at the short
    edge (f).  The wavelength of pair 3 is held fixed and the band is moved across it."""
    hd, theta, p = 32, 10000.0, 3
    base = float(P.rope_frequencies(hd, theta, None)[p])
    wl = 2 * math.pi / base
    for edge, expect in (("long", base / 8.0), ("short", base)):
        got = []
        for nudge in (1 - 2e-4, 1 + 2e-4):
            # long edge: wl = orig / low; short edge: wl = orig / high
            orig = wl * (1.0 if edge == "long" else 4.0) * nudge
            s = {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": orig}
            got.append(float(P.rope_frequencies(hd, theta, s)[p]))
        assert got[0] == pytest.approx(expect, rel=2e-3) and got[1] == pytest.approx(expect, rel=2e-3), (edge, got)
        assert got[0] != got[1]                      # one of them really is in the middle band


def test_rope_invariants():
    g = torch.Generator().manual_seed(2)
    hd = 16
    freqs = P.rope_frequencies(hd, 10000.0, None)
    q = torch.randn(1, 1, hd, generator=g, dtype=F64)
    k = torch.randn(1, 1, hd, generator=g, dtype=F64)

    def rot(x, pos):
        s, c = P.rope_tables([pos], freqs)
        return P.rope_interleaved(x, s, c)

    assert torch.allclose(rot(q, 0), q)                                       # position 0 is the identity
    assert torch.allclose(rot(q, 37).norm(), q.norm())                        # a rotation keeps the norm
    pairs = rot(q, 37).reshape(-1, 2).norm(dim=1)
    assert torch.allclose(pairs, q.reshape(-1, 2).norm(dim=1))                # ... of every pair
    d1 = (rot(q, 5) * rot(k, 2)).sum()
    d2 = (rot(q, 105) * rot(k, 102)).sum()
    assert torch.allclose(d1, d2, atol=1e-4)    # only the distance counts (angles are float32 products)
    assert not torch.allclose(d1, (rot(q, 5) * rot(k, 3)).sum(), atol=1e-3)
    # direction of the turn: a positive angle turns (1, 0) towards (cos, +sin)
    e = torch.zeros(1, 1, hd, dtype=F64)
    e[0, 0, 0] = 1.0
    out = rot(e, 1)
    assert out[0, 0, 0] == pytest.approx(math.cos(1.0), abs=1e-6) and out[0, 0, 1] == pytest.approx(math.sin(1.0), abs=1e-6)


def rotate_half_rope(x, sin, cos):
    """The checkpoint's own convention, written independently: pairs (j, j + hd/2)."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    s, c = sin[:, None, :], cos[:, None, :]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def test_permuted_interleaved_equals_half_split():
    # tools/export_llama3.py:571-583: permute_reverse makes neighbours of the pairs (j, j + hd/2)
    g = torch.Generator().manual_seed(3)
    H, hd, d, T = 3, 8, 10, 5
    w = torch.randn(H * hd, d, generator=g, dtype=F64)
    x = torch.randn(T, d, generator=g, dtype=F64)
    freqs = P.rope_frequencies(hd, 10000.0, None)
    sin, cos = P.rope_tables(range(T), freqs)
    a = P.rope_interleaved(P.linear(x, P.permute_reverse(w, H)).reshape(T, H, hd), sin, cos)
    b = rotate_half_rope(P.linear(x, w).reshape(T, H, hd), sin, cos)
    # same numbers in another order inside each head: inner products agree, and a[2j], a[2j+1] = b[j], b[j+hd/2]
    assert torch.allclose(a[..., 0::2], b[..., :hd // 2]) and torch.allclose(a[..., 1::2], b[..., hd // 2:])


# ------------------------------------------------------------------ attention

def test_attention_equals_library_when_heads_are_not_grouped():
    g = torch.Generator().manual_seed(4)
    T, H, hd = 9, 3, 8
    q, k, v = (torch.randn(T, H, hd, generator=g, dtype=F64) for _ in range(3))
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    assert torch.allclose(P.causal_attention(q, k, v, range(T)), want.transpose(0, 1), atol=1e-12)


def test_attention_grouping_is_by_consecutive_heads():
    g = torch.Generator().manual_seed(5)
    T, H, KVH, hd = 7, 6, 2, 4
    q = torch.randn(T, H, hd, generator=g, dtype=F64)
    k, v = (torch.randn(T, KVH, hd, generator=g, dtype=F64) for _ in range(2))
    kk, vv = k.repeat_interleave(H // KVH, dim=1), v.repeat_interleave(H // KVH, dim=1)   # heads 0,1,2 -> kv 0
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True)
    assert torch.allclose(P.causal_attention(q, k, v, range(T)), want.transpose(0, 1), atol=1e-12)


def test_attention_reference_vector_and_special_cases():
    # test/test_cuda_kernel/test_paged_attention_kernel.cpp:18-84: K = 0.1, V = 0.2, ctx 10, hd 128, 4 heads on 2
    T, H, KVH, hd = 10, 4, 2, 128
    out = P.causal_attention(torch.full((T, H, hd), 0.3), torch.full((T, KVH, hd), 0.1), torch.full((T, KVH, hd), 0.2),
                             range(T))
    assert torch.allclose(out, torch.full((T, H, hd), 0.2, dtype=F64))
    g = torch.Generator().manual_seed(6)
    q = torch.randn(5, 2, 4, generator=g, dtype=F64)
    v = torch.randn(5, 1, 4, generator=g, dtype=F64)
    out = P.causal_attention(q, torch.zeros(5, 1, 4), v, range(5))
    for t in range(5):        # equal keys -> the mean of the values seen so far; the first token sees itself only
        assert torch.allclose(out[t, 0], v[:t + 1, 0].mean(0))
    # a key in the future must not count: make the last key huge
    k = torch.zeros(5, 1, 4, dtype=F64)
    k[4] = 100.0
    out2 = P.causal_attention(q.abs(), k, v, range(5))
    assert torch.allclose(out2[:4], P.causal_attention(q.abs(), torch.zeros(5, 1, 4), v, range(5))[:4])
    # the scale is 1/sqrt(hd): with one hot key the weights follow exp(q.k / sqrt(hd))
    q1 = torch.zeros(2, 1, 4, dtype=F64)
    q1[1, 0, 0] = 2.0
    k1 = torch.zeros(2, 1, 4, dtype=F64)
    k1[0, 0, 0] = 3.0
    v1 = torch.tensor([[[1.0, 0, 0, 0]], [[0.0, 0, 0, 0]]], dtype=F64)
    w = math.exp(6.0 / 2.0) / (math.exp(6.0 / 2.0) + 1.0)
    assert P.causal_attention(q1, k1, v1, range(2))[1, 0, 0] == pytest.approx(w)


def test_attention_window():
    g = torch.Generator().manual_seed(7)
    T, hd, W = 12, 4, 5
    q, k, v = (torch.randn(T, 1, hd, generator=g, dtype=F64) for _ in range(3))
    out = P.causal_attention(q, k, v, range(T), window=W)
    mask = torch.ones(T, T, dtype=torch.bool).tril() & ~torch.ones(T, T, dtype=torch.bool).tril(-W)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), attn_mask=mask)
    assert torch.allclose(out, want.transpose(0, 1), atol=1e-12)


# ------------------------------------------------------------------ feed-forward, embedding

def test_swiglu_reference_vectors():
    # test/test_op/test_layer_swiglu.cpp:65-108: silu(1) * 1 = 0.7310586; gate 0 -> 0
    assert float(P.swiglu(torch.ones(1), torch.ones(1))) == pytest.approx(0.7310586, abs=1e-6)
    assert float(P.swiglu(torch.zeros(1), torch.full((1,), 5.0))) == 0.0
    g = torch.Generator().manual_seed(8)
    a, b = torch.randn(50, generator=g, dtype=F64), torch.randn(50, generator=g, dtype=F64)
    assert torch.allclose(P.swiglu(a, b), F.silu(a) * b)       # the activation is on the first argument


def test_embedding_rows_and_range():
    table = torch.arange(12, dtype=F64).reshape(4, 3)
    assert torch.equal(P.embedding(table, [2, 0]), table[[2, 0]])
    with pytest.raises(IndexError):
        P.embedding(table, [4])
    with pytest.raises(IndexError):
        P.embedding(table, [-1])


# ------------------------------------------------------------------ the whole model, a second way

def vectorised_forward(config, tensors, tokens):
    """The same model written once more in library routines and the checkpoint's own rotation
    convention (pairs (j, j + hd/2), no permutation).  If a norm sat in the wrong place in either
    version, or a residual were missing, the two would differ."""
    H, KVH = config["num_attention_heads"], config["num_key_value_heads"]
    d = config["hidden_size"]
    hd = config.get("head_dim") or d // H
    eps = config["rms_norm_eps"]
    T = len(tokens)
    scaling = config.get("rope_scaling")
    freqs = P.rope_frequencies(hd, config["rope_theta"], scaling)
    sin, cos = P.rope_tables(range(T), freqs)

    def norm(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w

    h = F.embedding(torch.tensor(tokens), tensors["model.embed_tokens.weight"])
    for i in range(config["num_hidden_layers"]):
        pre = f"model.layers.{i}."
        x = norm(h, tensors[pre + "input_layernorm.weight"])
        q = rotate_half_rope(F.linear(x, tensors[pre + "self_attn.q_proj.weight"]).view(T, H, hd), sin, cos)
        k = rotate_half_rope(F.linear(x, tensors[pre + "self_attn.k_proj.weight"]).view(T, KVH, hd), sin, cos)
        v = F.linear(x, tensors[pre + "self_attn.v_proj.weight"]).view(T, KVH, hd)
        k, v = k.repeat_interleave(H // KVH, 1), v.repeat_interleave(H // KVH, 1)
        a = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
        h = h + F.linear(a.transpose(0, 1).reshape(T, H * hd), tensors[pre + "self_attn.o_proj.weight"])
        x = norm(h, tensors[pre + "post_attention_layernorm.weight"])
        h = h + F.linear(F.silu(F.linear(x, tensors[pre + "mlp.gate_proj.weight"]))
                         * F.linear(x, tensors[pre + "mlp.up_proj.weight"]), tensors[pre + "mlp.down_proj.weight"])
    h = norm(h, tensors["model.norm.weight"])
    head = tensors["model.embed_tokens.weight"] if config.get("tie_word_embeddings") else tensors["lm_head.weight"]
    return F.linear(h, head)


@pytest.mark.parametrize("name", sorted(TINY))
def test_whole_model_two_ways(name, tmp_path):
    import nanoinfer_amd  # noqa: F401
    from nanoinfer_amd.weights.loader import make_random_model

    make_random_model(str(tmp_path), TINY[name], seed=5, dtype="float32")
    config, tensors = P.read_model_folder(str(tmp_path))
    g = torch.Generator().manual_seed(9)
    tokens = torch.randint(0, config["vocab_size"], (23,), generator=g).tolist()
    a = P.forward(config, tensors, tokens)
    b = vectorised_forward(config, tensors, tokens)
    assert a.shape == (23, config["vocab_size"])
    assert float((a - b).abs().max()) < 1e-9 * max(1.0, float(a.abs().max()))
    # causality of the whole: logits of a prefix do not change when tokens follow
    assert torch.allclose(P.forward(config, tensors, tokens[:10]), a[:10], atol=1e-10)


def test_whole_model_shift_of_positions(tmp_path):
    """Without frequency scaling only distances count: starting the sequence at position 40
    changes the logits by rounding of the float32 angles only."""
    import nanoinfer_amd  # noqa: F401
    from nanoinfer_amd.weights.loader import make_random_model

    make_random_model(str(tmp_path), TINY_A, seed=6, dtype="float32")
    config, tensors = P.read_model_folder(str(tmp_path))
    tokens = list(range(3, 20))
    a = P.forward(config, tensors, tokens)
    b = P.forward(config, tensors, tokens, first_position=40)
    assert float((a - b).abs().max()) < 1e-5


# ------------------------------------------------------------------ sampling

def test_argmax_lowest_index_on_ties():
    # test/test_cuda_kernel/test_argmax_kernel.cpp:18-65 plants maxima; cuda/argmax_kernel.cu:27 keeps the lowest index
    x = torch.zeros(10000, dtype=F64)
    for at in (100, 5000, 9999, 0):
        y = x.clone()
        y[at] = 10.0
        assert P.argmax(y) == at
    y = x.clone()
    y[7] = y[3] = 2.0
    assert P.argmax(y) == 3


def test_repetition_penalty_reference_vector():
    # test/test_engine/test_sampling.cpp:112-148
    logits = torch.tensor([2.0, -1.0, 3.0, 0.0, -2.0, 1.0, 0.5, -0.5, 1.5, -1.5], dtype=F64)
    out = P.repetition_penalty(logits, [0, 1, 4], 1.5)
    assert out[0] == pytest.approx(2.0 / 1.5) and out[1] == pytest.approx(-1.5) and out[4] == pytest.approx(-3.0)
    assert out[2] == 3.0 and out[5] == 1.0 and out[3] == 0.0
    assert torch.equal(P.repetition_penalty(logits, [0, 0, 0], 1.5), P.repetition_penalty(logits, [0], 1.5))


def test_temperature_and_filters():
    logits = torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=F64)
    assert torch.equal(P.temperature_scale(logits, 0.5), logits * 2)      # test_sampling.cpp:234-300
    assert torch.equal(P.temperature_scale(logits, 2.0), logits * 0.5)
    assert torch.equal(P.temperature_scale(logits, 1.0), logits) and torch.equal(P.temperature_scale(logits, 0.0), logits)
    p = P.filtered_distribution(logits, top_k=1, top_p=1.0)              # top-k = 1 is argmax (test_sampling.cpp:353-405)
    assert p[3] == 1.0 and p.sum() == 1.0
    p = P.filtered_distribution(logits, top_k=0, top_p=1.0)
    assert torch.allclose(p, torch.softmax(logits, 0))
    p = P.filtered_distribution(logits, top_k=2, top_p=1.0)
    assert torch.allclose(p[2:], torch.softmax(logits[2:], 0)) and p[0] == p[1] == 0
    big = torch.tensor([0.0, 10.0, 0.0, 0.0], dtype=F64)                 # one dominant token (test_sampling.cpp:444-479)
    p = P.filtered_distribution(big, top_k=0, top_p=0.9)
    assert p[1] == 1.0
    sm = torch.softmax(logits, 0)                                         # 0.032, 0.087, 0.237, 0.644
    p = P.filtered_distribution(logits, top_k=0, top_p=0.7)               # 0.644 < 0.7 <= 0.644 + 0.237
    assert p[0] == p[1] == 0 and torch.allclose(p[2:], sm[2:] / sm[2:].sum())


def test_inverse_cdf_walks_in_vocabulary_order():
    probs = torch.tensor([0.1, 0.0, 0.6, 0.3], dtype=F64)
    assert P.inverse_cdf(probs, 0.05) == 0 and P.inverse_cdf(probs, 0.1) == 0
    assert P.inverse_cdf(probs, 0.11) == 2 and P.inverse_cdf(probs, 0.7) == 2
    assert P.inverse_cdf(probs, 0.71) == 3 and P.inverse_cdf(probs, 1.0) == 3
