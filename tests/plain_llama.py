"""A plain, slow Llama forward: whole sequences, no cache, float64, one function per part.

This is the oracle of the test-suite.  It is written from the formulas of the
reference (cited at every function as file:line from the reference's root), shares no code
with ``nanoinfer_amd`` and reads a model folder with the ``safetensors`` package
and ``json`` only.

Deliberate choices, stated once:

* Arithmetic is float64 on the CPU; only the rotation frequencies and angles are
  formed in float32, as the reference forms them, because they are inputs of the
  model and not rounding of it.
* The reference rotates *interleaved* pairs ``(2p, 2p+1)`` and therefore permutes
  the rows of ``q_proj``/``k_proj`` when it exports a Hugging Face checkpoint.  The
  oracle does the same two things (``permute_reverse`` then ``rope_interleaved``);
  the engine keeps the file's row order and rotates pairs ``(p, p + hd/2)``.  The
  two are equal up to summation order, so agreement checks both.
* The reference divides the softmax by ``sum + 1e-6``.  After the maximum is
  subtracted ``sum >= 1``; the term guards nothing and is left out here and in
  the engine.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

F64 = torch.float64


# --------------------------------------------------------------------------- parts

def embedding(table: torch.Tensor, ids: Sequence[int]) -> torch.Tensor:
    """``h[t, :] = E[id[t], :]``, an id outside the table is an error.

    src/op/kernels/cpu/embedding_kernel.cpp:25-51 (aborts on ``token >= vocab``).
    """
    vocab = table.shape[0]
    for t in ids:
        if not 0 <= int(t) < vocab:
            raise IndexError(f"token id {t} outside vocabulary of {vocab}")
    return table.to(F64)[torch.tensor(list(ids), dtype=torch.long)]


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``y_j = x_j * rsqrt(mean(x^2) + eps) * w_j`` per row.

    src/op/kernels/cpu/rmsnorm_kernel.cpp:78-82, src/op/kernels/cuda/rmsnorm_kernel.cu:50-103.
    """
    x = x.to(F64)
    mean_sq = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return (x * (1.0 / torch.sqrt(mean_sq + eps))) * weight.to(F64)


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``y = x . W^T`` with ``W`` stored ``[out, in]``, no bias.

    src/op/kernels/cuda/matmul_kernel.cu:76-86, src/op/kernels/cpu/matmul_kernel.cpp:33-82.
    """
    return x.to(F64) @ weight.to(F64).t()


def rope_frequencies(head_dim: int, theta: float, scaling: Optional[dict]) -> np.ndarray:
    """Rotation frequency of each pair, float32 arithmetic as in the reference.

    ``f_p = 1 / theta^(2p/hd)``; with llama3 scaling ``wl = 2*pi/f_p`` decides between
    ``f_p / factor`` (long waves), a blend (middle band) and ``f_p`` (short waves).
    src/op/kernels/cpu/rope_kernel.cpp:121-139, src/op/kernels/cuda/rope_kernel.cu:108-127.
    """
    f32 = np.float32
    freqs = np.zeros(head_dim // 2, dtype=f32)
    for p in range(head_dim // 2):
        exponent = f32(f32(2 * p) / f32(head_dim))
        freq = f32(1.0) / f32(np.power(f32(theta), exponent, dtype=f32))
        if scaling is not None:
            factor = f32(scaling["factor"])
            low = f32(scaling["low_freq_factor"])
            high = f32(scaling["high_freq_factor"])
            orig = f32(scaling["original_max_position_embeddings"])
            wavelen = f32(f32(2.0) * f32(math.pi) / freq)
            low_freq_wavelen = f32(orig / low)
            high_freq_wavelen = f32(orig / high)
            if wavelen >= low_freq_wavelen:
                freq = f32(freq / factor)
            elif wavelen > high_freq_wavelen:
                smooth = f32(f32(orig / wavelen - low) / f32(high - low))
                freq = f32(f32(f32(1.0) - smooth) * freq / factor + smooth * freq)
        freqs[p] = freq
    return freqs


def rope_tables(positions: Sequence[int], freqs: np.ndarray):
    """``sin/cos[pos, p]`` of the float32 product ``pos * f_p``.

    src/op/kernels/cpu/rope_kernel.cpp:142-152 (both lanes of a pair hold the same value;
    one column per pair is kept here).
    """
    pos = np.asarray(list(positions), dtype=np.float32)[:, None]
    angle = (pos * freqs[None, :].astype(np.float32)).astype(np.float32)
    angle64 = torch.from_numpy(angle.astype(np.float64))
    return torch.sin(angle64), torch.cos(angle64)


def rope_interleaved(x: torch.Tensor, sin: torch.Tensor, cos: torch.Tensor) -> torch.Tensor:
    """Rotate pairs ``(x[2p], x[2p+1])`` of every head: ``x0*cos - x1*sin, x0*sin + x1*cos``.

    ``x`` is ``[T, heads, hd]``, ``sin``/``cos`` are ``[T, hd/2]``.
    src/op/kernels/cpu/rope_kernel.cpp:68-93, src/op/kernels/cuda/rope_kernel.cu:32-84.
    """
    x = x.to(F64)
    x0 = x[..., 0::2]
    x1 = x[..., 1::2]
    s = sin[:, None, :]
    c = cos[:, None, :]
    out = torch.empty_like(x)
    out[..., 0::2] = x0 * c - x1 * s
    out[..., 1::2] = x0 * s + x1 * c
    return out


def permute_reverse(w: torch.Tensor, n_heads: int) -> torch.Tensor:
    """Row permutation that turns a Hugging Face q/k projection into the interleaved order.

    Within each head new row ``2j`` is old row ``j`` and new row ``2j+1`` is old row ``j + hd/2``.
    tools/export_llama3.py:571-583.
    """
    out_dim, in_dim = w.shape
    return w.reshape(n_heads, 2, out_dim // n_heads // 2, in_dim).transpose(1, 2).reshape(out_dim, in_dim)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: Sequence[int],
                     window: Optional[int] = None) -> torch.Tensor:
    """Grouped-query causal attention of one whole sequence, key by key.

    ``q`` is ``[T, H, hd]``, ``k``/``v`` are ``[T, KVH, hd]``; query head ``h`` reads key head
    ``h // (H / KVH)``; the query at position ``P`` sees keys ``0..P`` (those within ``window``
    of it when a window is given, which Llama never has); scores are scaled by ``1/sqrt(hd)``,
    softmax subtracts the maximum.
    src/op/kernels/cpu/prefill_attention_kernel.cpp:95-157,
    src/op/kernels/cpu/paged_attention_kernel.cpp:85-132 (``kv_head = head / (H/KVH)``).
    """
    T, H, hd = q.shape
    KVH = k.shape[1]
    group = H // KVH
    scale = 1.0 / math.sqrt(hd)
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    out = torch.zeros(T, H, hd, dtype=F64)
    pos = list(positions)
    for t in range(T):
        lo = 0
        if window is not None:
            lo = max(0, t + 1 - window)
        assert pos[t] - pos[0] == t, "positions of a whole sequence are consecutive"
        for h in range(H):
            g = h // group
            scores = (k[lo:t + 1, g, :] @ q[t, h, :]) * scale
            m = scores.max()
            e = torch.exp(scores - m)
            p = e / e.sum()
            out[t, h, :] = p @ v[lo:t + 1, g, :]
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``g / (1 + exp(-g)) * u``.  src/op/kernels/cpu/swiglu_kernel.cpp:25-40."""
    gate = gate.to(F64)
    return gate / (1.0 + torch.exp(-gate)) * up.to(F64)


# --------------------------------------------------------------------------- model

def read_model_folder(folder: str):
    """config.json as a dict and every tensor of model.safetensors as float64."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    tensors: Dict[str, torch.Tensor] = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as fh:
        for name in fh.keys():
            tensors[name] = fh.get_tensor(name).to(F64)
    return config, tensors


def round_to_bfloat16(tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The matrices as a bfloat16 engine holds them (vectors of a norm stay as stored)."""
    out = {}
    for name, t in tensors.items():
        out[name] = t.to(torch.float32).to(torch.bfloat16).to(F64) if t.dim() == 2 else t
    return out


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens: Sequence[int],
            first_position: int = 0) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole sequence.

    Order of the parts: src/model/llama.cpp:297-386 (embedding, per layer norm -> q,k,v ->
    rotation -> attention -> o -> residual -> norm -> gate,up -> SwiGLU -> down -> residual,
    then the last norm and the head, which is the embedding matrix when weights are tied:
    src/model/llama.cpp:651-661).
    """
    H = config["num_attention_heads"]
    KVH = config.get("num_key_value_heads", H)
    d = config["hidden_size"]
    hd = config.get("head_dim") or d // H
    eps = config["rms_norm_eps"]
    theta = config.get("rope_theta", 10000.0)
    scaling = config.get("rope_scaling")
    if scaling is not None and scaling.get("rope_type", scaling.get("type")) in (None, "default"):
        scaling = None
    T = len(tokens)
    positions = [first_position + i for i in range(T)]
    freqs = rope_frequencies(hd, theta, scaling)
    sin, cos = rope_tables(positions, freqs)

    h = embedding(tensors["model.embed_tokens.weight"], tokens)
    for i in range(config["num_hidden_layers"]):
        pre = f"model.layers.{i}."
        x = rmsnorm(h, tensors[pre + "input_layernorm.weight"], eps)
        wq = permute_reverse(tensors[pre + "self_attn.q_proj.weight"], H)
        wk = permute_reverse(tensors[pre + "self_attn.k_proj.weight"], KVH)
        q = linear(x, wq).reshape(T, H, hd)
        k = linear(x, wk).reshape(T, KVH, hd)
        v = linear(x, tensors[pre + "self_attn.v_proj.weight"]).reshape(T, KVH, hd)
        q = rope_interleaved(q, sin, cos)
        k = rope_interleaved(k, sin, cos)
        a = causal_attention(q, k, v, positions).reshape(T, H * hd)
        h = h + linear(a, tensors[pre + "self_attn.o_proj.weight"])
        x = rmsnorm(h, tensors[pre + "post_attention_layernorm.weight"], eps)
        g = linear(x, tensors[pre + "mlp.gate_proj.weight"])
        u = linear(x, tensors[pre + "mlp.up_proj.weight"])
        h = h + linear(swiglu(g, u), tensors[pre + "mlp.down_proj.weight"])
    h = rmsnorm(h, tensors["model.norm.weight"], eps)
    head = tensors["model.embed_tokens.weight"] if config.get("tie_word_embeddings", False) \
        else tensors["lm_head.weight"]
    return linear(h, head)


# --------------------------------------------------------------------------- sampling

def argmax(logits: torch.Tensor) -> int:
    """Index of the largest logit, the lowest index among equals.

    src/op/kernels/cpu/argmax_kernel.cpp:23-41 (``std::max_element`` keeps the first),
    src/op/kernels/cuda/argmax_kernel.cu:27.
    """
    best = 0
    for i in range(1, logits.shape[0]):
        if logits[i] > logits[best]:
            best = i
    return best


def repetition_penalty(logits: torch.Tensor, generated: Sequence[int], penalty: float) -> torch.Tensor:
    """For every id already generated: ``l > 0 ? l / p : l * p`` (each id once).

    src/op/kernels/cpu/sampling_kernel.cpp:28-60, src/op/kernels/cuda/sampling_kernel.cu:38-60.
    """
    out = logits.clone()
    for t in set(int(g) for g in generated):
        out[t] = out[t] / penalty if out[t] > 0 else out[t] * penalty
    return out


def temperature_scale(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """``l * (1/T)``, untouched for ``T <= 0`` and ``T == 1``.

    src/op/kernels/cuda/sampling_kernel.cu:73-88.
    """
    if temperature <= 0 or temperature == 1.0:
        return logits.clone()
    return logits * (1.0 / temperature)


def filtered_distribution(logits: torch.Tensor, top_k: int, top_p: float) -> torch.Tensor:
    """Probabilities after top-k and top-p, renormalised, in vocabulary order.

    Keep the logits that are at least the k-th largest, softmax, then walk the descending order
    until the mass reaches ``top_p`` and keep every token at least as probable as the one where
    it did; renormalise.  Equal values at a cut are kept together (the reference's GPU kernel
    cuts by a threshold on the value as well, src/op/kernels/cuda/sampling_kernel.cu:202-296).
    Order of the stages: src/op/kernels/cpu/sampling_kernel.cpp:134-180,
    src/sampler/configurable_sampler.cpp:93-120.
    """
    V = logits.shape[0]
    order = sorted(range(V), key=lambda i: (-float(logits[i]), i))
    keep = order
    if 0 < top_k < V:
        kth = float(logits[order[top_k - 1]])
        keep = [i for i in order if float(logits[i]) >= kth]
    m = max(float(logits[i]) for i in keep)
    e = {i: math.exp(float(logits[i]) - m) for i in keep}
    z = sum(e.values())
    probs = {i: e[i] / z for i in keep}
    if 0.0 < top_p < 1.0:
        cum = 0.0
        cut = keep[-1]
        for i in keep:
            cum += probs[i]
            if cum >= top_p:
                cut = i
                break
        kept = [i for i in keep if float(logits[i]) >= float(logits[cut])]
        z = sum(probs[i] for i in kept)
        probs = {i: probs[i] / z for i in kept}
    out = torch.zeros(V, dtype=F64)
    for i, p in probs.items():
        out[i] = p
    return out


def inverse_cdf(probs: torch.Tensor, u: float) -> int:
    """First index, in vocabulary order, whose cumulative probability reaches ``u``.

    src/op/kernels/cuda/sampling_kernel.cu:330-398 (prefix scan in vocabulary order, first
    index with ``prev < u <= cum``; falls back to the last candidate).
    """
    cum = 0.0
    last = 0
    for i in range(probs.shape[0]):
        p = float(probs[i])
        if p > 0.0:
            last = i
            cum += p
            if cum >= u:
                return i
    return last
