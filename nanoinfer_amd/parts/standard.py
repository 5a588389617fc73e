"""The parts that the Llama family is assembled from.  Each takes its sizes and constants from
``spec.params`` and its tensors by the names in ``spec.weights``; none knows the model it is in.

Kinds registered here: embedding ``table``; norm ``rmsnorm``; position ``rope`` and ``none``;
mixer ``attention``; feed_forward ``swiglu``; block ``prenorm``; head ``linear``.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import numpy as np
import torch

from .. import kernels as K
from ..config.spec import PartSpec
from ..registry import get_part, register_part
from .base import Block, CacheNeed, KVNeed, LayerCache, Part, Runtime, WeightRequest, pending_for


class PartWeights(dict):
    """The tensors a part asked for, by their logical names; ``checkpoint`` is the whole set by
    checkpoint name, which a part hands on to :func:`build_part` for a part it holds inside
    itself (an attention's position encoding)."""

    def __init__(self, own: Dict[str, torch.Tensor], checkpoint: Dict[str, torch.Tensor]):
        super().__init__(own)
        self.checkpoint = checkpoint


def build_part(family: str, spec: PartSpec, tensors: Dict[str, torch.Tensor], rt: Runtime) -> Part:
    """Instantiate the registered class for ``spec.kind`` with the tensors it asked for."""
    cls = get_part(family, spec.kind)
    return cls(spec, PartWeights({logical: tensors[name] for logical, name in spec.weights.items()}, tensors), rt)


def requests_of(family: str, spec: PartSpec) -> List[WeightRequest]:
    return get_part(family, spec.kind).weight_requests(spec)


# ------------------------------------------------------------------ embedding

@register_part("embedding", "table")
class TableEmbedding(Part):
    """``h[t] = E[id[t]]``, no scaling (src/op/embedding.cpp:14-70, kernel embedding_kernel.cu:30-48).
    params: vocab_size, hidden_size.  weights: weight [vocab, hidden]."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        return [WeightRequest(spec.weights["weight"], (spec.params["vocab_size"], spec.params["hidden_size"]))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.vocab_size = int(spec.params["vocab_size"])
        self.hidden_size = int(spec.params["hidden_size"])
        self.weight = rt.matrix(spec.weights["weight"], weights["weight"])

    def forward(self, token_ids: torch.Tensor, ctx=None) -> torch.Tensor:
        out = torch.empty(token_ids.shape[0], self.hidden_size, dtype=torch.float32, device=self.rt.device)
        return K.embedding(token_ids, self.weight, out)


# ------------------------------------------------------------------ norm

@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    """``x * rsqrt(mean(x^2) + eps) * w`` in float32 (src/op/rmsnorm.cpp:14-69, rmsnorm_kernel.cu:50-103).
    params: size, eps.  weights: weight [size]."""

    graph_safe = True
    takes_addends = True      # ``pending`` may be float32 [S, T, size]: S addends, summed in their order

    @classmethod
    def weight_requests(cls, spec):
        return [WeightRequest(spec.weights["weight"], (spec.params["size"],))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.weight = rt.vector32(spec.weights["weight"], weights["weight"])
        self._spec = None

    def forward(self, h: torch.Tensor, pending: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None):
        if isinstance(pending, K.ScaledInput):
            pending = None        # the stream is complete; what came with it was meant for a product, not for this kernel
        n = h.shape[0] if rows is None else rows.shape[0]
        out = torch.empty(n, self.size, dtype=self.rt.dtype, device=self.rt.device)
        return K.add_rmsnorm(h, pending, self.weight, self.eps, out, rows)

    def as_deferred(self) -> "K.NormSpec":
        """Weight and eps of this norm, for a product onto the residual stream that can leave ``h * weight``
        and the rows' sums of squares behind (:class:`nanoinfer_amd.kernels.ScaledInput`): the product that
        stands behind the norm then divides by the root mean squares in its epilogue."""
        if self._spec is None:
            self._spec = K.NormSpec(self.weight, self.eps)
        return self._spec

    def as_prologue(self, h: torch.Tensor, pending: Optional[torch.Tensor] = None):
        """This norm of ``h`` as an input that a product can normalise itself; ``pending`` (float32
        addends [S, T, size] that ``h`` has not received) goes along for a part that ``carries_addends``."""
        return K.NormedInput(h, self.weight, self.eps, self.rt.dtype, pending)


# ------------------------------------------------------------------ position

ROPE_SCALINGS = {}     # kind -> rule(frequencies float32 [pairs], params dict) -> frequencies float32 [pairs]


def register_rope_scaling(kind: str):
    """``@register_rope_scaling("<kind>")`` over a function ``(freqs, params) -> freqs`` (numpy float32):
    another way to stretch the rotation to longer contexts is another entry here, named by the
    ``kind`` of the ``scaling`` parameter of a ``rope`` position part."""
    def deco(fn):
        ROPE_SCALINGS[kind] = fn
        return fn
    return deco


@register_rope_scaling("llama3")
def llama3_scaling(freqs: np.ndarray, params: dict) -> np.ndarray:
    """Long waves divided by ``factor``, short ones kept, a linear blend between, in float32
    arithmetic (src/op/kernels/cuda/rope_kernel.cu:108-127, src/op/kernels/cpu/rope_kernel.cpp:121-139)."""
    f32 = np.float32
    factor, low, high = f32(params["factor"]), f32(params["low_freq_factor"]), f32(params["high_freq_factor"])
    orig = f32(params["original_max_position_embeddings"])
    out = freqs.astype(f32).copy()
    for p in range(out.shape[0]):
        freq = out[p]
        wavelen = f32(f32(2.0) * f32(math.pi) / freq)
        if wavelen >= f32(orig / low):
            freq = f32(freq / factor)
        elif wavelen > f32(orig / high):
            smooth = f32(f32(orig / wavelen - low) / f32(high - low))
            freq = f32(f32(f32(1.0) - smooth) * freq / factor + smooth * freq)
        out[p] = freq
    return out


def rope_inverse_frequencies(rotary_dim: int, theta: float, scaling: Optional[dict]) -> np.ndarray:
    """Frequency of each rotated pair, ``theta^(-2p/rotary_dim)`` in float32 arithmetic
    (src/op/kernels/cuda/rope_kernel.cu:103-106), then the scaling rule that ``scaling["kind"]``
    names, if any, applied with the other entries of ``scaling`` as its parameters."""
    f32 = np.float32
    half = rotary_dim // 2
    out = np.empty(half, dtype=f32)
    for p in range(half):
        out[p] = f32(1.0) / f32(np.power(f32(theta), f32(f32(2 * p) / f32(rotary_dim)), dtype=f32))
    if scaling is not None:
        kind = scaling.get("kind")
        if kind not in ROPE_SCALINGS:
            raise ValueError(f"rotation scaling of kind {kind!r} is not registered; known: {sorted(ROPE_SCALINGS)}")
        out = np.asarray(ROPE_SCALINGS[kind](out, scaling), dtype=f32)
        if out.shape != (half,):
            raise ValueError(f"rotation scaling {kind!r} returned {out.shape} frequencies for {half} pairs")
    return out


@register_part("position", "rope")
class RotaryPosition(Part):
    """Rotation of pairs by ``pos * f_p``.  params: rotary_dim, theta, max_positions, scaling (None,
    or a dict with the ``kind`` of a registered rule and that rule's parameters).  One table per
    distinct set of constants is shared by all layers."""

    graph_safe = True

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.rotary_dim = int(p["rotary_dim"])
        self.max_positions = int(p["max_positions"])
        if self.rotary_dim % 2 or self.rotary_dim <= 0:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be positive and even")
        scaling = p.get("scaling")
        key = ("rope", self.rotary_dim, float(p["theta"]), self.max_positions,
               None if scaling is None else tuple(sorted(scaling.items())))
        if key not in rt.shared:
            inv = torch.from_numpy(rope_inverse_frequencies(self.rotary_dim, float(p["theta"]), scaling)).to(rt.device)
            rt.shared[key] = K.rope_table(inv, self.max_positions)
        self.cos, self.sin = rt.shared[key]

    def tables(self):
        return self.cos, self.sin


@register_part("position", "none")
class NoPosition(Part):
    """No position encoding: keys and queries are used as projected."""

    graph_safe = True

    max_positions = None

    def tables(self):
        return None


# ------------------------------------------------------------------ mixer

@register_part("mixer", "attention")
class Attention(Part):
    """Grouped-query causal attention over the paged cache (src/op/attention.cpp:101-198).

    params: hidden_size, num_heads, num_kv_heads, head_dim, scale (None: 1/sqrt(head_dim)),
    window (None: all keys), position (a PartSpec of family ``position``).
    weights: q [H*hd, d], k [KVH*hd, d], v [KVH*hd, d], o [d, H*hd]; no bias.
    The three input projections are stacked into one matrix at load, so one product feeds the
    rotation-and-cache-write kernel directly.
    """

    graph_safe = True
    MFMA_MIN_PORTION = 8     # a step whose longest portion has this many tokens goes to the matrix-core kernel

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, H, KVH, hd = p["hidden_size"], p["num_heads"], p["num_kv_heads"], p["head_dim"]
        return [WeightRequest(w["q"], (H * hd, d)), WeightRequest(w["k"], (KVH * hd, d)),
                WeightRequest(w["v"], (KVH * hd, d)), WeightRequest(w["o"], (d, H * hd))] + \
            requests_of("position", p["position"])       # a position encoding may have tensors of its own

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.H = int(p["num_heads"])
        self.KVH = int(p["num_kv_heads"])
        self.hd = int(p["head_dim"])
        if self.H % self.KVH:
            raise ValueError(f"{self.H} query heads do not divide into {self.KVH} kv heads")
        self.scale = float(p["scale"]) if p.get("scale") is not None else 1.0 / math.sqrt(self.hd)
        self.window = None if p.get("window") is None else int(p["window"])
        K.attention_lib(self.hd)  # refuses an unsupported head size now, not at the first step
        pos_spec: PartSpec = p["position"]
        self.position = build_part("position", pos_spec, getattr(weights, "checkpoint", {}), rt)
        names = spec.weights
        self.w_qkv = rt.weight("|".join((names["q"], names["k"], names["v"])),
                               torch.cat([weights["q"], weights["k"], weights["v"]], dim=0))
        self.w_o = rt.weight(names["o"], weights["o"])

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv=KVNeed(self.KVH, self.hd, self.window))

    # The pass is four stages, each a method of its own, so that a variant of attention replaces the stage
    # it changes and keeps the others: project (x -> stacked q, k, v), rotate_and_write (position encoding,
    # keys and values into the cache pages), attend (queries over the cache), output (the o product, onto the
    # residual stream where it can).  The first two also exist fused in one kernel for steps of few rows; the
    # fused kernel stands in only for a class that has left both stages as they are here.

    def _fused_projection(self, T: int, d: int, dtype) -> bool:
        """Whether the product with the stacked matrix rotates and stores in its own epilogue for T rows."""
        cls = type(self)
        if cls.project is not Attention.project or cls.rotate_and_write is not Attention.rotate_and_write:
            return False
        tables = self.position.tables()
        return (tables is not None and K.qkv_rope_ok(T, d, self.hd, 2 * tables[0].shape[1], dtype)
                and K.qkv_rope_wins(T, d, dtype))

    def takes_normed(self, T: int) -> bool:
        """Whether ``forward`` takes the norm before it as a prologue of its first product for T tokens."""
        d = self.w_qkv.shape[1]
        return (K.FUSE_NORMS and self._fused_projection(T, d, self.rt.dtype)
                and K.norm_prologue_ok(T, d, self.rt.dtype, self.w_qkv))

    def adds_residual(self, T: int) -> bool:
        """Whether ``forward`` can take ``residual=h`` for T tokens: its output then goes into the residual
        stream without a kernel for the sum (added by the product itself, or left as float32 addends)."""
        return K.FUSE_NORMS and K.residual_epilogue_ok(T, self.H * self.hd, self.rt.dtype, self.w_o)

    def carries_addends(self, T: int, addends: int) -> bool:
        """Whether ``forward`` can be given, for T tokens, a normed input that holds ``addends`` pending
        addends of ``h``, together with ``residual=h``: its first product normalises ``h`` plus the addends,
        its last one adds them into ``h`` with its own output."""
        d = self.w_qkv.shape[1]
        return (self.takes_normed(T) and self.adds_residual(T)
                and K.norm_prologue_ok(T, d, self.rt.dtype, self.w_qkv, addends)
                and K.residual_takes_addends(T, self.H * self.hd, self.rt.dtype, self.w_o))

    def takes_scaled(self, T: int) -> bool:
        """Whether ``forward`` takes, for T tokens, the input that the product before the norm left half done
        (a :class:`nanoinfer_amd.kernels.ScaledInput`): its first product divides by the rows' root mean squares."""
        d = self.w_qkv.shape[1]
        return (type(self).project is Attention.project and K.takes_scaled_ok(T, d, self.rt.dtype, self.w_qkv)
                and (self._fused_projection(T, d, self.rt.dtype) or type(self).rotate_and_write is Attention.rotate_and_write))

    def leaves_scaled(self, T: int) -> bool:
        """Whether ``forward``, given ``residual=h`` and ``leave`` (the next norm's weight and eps), returns
        that norm's input half done for T tokens."""
        return (type(self).output is Attention.output and self.adds_residual(T)
                and K.leaves_scaled_ok(T, self.H * self.hd, self.rt.dtype, self.w_o))

    def project(self, x, ctx) -> torch.Tensor:
        """Stage 1: ``x`` [T, d] -> [T, (H + 2 KVH) * hd], the query heads, then the key heads, then the
        value heads, as projected."""
        return K.linear(x, self.w_qkv)

    def rotate_and_write(self, qkv: torch.Tensor, ctx, cache: LayerCache) -> torch.Tensor:
        """Stage 2: the position encoding on the query and key heads of ``qkv`` (in place), and the keys and
        values of the step's tokens into their places in the cache pages (where this entry of the order writes)."""
        tables = self.position.tables()
        cos, sin = tables if tables is not None else (None, None)
        slots = cache.slot_mapping if cache.writes else None
        K.rope_kv_write(qkv, ctx.positions, cos, sin, slots, cache.kpool, cache.vpool, self.H, self.KVH, self.hd)
        return qkv

    def project_rotate_write(self, x, ctx, cache: LayerCache) -> torch.Tensor:
        """Stages 1 and 2: by one kernel where few rows allow it and neither stage has been replaced."""
        T = x.shape[0]
        if self._fused_projection(T, x.shape[1], x.dtype):
            cos, sin = self.position.tables()
            return K.skinny_qkv_rope(x, self.w_qkv, ctx.positions, cos, sin, cache.slot_mapping if cache.writes else None,
                                     cache.kpool, cache.vpool, self.H, self.KVH, self.hd)
        return self.rotate_and_write(self.project(x, ctx), ctx, cache)

    def attend(self, qkv: torch.Tensor, ctx, cache: LayerCache, leave_runs: bool = False):
        """Stage 3: every query of ``qkv`` over the keys and values of its sequence in the cache, up to its own
        position (inside the window, if there is one).  Returns ``out`` [T, H * hd]; or, with ``leave_runs``
        where the key ranges were cut into runs that the output product can merge itself, ``(workspace, runs)``."""
        T = qkv.shape[0]
        dtype = qkv.dtype
        out = torch.empty(T, self.H * self.hd, dtype=dtype, device=qkv.device)
        tiles = None
        if ctx.max_q_len >= self.MFMA_MIN_PORTION and K.mfma_attention_ok(dtype, self.hd):
            # prompt portions: tiles of tokens on the matrix cores (a recorded step has them only if
            # it was recorded with them)
            max_keys = ctx.max_context if self.window is None else min(ctx.max_context, self.window + ctx.max_q_len)
            tile_tokens, nsplit = K.mfma_plan(self.hd, self.H // self.KVH, self.KVH, T, ctx.max_q_len, max_keys, dtype)
            tiles = ctx.q_tiles(tile_tokens)
        if tiles is not None:
            if nsplit is None:
                nsplit = K.mfma_splits(tiles.shape[0], self.KVH, self.H // self.KVH, max_keys)
            ws = ctx.workspace(T * self.H * nsplit * (self.hd + 2)) if nsplit > 1 else None
            K.mfma_attention(qkv, cache.kpool, cache.vpool, cache.block_table, tiles, out, self.H, self.KVH, self.hd,
                             self.scale, self.window, nsplit, ws, tile_tokens)
            return out
        # single tokens and short portions, token by token
        max_keys = ctx.max_context if self.window is None else min(ctx.max_context, self.window)
        on_matrix_cores = K.mfma_token_ok(dtype, self.hd)
        choose = K.mfma_token_splits if on_matrix_cores else K.choose_splits
        nsplit = choose(T, self.KVH, self.H // self.KVH, max_keys)
        ws = ctx.workspace(T * self.H * nsplit * (self.hd + 2)) if nsplit > 1 else None
        if (leave_runs and on_matrix_cores and nsplit > 1 and K.MERGE_IN_PRODUCT
                and K.skinny_merge_wins(T, self.H, self.hd, nsplit, dtype, self.w_o)):
            # one or two rows: the output product merges the key runs in its prologue, no kernel of its own does
            K.mfma_token_attention(qkv, cache.kpool, cache.vpool, cache.block_table, ctx.seq_of_token, ctx.positions,
                                   out, self.H, self.KVH, self.hd, self.scale, self.window, nsplit, ws, merge=False)
            return ws, nsplit
        attend = K.mfma_token_attention if on_matrix_cores else K.token_attention
        attend(qkv, cache.kpool, cache.vpool, cache.block_table, ctx.seq_of_token, ctx.positions, out,
               self.H, self.KVH, self.hd, self.scale, self.window, nsplit, ws)
        return out

    def output(self, attended, T: int, residual: Optional[torch.Tensor] = None, carried: Optional[torch.Tensor] = None,
               leave=None):
        """Stage 4: the o product of what :meth:`attend` returned.  With ``residual`` (the float32 stream) the
        product goes into it (None is returned) or comes back as float32 addends for the next norm; ``carried``
        are addends that the stream has not received and that go in with it; with ``leave`` (the next norm's
        weight and eps, where :meth:`leaves_scaled` holds) that norm's input comes back half done."""
        if isinstance(attended, tuple):
            ws, nsplit = attended
            if residual is not None:
                if leave is not None and not K.leaves_scaled_ok(T, self.H * self.hd, self.rt.dtype, self.w_o):
                    leave = None
                left = K.skinny_gemm_merged(ws, nsplit, T, self.H, self.hd, self.w_o, residual, residual=True,
                                            pending=carried, leave=leave)
                return left if isinstance(left, K.ScaledInput) else None
            y = torch.empty(T, self.w_o.rows.shape[0], dtype=self.rt.dtype, device=ws.device)
            return K.skinny_gemm_merged(ws, nsplit, T, self.H, self.hd, self.w_o, y)
        return K.linear(attended, self.w_o, residual=residual, pending=carried, leave=leave)

    def forward(self, x, ctx, cache: LayerCache, residual: Optional[torch.Tensor] = None, leave=None):
        T = x.shape[0]
        carried = getattr(x, "pending", None)       # addends of the residual stream that came with a normed input
        if carried is not None and residual is None:
            raise K.KernelError("pending addends of the residual stream need residual=h to go into")
        qkv = self.project_rotate_write(x, ctx, cache)
        leave_runs = type(self).output is Attention.output      # a replaced output stage gets the merged rows
        attended = self.attend(qkv, ctx, cache, leave_runs=leave_runs)
        if leave is not None:
            return self.output(attended, T, residual, carried, leave)
        return self.output(attended, T, residual, carried)


# ------------------------------------------------------------------ feed-forward

@register_part("feed_forward", "swiglu")
class SwiGLU(Part):
    """``down(silu(gate(x)) * up(x))`` (src/model/llama.cpp:364-379, swiglu_kernel.cu:31-39).
    params: hidden_size, intermediate_size.  weights: gate [I, d], up [I, d], down [d, I].
    gate and up are stacked so one product yields both halves."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, i = p["hidden_size"], p["intermediate_size"]
        return [WeightRequest(w["gate"], (i, d)), WeightRequest(w["up"], (i, d)), WeightRequest(w["down"], (d, i))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.intermediate_size = int(spec.params["intermediate_size"])
        names = spec.weights
        self.w_gate_up = rt.weight(names["gate"] + "|" + names["up"], torch.cat([weights["gate"], weights["up"]], dim=0))
        self.w_down = rt.weight(names["down"], weights["down"])

    def takes_normed(self, T: int) -> bool:
        d = self.w_gate_up.shape[1]
        return (K.FUSE_NORMS and self.intermediate_size % 16 == 0
                and K.norm_prologue_ok(T, d, self.rt.dtype, self.w_gate_up))

    def adds_residual(self, T: int) -> bool:
        return K.FUSE_NORMS and K.residual_epilogue_ok(T, self.intermediate_size, self.rt.dtype, self.w_down)

    def carries_addends(self, T: int, addends: int) -> bool:
        d = self.w_gate_up.shape[1]
        return (self.takes_normed(T) and self.adds_residual(T)
                and K.norm_prologue_ok(T, d, self.rt.dtype, self.w_gate_up, addends, swiglu=True)
                and K.residual_takes_addends(T, self.intermediate_size, self.rt.dtype, self.w_down))

    def takes_scaled(self, T: int) -> bool:
        return K.swiglu_takes_scaled(T, self.w_gate_up.shape[1], self.rt.dtype, self.w_gate_up)

    def leaves_scaled(self, T: int) -> bool:
        return self.adds_residual(T) and K.leaves_scaled_ok(T, self.intermediate_size, self.rt.dtype, self.w_down)

    def forward(self, x, ctx, residual: Optional[torch.Tensor] = None, leave=None):
        carried = getattr(x, "pending", None)       # addends of the residual stream that came with a normed input
        if carried is not None and residual is None:
            raise K.KernelError("pending addends of the residual stream need residual=h to go into")
        return K.linear(K.linear_swiglu(x, self.w_gate_up), self.w_down, residual=residual, pending=carried, leave=leave)


# ------------------------------------------------------------------ block

@register_part("block", "prenorm")
class PreNormBlock(Block):
    """``h += mixer(norm1(h)); h += ffn(norm2(h))`` (src/model/llama.cpp:324-379).

    The residual stream ``h`` is float32.  The last addend is handed on as ``pending`` and is
    summed into ``h`` by the next norm, in float32, in the same pass that normalises.  Two optional
    abilities of a mixer or feed-forward shorten this for steps of few tokens: ``adds_residual(T)``
    (given ``residual=h`` its last product adds into ``h`` itself and nothing is pending, or it
    returns float32 addends [S, T, d] for the next norm to sum) and ``takes_normed(T)`` (its first
    product normalises ``h`` itself, given the norm's ``as_prologue(h)``).  A part that has both may
    also say ``carries_addends(T, S)``: given ``as_prologue(h, pending)`` with S float32 addends that
    ``h`` has not received, and ``residual=h``, its first product normalises ``h`` plus the addends and
    its last one brings them into ``h`` with its own output, so the shares of a cut product need no
    kernel that sums them.  A part without these is run the plain way.
    """

    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "feed_forward"}

    def _normed_input(self, norm, part, h, pending):
        """What ``part`` is given for ``norm(h + pending)``: the norm as a prologue where both sides can, else its
        output.  Float32 addends go along with the prologue where the part ``carries_addends``: its first product
        normalises ``h`` plus the addends, its last one adds them into ``h`` (it is then run with ``residual=h``)."""
        T = h.shape[0]
        if isinstance(pending, K.ScaledInput):
            # the stream is complete, and the product before left this norm's input half done
            takes = getattr(part, "takes_scaled", None)
            if takes is not None and takes(T) and pending.made_for(getattr(norm, "weight", None), getattr(norm, "eps", 0.0)):
                return pending
            pending = None
        takes = getattr(part, "takes_normed", None)
        prologue = getattr(norm, "as_prologue", None)
        if takes is not None and prologue is not None and takes(T):
            if pending is None:
                return prologue(h)
            carries = getattr(part, "carries_addends", None)
            if (carries is not None and getattr(norm, "takes_addends", False) and pending.dim() == 3
                    and pending.dtype == torch.float32 and carries(T, pending.shape[0])):
                return prologue(h, pending)
        return norm.forward(h, pending_for(norm, pending, self.rt.dtype))

    @staticmethod
    def _deferred(norm, producer, consumer, T: int):
        """``norm``'s weight and eps if, for T tokens, ``producer`` (which adds into the stream) can leave the
        norm's input half done and ``consumer`` can take it so; else None."""
        spec = getattr(norm, "as_deferred", None)
        leaves = getattr(producer, "leaves_scaled", None)
        takes = getattr(consumer, "takes_scaled", None)
        if spec is None or leaves is None or takes is None or not (leaves(T) and takes(T)):
            return None
        return spec()

    leaves_for_next = True      # ``forward`` takes ``leave=``: what ``wants_scaled`` of the block behind this one returned

    def wants_scaled(self, T: int):
        """For the block that runs before this one: weight and eps of this block's first norm if its mixer can
        take that norm's input half done for T tokens (see :meth:`_deferred`), else None."""
        spec = getattr(self.mixer_norm, "as_deferred", None)
        takes = getattr(self.mixer, "takes_scaled", None)
        return spec() if spec is not None and takes is not None and takes(T) else None

    def forward(self, h, pending, ctx, cache: LayerCache, leave=None):
        T = h.shape[0]
        x = self._normed_input(self.mixer_norm, self.mixer, h, pending)
        adds = getattr(self.mixer, "adds_residual", None)
        if adds is not None and adds(T):
            spec = self._deferred(self.ffn_norm, self.mixer, self.ffn, T)
            a = self.mixer.forward(x, ctx, cache, residual=h, **({} if spec is None else {"leave": spec}))
        else:
            a = self.mixer.forward(x, ctx, cache)
        x = self._normed_input(self.ffn_norm, self.ffn, h, a)
        adds = getattr(self.ffn, "adds_residual", None)
        if adds is not None and adds(T):
            leaves = getattr(self.ffn, "leaves_scaled", None)
            spec = leave if (leave is not None and leaves is not None and leaves(T)) else None
            f = self.ffn.forward(x, ctx, residual=h, **({} if spec is None else {"leave": spec}))
        else:
            f = self.ffn.forward(x, ctx)
        return h, f


# ------------------------------------------------------------------ head

@register_part("head", "linear")
class LinearHead(Part):
    """``logits = x . W^T`` in float32 output (src/model/llama.cpp:383-386).  params: vocab_size,
    hidden_size.  weights: weight [vocab, hidden]; a tied head names the embedding's tensor and
    shares its device buffer."""

    graph_safe = True
    writes_into = True       # ``forward`` takes ``out=``: float32 [R, vocab] to write the logits into

    @classmethod
    def weight_requests(cls, spec):
        return [WeightRequest(spec.weights["weight"], (spec.params["vocab_size"], spec.params["hidden_size"]))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.vocab_size = int(spec.params["vocab_size"])
        # the large matrix is streamed as stored: re-tiling gains nothing at its size and would double it
        self.weight = rt.matrix(spec.weights["weight"], weights["weight"])

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        return K.linear(x, self.weight, out_dtype=torch.float32, out=out)
