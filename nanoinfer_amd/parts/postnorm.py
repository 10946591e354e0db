"""Parts around a stream that is normed *behind* every sum: the block ``h <- norm(alpha h + sublayer(h))``, attention in
a window with a norm a head, a sink in the softmax and a gate a head, whose keys and values another layer may read
again, and the dense feed-forward with capped hidden units that routed experts use as the expert every token shares.

Kinds registered here: block ``postnorm``; mixer ``sink_attention``; feed_forward ``capped_glu``.  Every size and
constant is a parameter of the part's spec.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .. import kernels as K
from ..registry import register_part
from .base import Block, CacheNeed, KVNeed, LayerCache, Part, WeightRequest
from .standard import requests_of
from .stateful import WindowAttention


@dataclass
class StreamCopy:
    """What a ``postnorm`` block hands on as ``pending``: nothing is pending, the stream is complete, and ``x`` is the
    same stream in the compute type, which the norm that made the stream wrote in the same pass.  The block behind
    reads it instead of rounding the stream again; whoever does not know it takes the stream itself."""

    x: torch.Tensor


# ------------------------------------------------------------------ softmax attention in a window, with a sink

@register_part("mixer", "sink_attention")
class SinkAttention(WindowAttention):
    """Causal softmax attention with grouped heads in which query i sees key j if ``0 <= i - j < window`` (None: every
    earlier key).  In float32: an RMS norm of every query head and of every key head on its own, each with one weight
    shared by the heads; then the rotation of the first channels of every head (``position``; ``adjacent_pairs``: channel
    2i turns with channel 2i + 1); ``score = q . k * scale``; the softmax's denominator holds one more term
    ``exp(sink[h])`` that has no key and no value; head h's output is multiplied by ``sigmoid(W_g x)[h]``; then ``W_o``.

    A part with ``shares_kv`` has no key and value projections: it reads the keys (normed and rotated) and values that
    another entry of the order wrote (``LayerRun.writes_cache`` False) with its own queries, window, sink and gate.
    ``cache_window`` is what the pages have to keep for every part that reads them: the largest of their windows (None:
    every key).

    params: hidden_size, num_heads, num_kv_heads, key_dim, value_dim, scale, window, cache_window, eps, position,
    adjacent_pairs, shares_kv.
    weights: q [H*dk, d], q_norm [dk], sink [H], g [H, d], o [d, H*dv]; without ``shares_kv`` also k [G*dk, d],
    v [G*dv, d], k_norm [dk]."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, H, G, dk, dv = p["hidden_size"], p["num_heads"], p["num_kv_heads"], p["key_dim"], p["value_dim"]
        out = [WeightRequest(w["q"], (H * dk, d)), WeightRequest(w["q_norm"], (dk,)), WeightRequest(w["sink"], (H,)),
               WeightRequest(w["g"], (H, d)), WeightRequest(w["o"], (d, H * dv))]
        if not p.get("shares_kv"):
            out += [WeightRequest(w["k"], (G * dk, d)), WeightRequest(w["v"], (G * dv, d)), WeightRequest(w["k_norm"], (dk,))]
        if p.get("position") is not None:
            out += requests_of("position", p["position"])
        return out

    def __init__(self, spec, weights, rt):
        p = dict(spec.params)
        self.shares_kv = bool(p.get("shares_kv", False))
        p.update(qk_norm=False, keep_first=0, out_scale=1.0)      # the norms here are a head's own, set up below
        super().__init__(type(spec)(spec.kind, p, spec.weights), weights, rt)
        names = spec.weights
        self.adjacent = bool(p.get("adjacent_pairs", False))
        kept = p["cache_window"] if "cache_window" in p else p.get("window")      # what the pages keep; absent: this part's own window
        self.cache_window = None if kept is None else int(kept)
        if self.cache_window is not None and (self.window is None or self.window > self.cache_window):
            raise ValueError(f"a window of {self.window} keys reads pages that keep {self.cache_window}")
        self.head_q_norm = rt.vector32(names["q_norm"], weights["q_norm"])
        self.head_k_norm = None if self.shares_kv else rt.vector32(names["k_norm"], weights["k_norm"])
        self.core.sink = rt.vector32(names["sink"], weights["sink"])
        self.gate_col = self.H * self.dk + (0 if self.shares_kv else self.G * (self.dk + self.dv))

    def _stacked_projection(self, names, weights, rt):
        """q | k | v | g, or q | g for a part that reads another's keys and values."""
        order = ("q", "g") if self.shares_kv else ("q", "k", "v", "g")
        return rt.weight("|".join(names[k] for k in order), torch.cat([weights[k] for k in order], dim=0))

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv=KVNeed(self.G, self.dk, self.cache_window, self.dv))

    def forward(self, x, ctx, cache: LayerCache, out: Optional[torch.Tensor] = None):
        if cache.writes == self.shares_kv:
            raise K.KernelError("a sink_attention part writes the keys and values it makes, and only those")
        proj = K.linear(x, self.w_qkv, out_dtype=torch.float32)
        q = torch.empty(x.shape[0], self.H * self.dk, dtype=self.rt.dtype, device=proj.device)
        if self.shares_kv:
            K.qk_norm_rope_store(proj, ctx.positions, None, self.head_q_norm, None, self.eps, self.freq, self.amplitude, q, None, None,
                                 self.H, per_head=True, adjacent=self.adjacent, q_dim=self.dk, queries_only=True)
        else:
            K.qk_norm_rope_store(proj, ctx.positions, cache.slot_mapping, self.head_q_norm, self.head_k_norm, self.eps, self.freq,
                                 self.amplitude, q, cache.kpool, cache.vpool, self.H, per_head=True, adjacent=self.adjacent)
        attended = self.attend(q, ctx, cache, self.window, 0, 1.0)
        gated = K.gate_rows(attended, proj, self.gate_col, out=attended, every=self.dv)
        return K.linear(gated, self.w_o, out_dtype=torch.float32, out=out)


# ------------------------------------------------------------------ feed-forward with capped hidden units

@register_part("feed_forward", "capped_glu")
class CappedGLU(Part):
    """``W_down (g * sigmoid(slope * g) * (u + 1))`` with ``g = min(W_gate x, limit)`` and ``u = clamp(W_up x, -limit,
    limit)``.  params: hidden_size, intermediate_size, limit, slope.  weights: gate [I, d], up [I, d], down [d, I].
    gate and up are stacked so one product yields both halves."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, i = p["hidden_size"], p["intermediate_size"]
        return [WeightRequest(w["gate"], (i, d)), WeightRequest(w["up"], (i, d)), WeightRequest(w["down"], (d, i))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, names = spec.params, spec.weights
        self.intermediate_size = int(p["intermediate_size"])
        self.limit, self.slope = float(p["limit"]), float(p.get("slope", 1.0))
        if not self.limit > 0:
            raise ValueError("capped hidden units need a positive limit")
        self.w_gate_up = rt.weight(names["gate"] + "|" + names["up"], torch.cat([weights["gate"], weights["up"]], dim=0))
        self.w_down = rt.weight(names["down"], weights["down"])

    def hidden(self, x) -> torch.Tensor:
        """What the down product takes (for a part that places that product's result itself)."""
        return K.experts_act(K.linear(x, self.w_gate_up), None, self.intermediate_size, "capped_glu", self.limit, self.slope)

    def forward(self, x, ctx):
        return K.linear(self.hidden(x), self.w_down, out_dtype=torch.float32)


# ------------------------------------------------------------------ block

@register_part("block", "postnorm")
class PostNormBlock(Block):
    """``h <- norm1(alpha h + mixer(h)); h <- norm2(alpha h + ffn(h))``: the sublayers read the stream itself, and the
    norm stands behind the sum, so the float32 stream is a normed vector at every point.  Sum, norm and stream are
    float32; the norm's kernel also writes the stream in the compute type for the products that read it next.
    ``ffn_norm`` and ``ffn`` may be absent together: the block is its first half alone.  params: alpha."""

    ROLES = {"mixer": "mixer", "mixer_norm": "norm", "ffn": "feed_forward", "ffn_norm": "norm"}
    OPTIONAL = ("ffn", "ffn_norm")

    @classmethod
    def _roles(cls, spec):
        missing = [r for r in cls.ROLES if r not in spec.parts and r not in cls.OPTIONAL]
        extra = [r for r in spec.parts if r not in cls.ROLES]
        if ("ffn" in spec.parts) != ("ffn_norm" in spec.parts):
            missing.append("ffn_norm" if "ffn" in spec.parts else "ffn")
        if missing or extra:
            raise ValueError(f"a block of kind {spec.kind!r} has the parts {sorted(cls.ROLES)}; "
                             f"missing: {missing}, not known: {extra}")
        return [(r, f) for r, f in cls.ROLES.items() if r in spec.parts]

    def __init__(self, spec, tensors, rt):
        super().__init__(spec, tensors, rt)
        self.alpha = float(spec.params.get("alpha", 1.0))
        for norm in (self.mixer_norm,) + ((self.ffn_norm,) if "ffn" in self.roles else ()):
            if not hasattr(norm, "weight") or not hasattr(norm, "eps"):
                raise ValueError("a postnorm block's norms are RMS norms with a weight and an eps")
        K.stream_lib()

    def _behind(self, h, y, norm):
        """The stream after ``norm(alpha h + y)``, and the same in the compute type (the stream itself where that is float32)."""
        if self.rt.dtype == torch.float32:
            return K.post_norm(h, y, self.alpha, norm.weight, norm.eps)
        x = torch.empty(h.shape, dtype=self.rt.dtype, device=h.device)
        K.post_norm(h, y, self.alpha, norm.weight, norm.eps, x=x)
        return x

    def forward(self, h, pending, ctx, cache: LayerCache):
        if isinstance(pending, StreamCopy):
            x = pending.x
        else:
            if pending is not None:
                raise K.KernelError("a postnorm block reads a complete stream: nothing may be pending")
            x = h if self.rt.dtype == torch.float32 else h.to(self.rt.dtype)
        y = self.mixer.forward(x, ctx, cache)
        x = self._behind(h, y if y.dtype == torch.float32 else y.to(torch.float32), self.mixer_norm)
        if "ffn" in self.roles:
            y = self.ffn.forward(x, ctx)
            x = self._behind(h, y if y.dtype == torch.float32 else y.to(torch.float32), self.ffn_norm)
        return h, (None if self.rt.dtype == torch.float32 else StreamCopy(x))
