"""Parts beyond the Llama family's: a block whose sublayers run side by side, mixers with a memory of
fixed size, routed experts, and inputs that reach the stream from outside the layers.

Kinds registered here: embedding ``scaled_table``; pass_input ``vector_rows``; token_input
``gated_side_rows``; mixer ``bias_attention`` and ``channel_delta``; feed_forward ``routed_experts``;
block ``parallel``.  Every size and constant is a parameter of the part's spec.
"""
from __future__ import annotations

import math
from typing import List, Optional

import numpy as np
import torch

from .. import kernels as K
from ..registry import register_part
from .base import Block, CacheNeed, KVNeed, LayerCache, Part, StateNeed, WeightRequest
from .standard import build_part


def _pad16(n: int) -> int:
    return (n + 15) // 16 * 16


def _padded_rows(w: torch.Tensor, rows: int) -> torch.Tensor:
    """``w`` [n, k] with zero rows appended up to ``rows``."""
    if w.shape[0] == rows:
        return w
    out = torch.zeros(rows, w.shape[1], dtype=w.dtype)
    out[: w.shape[0]] = w
    return out


def _padded_cols(w: torch.Tensor, cols: int) -> torch.Tensor:
    if w.shape[1] == cols:
        return w
    out = torch.zeros(w.shape[0], cols, dtype=w.dtype)
    out[:, : w.shape[1]] = w
    return out


# ------------------------------------------------------------------ embedding

@register_part("embedding", "scaled_table")
class ScaledTableEmbedding(Part):
    """``h[t] = E[id[t]] * scale + P[position[t]]``; the position rows are learned and not scaled.  With a ``norm``
    among the weights the row is then divided by its root mean square and multiplied by that weight, in float32.
    params: vocab_size, hidden_size, scale, max_positions, eps (of the norm).  weights: weight [vocab, hidden], positions
    [max_positions, hidden] (absent from the spec's weights: no position rows), norm [hidden] (absent: no norm)."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        out = [WeightRequest(w["weight"], (p["vocab_size"], p["hidden_size"]))]
        if "positions" in w:
            out.append(WeightRequest(w["positions"], (p["max_positions"], p["hidden_size"])))
        if "norm" in w:
            out.append(WeightRequest(w["norm"], (p["hidden_size"],)))
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden_size = int(spec.params["hidden_size"])
        self.scale = float(spec.params.get("scale", 1.0))
        self.weight = rt.matrix(spec.weights["weight"], weights["weight"])
        self.positions = rt.matrix(spec.weights["positions"], weights["positions"]) if "positions" in spec.weights else None
        self.norm = rt.vector32(spec.weights["norm"], weights["norm"]) if "norm" in spec.weights else None
        self.eps = float(spec.params.get("eps", 0.0))

    def forward(self, token_ids: torch.Tensor, ctx=None) -> torch.Tensor:
        out = torch.empty(token_ids.shape[0], self.hidden_size, dtype=torch.float32, device=self.rt.device)
        K.embed_scaled(token_ids, ctx.positions, self.weight, self.positions, self.scale, out)
        return out if self.norm is None else K.post_norm(out, None, 1.0, self.norm, self.eps)


# ------------------------------------------------------------------ what a pass adds on entering

@register_part("pass_input", "vector_rows")
class VectorRows(Part):
    """A table of learned vectors, one of which is added to every row of the stream where an entry of the
    order says so (``LayerRun.enter``).  params: rows, size, again (default False: with it, every pass but the
    first also adds the embedding's output, the stream as it was before the first layer, ahead of the vector).
    weights: table [rows, size]."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        return [WeightRequest(spec.weights["table"], (spec.params["rows"], spec.params["size"]))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        table = weights["table"].to(device=rt.device, dtype=torch.float32).contiguous()
        self.rows = [table[i] for i in range(table.shape[0])]
        # the model keeps a copy of the embedding's output for a pass input that says so, and hands it to forward
        self.wants_embedding = bool(spec.params.get("again", False)) and len(self.rows) > 1

    def settle(self, h: torch.Tensor, pending: Optional[torch.Tensor]) -> torch.Tensor:
        """``h`` with an addend it has not received yet."""
        return h if pending is None else K.stream_add(h, pending.contiguous())

    def forward(self, h: torch.Tensor, row: int, embedded: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self.wants_embedding:
            if embedded is None:
                raise K.KernelError("this pass input adds the embedding's output again and was not given it")
            return K.add_rows_vector(h, embedded if row > 0 else None, self.rows[row])
        return K.add_vector(h, self.rows[row])


# ------------------------------------------------------------------ a token's own input to a layer

@register_part("token_input", "gated_side_rows")
class GatedSideRows(Part):
    """What the token itself adds to the stream at the end of a layer:
    ``y = W_proj (gelu_tanh(W_gate x) * S[id, first : first + size])``, ``x += y / rms(y) * w``.
    params: hidden_size, size, first, table_cols, vocab_size, eps.
    weights: table [vocab, table_cols] (shared by the layers), gate [size, hidden], proj [hidden, size], norm [hidden]."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, n = p["hidden_size"], p["size"]
        return [WeightRequest(w["table"], (p["vocab_size"], p["table_cols"])), WeightRequest(w["gate"], (n, d)),
                WeightRequest(w["proj"], (d, n)), WeightRequest(w["norm"], (d,))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, names = spec.params, spec.weights
        self.size, self.first, self.eps = int(p["size"]), int(p["first"]), float(p["eps"])
        self.width = _pad16(self.size)       # rows of few elements are padded to what the products stream
        self.table = rt.matrix(names["table"], weights["table"])
        self.w_gate = rt.weight(names["gate"] + "|rows16", _padded_rows(weights["gate"], self.width))
        self.w_proj = rt.weight(names["proj"] + "|cols16", _padded_cols(weights["proj"], self.width))
        self.norm = rt.vector32(names["norm"], weights["norm"])

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx) -> torch.Tensor:
        """``h``: the complete float32 stream, ``x``: the same in the compute type."""
        z = K.linear(x, self.w_gate, out_dtype=torch.float32)
        g = torch.empty(z.shape[0], self.width, dtype=self.rt.dtype, device=z.device)
        K.gated_side(z, self.table, ctx.token_ids, self.first, self.size, g)
        y = K.linear(g, self.w_proj, out_dtype=torch.float32)
        return K.add_rmsnormed(h, y, self.norm, self.eps)


# ------------------------------------------------------------------ attention with a bias by distance

def distance_rows(rows: int, far: float, distances: int) -> np.ndarray:
    """Row of a bias table of ``rows`` rows for every distance 0..distances-1: the distance itself below
    ``rows // 2``, then logarithmic steps that reach the last row at distance ``far``:
    ``min(rows - 1, half + floor(ln(n / half) / ln(far / half) * (rows - half)))``."""
    half = rows // 2
    n = np.arange(distances, dtype=np.float64)
    out = np.arange(distances, dtype=np.int64)
    if half < 1:
        return np.zeros(distances, dtype=np.int64)
    beyond = n >= half
    with np.errstate(divide="ignore"):
        steps = np.floor(np.log(np.maximum(n, 1.0) / half) / math.log(far / half) * (rows - half))
    out[beyond] = np.minimum(rows - 1, half + steps[beyond].astype(np.int64))
    return out


class PagedSoftmax:
    """Causal softmax attention of ``H`` query heads on ``G`` key/value heads over pages, as the kernels of
    ``csrc/bias_attention.hip`` compute it: ``score = q . k * scale * temp(i) + bias[i - j, head]``, scores, weights and
    both products in float32.  ``sink`` (float32 [H] on the device, or None): one more term ``exp(sink[head])`` in the
    denominator of every row of that head, with no key and no value.  Holds the sizes, the constants and the kernels' tile
    sizes; a mixer calls it with its queries and the pools it reads (keys and values may be the same pool)."""

    def __init__(self, H: int, G: int, dk: int, dv: int, scale: float, temp_coef: float = 0.0, temp_every: int = 0,
                 bias: Optional[torch.Tensor] = None, one_pool: bool = False, sink: Optional[torch.Tensor] = None):
        if H % G:
            raise ValueError(f"{H} query heads do not divide into {G} kv heads")
        self.H, self.G, self.dk, self.dv = H, G, dk, dv
        self.scale, self.temp_coef, self.temp_every, self.bias = float(scale), float(temp_coef), int(temp_every), bias
        self.sink = sink
        group = H // G
        self.heads_per_chunk = min(group, K.bias_attention_rows())
        self.tile_tokens = max(1, K.bias_attention_rows() // self.heads_per_chunk)
        K.bias_attention_lib()
        # steps with portions of prompts: larger tiles on the matrix cores, where the kernel takes these sizes
        # (``one_pool``: the caller hands the same pool over as keys and as values, which the kernel then stages once)
        wide = K.bias_attention_mfma_rows(dk, dv, one_pool)
        self.wide_heads = min(group, wide) if wide else 0
        self.wide_tokens = max(1, wide // self.wide_heads) if wide else 0

    def __call__(self, qkv, ctx, kpool, vpool, block_table, window: Optional[int] = None, keep_first: int = 0, out_scale: float = 1.0):
        T = qkv.shape[0]
        out = torch.empty(T, self.H * self.dv, dtype=qkv.dtype, device=qkv.device)
        if self.wide_heads and ctx.max_q_len >= K.BIAS_ATTENTION_MFMA_FROM:
            tiles = ctx.q_tiles(self.wide_tokens)
            if tiles is None:
                raise K.KernelError("this step was recorded without the tiles of its tokens")
            return K.bias_attention_mfma(qkv, kpool, vpool, block_table, tiles, ctx.positions, self.bias, out, self.H,
                                         self.scale, self.temp_coef, self.temp_every, self.wide_heads, window, keep_first, out_scale,
                                         sink=self.sink)
        tiles = ctx.q_tiles(self.tile_tokens)
        if tiles is None:
            raise K.KernelError("this step was recorded without the tiles of its tokens")
        chunks = -(-(self.H // self.G) // self.heads_per_chunk)
        # a step of single tokens has tiles of one token: its rows are the heads of a chunk, four a wavefront
        rows = min(self.tile_tokens, ctx.max_q_len) * self.heads_per_chunk
        # all four wavefronts stage the keys and values, also where fewer of them have rows; the keys are cut into
        # runs by the wavefronts that have rows
        waves = 4
        # with a window a tile walks the kept first keys, the window and its own tokens, in whole tiles of 64 keys
        max_keys = ctx.max_context if window is None else min(ctx.max_context, window + keep_first + self.tile_tokens + 128)
        runs = K.bias_attention_runs(tiles.shape[0], self.G, chunks, max_keys, min(4, -(-rows // 4)))
        ws = ctx.workspace(T * self.H * runs * (self.dv + 2)) if runs > 1 else None
        return K.bias_attention(qkv, kpool, vpool, block_table, tiles, ctx.positions, self.bias, out, self.H,
                                self.scale, self.temp_coef, self.temp_every, self.heads_per_chunk, runs, ws, waves, window,
                                keep_first, out_scale, sink=self.sink)


@register_part("mixer", "bias_attention")
class BiasAttention(Part):
    """Causal softmax attention with grouped heads and no rotation: positions enter through a learned bias
    by distance, ``score = q . k * scale * temp(i) + B[row(i - j), head]``, and a temperature of the query
    that grows with its position, ``temp(p) = 1 + coef * ln(floor((p + 1) / every) + 1)``.  Keys and values
    have sizes of their own.

    params: hidden_size, num_heads, num_kv_heads, key_dim, value_dim, scale, bias_far and bias_rows (None:
    no bias), temp_coef and temp_every (None: no temperature), max_positions.
    weights: q [H*dk, d], k [G*dk, d], v [G*dv, d], o [d, H*dv], bias [bias_rows, H]."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, H, G, dk, dv = p["hidden_size"], p["num_heads"], p["num_kv_heads"], p["key_dim"], p["value_dim"]
        out = [WeightRequest(w["q"], (H * dk, d)), WeightRequest(w["k"], (G * dk, d)), WeightRequest(w["v"], (G * dv, d)),
               WeightRequest(w["o"], (d, H * dv))]
        if "bias" in w:
            out.append(WeightRequest(w["bias"], (p["bias_rows"], H)))
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, names = spec.params, spec.weights
        self.H, self.G = int(p["num_heads"]), int(p["num_kv_heads"])
        self.dk, self.dv = int(p["key_dim"]), int(p["value_dim"])
        if self.H % self.G:
            raise ValueError(f"{self.H} query heads do not divide into {self.G} kv heads")
        self.scale = float(p["scale"])
        self.temp_coef = 0.0 if p.get("temp_coef") is None else float(p["temp_coef"])
        self.temp_every = 0 if p.get("temp_coef") is None else int(p["temp_every"])
        self.w_qkv = self._stacked_projection(names, weights, rt)
        self.w_o = rt.weight(names["o"], weights["o"])
        self.bias = self._bias_table(p, names, weights, rt)
        self.core = PagedSoftmax(self.H, self.G, self.dk, self.dv, self.scale, self.temp_coef, self.temp_every, self.bias)

    def _stacked_projection(self, names, weights, rt):
        """The matrix of the part's first product: q | k | v (a subclass may stack others)."""
        return rt.weight("|".join((names["q"], names["k"], names["v"])), torch.cat([weights["q"], weights["k"], weights["v"]], dim=0))

    def _bias_table(self, p, names, weights, rt) -> Optional[torch.Tensor]:
        """float32 [distances, H] on the device: what is added to a score at every distance (None: nothing)."""
        if "bias" not in names:
            return None
        # the learned rows laid out by distance, once: the kernel then looks a score's bias up without a logarithm
        rows = distance_rows(int(p["bias_rows"]), float(p["bias_far"]), int(p["max_positions"]))
        table = weights["bias"].to(torch.float32)[torch.from_numpy(rows)]
        return table.to(rt.device).contiguous()

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv=KVNeed(self.G, self.dk, None, self.dv))

    def forward(self, x, ctx, cache: LayerCache):
        qkv = K.linear(x, self.w_qkv)
        if cache.writes:
            K.kv_store(qkv, self.H * self.dk, (self.H + self.G) * self.dk, cache.slot_mapping, cache.kpool, cache.vpool)
        return K.linear(self.attend(qkv, ctx, cache), self.w_o, out_dtype=torch.float32)

    def attend(self, qkv, ctx, cache: LayerCache, window: Optional[int] = None, keep_first: int = 0, out_scale: float = 1.0):
        """The queries in the first ``H * dk`` columns of ``qkv`` over the keys and values of the cache: [T, H * dv] in
        the compute type.  ``window`` n: a query sees its last n keys and the sequence's first ``keep_first``;
        ``out_scale`` multiplies the result."""
        return self.core(qkv, ctx, cache.kpool, cache.vpool, cache.block_table, window, keep_first, out_scale)


# ------------------------------------------------------------------ gated delta rule, a decay per key channel

@register_part("mixer", "channel_delta")
class ChannelDelta(Part):
    """The gated delta rule with one decay per head and key channel.  Per head, with a memory ``S``
    [key channel, value channel] in float32 that is carried from token to token:

        ``S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q``

    q, k (``num_kv_heads`` heads of ``key_dim``, shared by groups of heads) and v (``num_heads`` of
    ``value_dim``) pass a causal convolution over ``taps`` tokens per channel and silu; q and k become unit
    vectors per head (q also times key_dim^-1/2); ``beta = sigmoid(W_b x)``;
    ``g = exp(-exp(A) softplus(W_a2 W_a1 x + dt))`` per head and key channel; the read-out of a head is divided
    by its root mean square, times a weight shared by the heads, times ``sigmoid(W_g2 W_g1 x)``; then ``W_o``.
    The memory and the last ``taps - 1`` inputs of the convolutions are the per-request state.

    params: hidden_size, num_heads, num_kv_heads, key_dim, value_dim, taps, decay_rank, gate_rank, eps.
    weights: q, k [G*dk, d], v [H*dv, d], q_conv, k_conv [G*dk, taps], v_conv [H*dv, taps], beta [H, d],
    A_log [H], dt_bias [H*dk], decay_in [ra, d], decay_out [H*dk, ra], gate_in [rg, d], gate_out [H*dv, rg],
    norm [dv], o [d, H*dv]."""

    graph_safe = True
    idempotent = False        # a step moves the memory on: running it twice is not running it once

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, H, G, dk, dv = p["hidden_size"], p["num_heads"], p["num_kv_heads"], p["key_dim"], p["value_dim"]
        taps, ra, rg = p["taps"], p["decay_rank"], p["gate_rank"]
        return [WeightRequest(w["q"], (G * dk, d)), WeightRequest(w["q_conv"], (G * dk, taps)),
                WeightRequest(w["k"], (G * dk, d)), WeightRequest(w["k_conv"], (G * dk, taps)),
                WeightRequest(w["v"], (H * dv, d)), WeightRequest(w["v_conv"], (H * dv, taps)),
                WeightRequest(w["beta"], (H, d)), WeightRequest(w["A_log"], (H,)), WeightRequest(w["norm"], (dv,)),
                WeightRequest(w["decay_in"], (ra, d)), WeightRequest(w["decay_out"], (H * dk, ra)),
                WeightRequest(w["dt_bias"], (H * dk,)),
                WeightRequest(w["gate_in"], (rg, d)), WeightRequest(w["gate_out"], (H * dv, rg)),
                WeightRequest(w["o"], (d, H * dv))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, names = spec.params, spec.weights
        self.H, self.G = int(p["num_heads"]), int(p["num_kv_heads"])
        self.dk, self.dv, self.taps = int(p["key_dim"]), int(p["value_dim"]), int(p["taps"])
        self.eps = float(p["eps"])
        if self.H % self.G:
            raise ValueError(f"{self.H} heads do not divide into {self.G} kv heads")
        H, dk, dv = self.H, self.dk, self.dv
        self.channels = 2 * self.G * dk + H * dv
        # one product for q, k, v and beta (float32 out: they enter the recurrence) ...
        stacked = torch.cat([weights["q"], weights["k"], weights["v"], weights["beta"]], dim=0)
        self.w_in = rt.weight("|".join(names[k] for k in ("q", "k", "v", "beta")) + "|rows16",
                              _padded_rows(stacked, _pad16(stacked.shape[0])))
        # ... one for the first steps of the decay's and the gate's projections, padded to whole 16 rows each ...
        ra, rg = _pad16(int(p["decay_rank"])), _pad16(int(p["gate_rank"]))
        self.w_low = rt.weight(names["decay_in"] + "|" + names["gate_in"] + "|rows16",
                               torch.cat([_padded_rows(weights["decay_in"], ra), _padded_rows(weights["gate_in"], rg)], dim=0))
        # ... and one for their second steps: the two matrices on the diagonal of one
        second = torch.zeros(H * dk + H * dv, ra + rg, dtype=weights["decay_out"].dtype)
        second[: H * dk, : weights["decay_out"].shape[1]] = weights["decay_out"]
        second[H * dk:, ra: ra + weights["gate_out"].shape[1]] = weights["gate_out"]
        self.w_second = rt.weight(names["decay_out"] + "|" + names["gate_out"] + "|diagonal", second)
        self.w_o = rt.weight(names["o"], weights["o"])
        key = ("conv", names["q_conv"], names["k_conv"], names["v_conv"])
        if key not in rt.shared:
            rt.shared[key] = torch.cat([weights["q_conv"], weights["k_conv"], weights["v_conv"]], dim=0).to(
                device=rt.device, dtype=torch.float32).contiguous()
        self.conv = rt.shared[key]
        self.a_log = rt.vector32(names["A_log"], weights["A_log"])
        self.dt_bias = rt.vector32(names["dt_bias"], weights["dt_bias"])
        self.norm = rt.vector32(names["norm"], weights["norm"])
        self.state_size = H * dv * dk + (self.taps - 1) * self.channels
        K.delta_rule_lib(dk)

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state=StateNeed((self.state_size,), torch.float32))

    def forward(self, x, ctx, cache: LayerCache):
        if not cache.writes:
            raise K.KernelError("a channel_delta mixer moves its memory on: it cannot read another entry's cache")
        proj = K.linear(x, self.w_in, out_dtype=torch.float32)
        low = K.linear(K.linear(x, self.w_low), self.w_second, out_dtype=torch.float32)
        seq = ctx.per_seq
        y = K.delta_rule(proj, low, self.conv, self.a_log, self.dt_bias, self.norm, cache.state, ctx.seq_of_token,
                         seq.q_start, seq.q_len, seq.state_slot, self.G, self.H, self.dk, self.dv, self.taps, self.eps,
                         self.rt.dtype, max_q_len=ctx.max_q_len)
        return K.linear(y, self.w_o, out_dtype=torch.float32)


# ------------------------------------------------------------------ routed experts

@register_part("feed_forward", "routed_experts")
class RoutedExperts(Part):
    """``experts`` small feed-forwards of which every token uses the ``top`` with the largest router logits
    ``W_r x`` (float32), and optionally one more (``shared``) that every token uses with weight 1.

    params: hidden_size, expert_size, experts, top;
    activation: "relu2" (an expert is ``W_down relu(W_up x)^2``), "swiglu" (``W_down (silu(W_gate x) * (W_up x))``) or
    "capped_glu" (``g = min(W_gate x, limit)``, ``u = clamp(W_up x, -limit, limit)``, ``W_down (g sigmoid(slope g) (u + 1))``,
    with the params ``limit`` and ``slope``);
    mix: "softmax_chosen" (the softmax over the chosen logits alone, the default), "softmax_all" (the softmax over all
    experts, the chosen ones' shares not renormalised) or "sigmoid" (an expert's score is the sigmoid of its logit, and the
    chosen ones' scores are their weights as they are); mix_scale (default 1) multiplies every weight;
    groups, keep (default 1, 1): the experts form ``groups`` equal groups of neighbours, a group counts as much as the
    sum of its ``group_top`` (default 1) best experts, and only the best ``keep`` groups can be chosen from;
    shared: None or the PartSpec of a feed-forward.
    weights: router [experts, d], up<e> [expert_size, d], down<e> [d, expert_size], with a gated activation also gate<e>;
    correction [experts] (absent: none): added to the scores that choose the experts and the groups, never to the weights.

    The experts' matrices are laid side by side, up [E * ff, d] (gated: [E * 2 ff, d], an expert's gate rows and then
    its up rows) and down [d, E * ff].  For a few rows only the chosen experts' rows are read; for many, all experts
    run as two dense products with the mix of an expert that was not chosen at zero, which the matrix cores do
    faster than a gather would here.  With a shared expert the result is two float32 addends [2, T, d], which the
    next norm sums in float32."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, ff = p["hidden_size"], p["expert_size"]
        out = [WeightRequest(w["router"], (p["experts"], d))]
        if "correction" in w:
            out.append(WeightRequest(w["correction"], (p["experts"],)))
        for e in range(p["experts"]):
            if p.get("activation", "relu2") != "relu2":
                out.append(WeightRequest(w[f"gate{e}"], (ff, d)))
            out += [WeightRequest(w[f"up{e}"], (ff, d)), WeightRequest(w[f"down{e}"], (d, ff))]
        if p.get("shared") is not None:
            from .standard import requests_of
            out += requests_of("feed_forward", p["shared"])
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, names = spec.params, spec.weights
        self.E, self.top, self.ff = int(p["experts"]), int(p["top"]), int(p["expert_size"])
        activation = p.get("activation", "relu2")
        if activation not in K.EXPERT_FORMS:
            raise ValueError(f"expert activation {activation!r} is not known (known: {sorted(K.EXPERT_FORMS)})")
        self.activation = activation
        self.gated = activation != "relu2"
        self.limit, self.slope = float(p.get("limit", 0.0)), float(p.get("slope", 1.0))
        if activation == "capped_glu" and not self.limit > 0:
            raise ValueError("capped experts need a positive limit")
        self.mix = p.get("mix", "softmax_chosen")
        if self.mix not in K.ROUTE_SCORINGS:
            raise ValueError(f"expert mix {self.mix!r} is not known (known: {sorted(K.ROUTE_SCORINGS)})")
        self.mix_scale = float(p.get("mix_scale", 1.0))
        self.groups, self.keep, self.group_top = int(p.get("groups", 1)), int(p.get("keep", 1)), int(p.get("group_top", 1))
        self.correction = rt.vector32(names["correction"], weights["correction"]) if "correction" in names else None
        if self.groups < 1 or self.E % self.groups or not 1 <= self.keep <= self.groups or self.top > self.E // self.groups * self.keep:
            raise ValueError(f"{self.top} experts cannot be chosen from {self.keep} of {self.groups} groups of {self.E}")
        self.w_router = rt.weight(names["router"], weights["router"])
        order = [k for e in range(self.E) for k in ((f"gate{e}", f"up{e}") if self.gated else (f"up{e}",))]
        self.w_up = rt.weight("|".join(names[k] for k in order), torch.cat([weights[k] for k in order], dim=0), tiled=False)
        self.w_down = rt.weight("|".join(names[f"down{e}"] for e in range(self.E)),
                                torch.cat([weights[f"down{e}"] for e in range(self.E)], dim=1), tiled=False)
        self.shared = None
        if p.get("shared") is not None:
            self.shared = build_part("feed_forward", p["shared"], getattr(weights, "checkpoint", {}), rt)

    def forward(self, x, ctx):
        T = x.shape[0]
        z = K.linear(x, self.w_router, out_dtype=torch.float32)
        few = T <= K.EXPERTS_FEW_ROWS
        chosen, mix, mix_all = K.route_top(z, self.top, mix_all=not few, groups=self.groups, keep=self.keep, scoring=self.mix,
                                           correction=self.correction, group_top=self.group_top, scale=self.mix_scale)
        out = None
        if self.shared is not None:
            out = torch.empty(2, T, self.w_down.shape[0], dtype=torch.float32, device=x.device)
        if few:
            y = K.experts_few(x, self.w_up.rows, self.w_down.rows, chosen, mix, self.ff, self.activation, None if out is None else out[0],
                              limit=self.limit, slope=self.slope)
        else:
            act = K.experts_act(K.linear(x, self.w_up), mix_all, self.ff, self.activation, self.limit, self.slope)
            y = K.linear(act, self.w_down, out_dtype=torch.float32, out=None if out is None else out[0])
        if out is None:
            return y
        K.linear(self.shared.hidden(x), self.shared.w_down, out_dtype=torch.float32, out=out[1])
        return out


# ------------------------------------------------------------------ block

@register_part("block", "parallel")
class ParallelBlock(Block):
    """``n = norm(h); h += mixer(n) + ffn(n)``: one norm, read by both sublayers, whose outputs are added to
    each other and then to the float32 stream; after that, if the block has one, the token's own input
    (``side``) is added.  ``ffn`` and ``side`` may be absent from the spec."""

    ROLES = {"norm": "norm", "mixer": "mixer", "ffn": "feed_forward", "side": "token_input"}
    OPTIONAL = ("ffn", "side")

    @classmethod
    def _roles(cls, spec):
        missing = [r for r in cls.ROLES if r not in spec.parts and r not in cls.OPTIONAL]
        extra = [r for r in spec.parts if r not in cls.ROLES]
        if missing or extra:
            raise ValueError(f"a block of kind {spec.kind!r} has the parts {sorted(cls.ROLES)}; "
                             f"missing: {missing}, not known: {extra}")
        return [(r, f) for r, f in cls.ROLES.items() if r in spec.parts]

    def forward(self, h, pending, ctx, cache: LayerCache):
        from .base import pending_for
        n = self.norm.forward(h, pending_for(self.norm, pending, self.rt.dtype))
        a = self.mixer.forward(n, ctx, cache)
        f = self.ffn.forward(n, ctx) if "ffn" in self.roles else None
        side = getattr(self, "side", None) if "side" in self.roles else None
        x = None
        if side is not None and self.rt.dtype != torch.float32:
            x = torch.empty(h.shape, dtype=self.rt.dtype, device=h.device)
        K.stream_add(h, a, f, x)
        if side is not None:
            side.forward(h, h if x is None else x, ctx)
        return h, None
