"""Parts that keep something of fixed size per request beside (or instead of) keys and values in pages, and an
attention whose window keeps the first tokens of a sequence in sight.

Kinds registered here: embedding ``pair_hash_table``; mixer ``window_attention``, ``decay_attention``,
``selective_scan`` and ``side_by_side`` (two mixers that read the same input, their outputs summed).  Every size
and constant is a parameter of the part's spec.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import kernels as K
from ..registry import get_part, register_part
from .base import CacheNeed, KVNeed, LayerCache, Part, StateNeed, WeightRequest
from .hybrid import BiasAttention
from .standard import build_part, requests_of


def _up4(n: int) -> int:
    return (n + 3) // 4 * 4


# ------------------------------------------------------------------ embedding

@register_part("embedding", "pair_hash_table")
class PairHashEmbedding(Part):
    """``h[t] = E[id[t]] * scale + P[(prev * mul_prev + id[t] * mul_cur) mod buckets]``: a second table is read by a
    hash of the pair (token before, token); a sequence's first token takes the row behind the buckets.  The token
    before a portion's first is the last token of the sequence so far, kept per request in a state slot.  With
    ``sinusoid_base`` b a vector of the position p is added as well: column 2i ``sin(p * b^(-2i / hidden))``, column
    2i + 1 the cosine of the same angle (frequencies worked out in float64 and rounded once, the angle a float32 product).
    params: vocab_size, hidden_size, scale, buckets, mul_prev, mul_cur (``buckets`` None and no ``pairs``: no second
    table), sinusoid_base (None: none).
    weights: weight [vocab, hidden], pairs [buckets + 1, hidden]."""

    graph_safe = True
    idempotent = False        # a step leaves its last token behind: run twice, its first row would see that one

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        out = [WeightRequest(w["weight"], (p["vocab_size"], p["hidden_size"]))]
        if "pairs" in w:
            out.append(WeightRequest(w["pairs"], (p["buckets"] + 1, p["hidden_size"])))
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.scale = float(p.get("scale", 1.0))
        self.weight = rt.matrix(spec.weights["weight"], weights["weight"])
        self.pairs, self.buckets, self.mul_prev, self.mul_cur = None, 0, 0, 0
        if "pairs" in spec.weights:
            self.buckets, self.mul_prev, self.mul_cur = int(p["buckets"]), int(p["mul_prev"]), int(p["mul_cur"])
            self.pairs = rt.matrix(spec.weights["pairs"], weights["pairs"])
        self.freq = None
        if p.get("sinusoid_base") is not None:
            d, base = self.hidden_size, float(p["sinusoid_base"])
            freq = torch.tensor([base ** (-2.0 * i / d) for i in range((d + 1) // 2)], dtype=torch.float64)
            self.freq = freq.to(torch.float32).to(rt.device)

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state=StateNeed((1,), torch.int32))

    def forward(self, token_ids: torch.Tensor, ctx, cache: LayerCache = None) -> torch.Tensor:
        if cache is None or cache.state is None:
            raise K.KernelError("a pair_hash_table embedding needs its state slots")
        out = torch.empty(token_ids.shape[0], self.hidden_size, dtype=torch.float32, device=self.rt.device)
        seq = ctx.per_seq
        return K.embed_pair_hash(token_ids, ctx.positions, ctx.seq_of_token, seq.q_start, seq.q_len, seq.state_slot, cache.state,
                                 self.weight, self.pairs, self.buckets, self.mul_prev, self.mul_cur, self.scale, out, freq=self.freq)


# ------------------------------------------------------------------ softmax attention in a window that keeps the first tokens

@register_part("mixer", "window_attention")
class WindowAttention(BiasAttention):
    """Causal softmax attention with grouped heads in which query i sees key j if ``i - j < window`` or
    ``j < keep_first`` (``window`` None: every earlier key).  Before the scores, in float32: an RMS norm over a
    token's whole query projection and one over its whole key projection (all heads at once; ``qk_norm``), then a
    rotation of the first channels of every head (``position``: a PartSpec of family ``position`` whose part
    answers ``frequencies()``, or None).  ``score = q . k * scale``; keys and values have sizes of their own; the
    output is multiplied by ``out_scale`` before its projection.  Kept keys keep their true positions, so every
    page of a request stays in the pool.

    params: hidden_size, num_heads, num_kv_heads, key_dim, value_dim, scale, window, keep_first, qk_norm, eps, position,
    out_scale.  weights: q [H*dk, d], k [G*dk, d], v [G*dv, d], o [d, H*dv], q_norm [H*dk], k_norm [G*dk]."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, H, G, dk, dv = p["hidden_size"], p["num_heads"], p["num_kv_heads"], p["key_dim"], p["value_dim"]
        out = [WeightRequest(w["q"], (H * dk, d)), WeightRequest(w["k"], (G * dk, d)), WeightRequest(w["v"], (G * dv, d)),
               WeightRequest(w["o"], (d, H * dv))]
        if p.get("qk_norm"):
            out += [WeightRequest(w["q_norm"], (H * dk,)), WeightRequest(w["k_norm"], (G * dk,))]
        if p.get("position") is not None:
            out += requests_of("position", p["position"])
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)       # the stacked q | k | v matrix, the o matrix, the kernels' tile sizes
        p, names = spec.params, spec.weights
        self.window = None if p.get("window") is None else int(p["window"])
        self.keep_first = int(p.get("keep_first", 0)) if self.window is not None else 0
        self.out_scale = float(p.get("out_scale", 1.0))
        self.eps = float(p.get("eps", 0.0))
        self.q_norm = self.k_norm = None
        if p.get("qk_norm"):
            self.q_norm = rt.vector32(names["q_norm"], weights["q_norm"])
            self.k_norm = rt.vector32(names["k_norm"], weights["k_norm"])
        self.freq, self.amplitude = None, 1.0
        if p.get("position") is not None:
            position = build_part("position", p["position"], getattr(weights, "checkpoint", {}), rt)
            self.freq, self.amplitude = position.frequencies()
            if 2 * self.freq.shape[0] > self.dk:
                raise ValueError(f"{2 * self.freq.shape[0]} rotated channels do not fit a head of {self.dk}")

    def forward(self, x, ctx, cache: LayerCache, out: Optional[torch.Tensor] = None):
        proj = K.linear(x, self.w_qkv, out_dtype=torch.float32)
        q = torch.empty(x.shape[0], self.H * self.dk, dtype=self.rt.dtype, device=proj.device)
        K.qk_norm_rope_store(proj, ctx.positions, cache.slot_mapping if cache.writes else None, self.q_norm, self.k_norm, self.eps,
                             self.freq, self.amplitude, q, cache.kpool, cache.vpool, self.H)
        attended = self.attend(q, ctx, cache, self.window, self.keep_first, self.out_scale)
        return K.linear(attended, self.w_o, out_dtype=torch.float32, out=out)


# ------------------------------------------------------------------ linear attention with a decay a head

@register_part("mixer", "decay_attention")
class DecayAttention(Part):
    """Linear attention whose memory fades by a constant factor a head.  Per head, with a memory ``S`` [key channel,
    value channel] in float32 that starts at zero and is carried from token to token:

        ``S <- decay[h] S + k v^T;  o = S^T q``        q, k, v = silu of their projections

    The read-outs of all heads together are divided by their root mean square, times ``norm``, times
    ``sigmoid(W_g x)``, times ``out_scale``; then ``W_o``.  The memory is the per-request state.

    params: hidden_size, num_heads, key_dim, value_dim, decay (one number a head), eps, out_scale.
    weights: q, k [H*dk, d], v, g [H*dv, d], norm [H*dv], o [d, H*dv]."""

    graph_safe = True
    idempotent = False        # a step moves the memory on

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, H, dk, dv = p["hidden_size"], p["num_heads"], p["key_dim"], p["value_dim"]
        return [WeightRequest(w["q"], (H * dk, d)), WeightRequest(w["k"], (H * dk, d)), WeightRequest(w["v"], (H * dv, d)),
                WeightRequest(w["g"], (H * dv, d)), WeightRequest(w["norm"], (H * dv,)), WeightRequest(w["o"], (d, H * dv))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, names = spec.params, spec.weights
        self.H, self.dk, self.dv = int(p["num_heads"]), int(p["key_dim"]), int(p["value_dim"])
        self.eps, self.out_scale = float(p["eps"]), float(p.get("out_scale", 1.0))
        decay = [float(x) for x in p["decay"]]
        if len(decay) != self.H:
            raise ValueError(f"{len(decay)} decays for {self.H} heads")
        self.decay = torch.tensor(decay, dtype=torch.float32).to(rt.device)
        order = ("q", "k", "v", "g")
        self.w_in = rt.weight("|".join(names[k] for k in order), torch.cat([weights[k] for k in order], dim=0))
        self.w_o = rt.weight(names["o"], weights["o"])
        self.norm = rt.vector32(names["norm"], weights["norm"])
        self.state_size = K.decay_state_floats(self.H, self.dk, self.dv)
        K.state_mixers_lib()

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state=StateNeed((self.state_size,), torch.float32))

    def forward(self, x, ctx, cache: LayerCache, out: Optional[torch.Tensor] = None):
        if not cache.writes:
            raise K.KernelError("a decay_attention mixer moves its memory on: it cannot read another entry's cache")
        H, dk, dv = self.H, self.dk, self.dv
        proj = K.linear(x, self.w_in, out_dtype=torch.float32)
        seq = ctx.per_seq
        # long portions go in runs, which read their operands twice and want silu applied beforehand; steps of few
        # tokens apply it as they read the projections, a launch fewer
        raw = not K.decay_in_runs(ctx.max_q_len, x.shape[0])
        act = proj if raw else K.silu_rows(proj, 2 * H * dk + H * dv)
        o = K.decay_attention(act, self.decay, cache.state, seq.q_start, seq.q_len, seq.state_slot, H, dk, dv,
                              max_q_len=ctx.max_q_len, raw=raw)
        y = K.gated_rmsnorm(o, proj, 2 * H * dk + H * dv, self.norm, self.eps, self.out_scale, self.rt.dtype)
        return K.linear(y, self.w_o, out_dtype=torch.float32, out=out)


# ------------------------------------------------------------------ two mixers side by side

@register_part("mixer", "side_by_side")
class SideBySide(Part):
    """Two mixers that read the same input; the result is the sum of theirs (each weighs its own output, its
    ``out_scale``).  One of them may keep keys and values in pages and one a state of fixed size: the pair asks the
    cache for both.  params: left, right (PartSpecs of family ``mixer`` whose ``forward`` takes ``out=``), hidden_size.
    The two outputs are handed on as float32 addends [2, T, d], which the next norm sums in float32."""

    @classmethod
    def weight_requests(cls, spec):
        return requests_of("mixer", spec.params["left"]) + requests_of("mixer", spec.params["right"])

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        checkpoint = getattr(weights, "checkpoint", {})
        self.left = build_part("mixer", spec.params["left"], checkpoint, rt)
        self.right = build_part("mixer", spec.params["right"], checkpoint, rt)
        self.hidden_size = int(spec.params["hidden_size"])
        a, b = self.left.cache_need(), self.right.cache_need()
        if (a.kv is not None and b.kv is not None) or (a.state is not None and b.state is not None):
            raise ValueError("two mixers side by side cannot both keep pages, or both keep a state")
        self._need = CacheNeed(kv=a.kv if a.kv is not None else b.kv, state=a.state if a.state is not None else b.state)
        self.graph_safe = bool(getattr(self.left, "graph_safe", False) and getattr(self.right, "graph_safe", False))
        self.idempotent = bool(getattr(self.left, "idempotent", True) and getattr(self.right, "idempotent", True))

    def cache_need(self) -> CacheNeed:
        return self._need

    def forward(self, x, ctx, cache: LayerCache):
        out = torch.empty(2, x.shape[0], self.hidden_size, dtype=torch.float32, device=x.device)
        self.left.forward(x, ctx, cache, out=out[0])
        self.right.forward(x, ctx, cache, out=out[1])
        return out


# ------------------------------------------------------------------ selective scan

@register_part("mixer", "selective_scan")
class SelectiveScan(Part):
    """A diagonal recurrence per channel whose step size, input and read-out depend on the token:

        ``[x | z] = W_in h;  u = silu(conv(x) + b_conv)`` (causal, ``taps`` tokens per channel, the last tap the token's own)
        ``[r | B | C] = W_x u;  dt = softplus(W_dt r + b_dt);  A = -exp(A_log)``
        ``S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c u_c B_n;  y_c = sum_n S[c, n] C_n + D_c u_c``
        ``out = W_o (y * silu(z))``

    The state ``S`` [inner, state] (float32, zero at the start) and the convolution's last ``taps - 1`` inputs are the
    per-request state.  dt, A, exp and the state are float32.

    params: hidden_size, inner, state, dt_rank, taps.
    weights: in [2 inner, d], conv [inner, taps], conv_b [inner], x [dt_rank + 2 state, inner], dt [inner, dt_rank],
    dt_b [inner], A_log [inner, state], D [inner], o [d, inner]."""

    graph_safe = True
    idempotent = False        # a step moves the state on

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, I, N, R, taps = p["hidden_size"], p["inner"], p["state"], p["dt_rank"], p["taps"]
        return [WeightRequest(w["in"], (2 * I, d)), WeightRequest(w["conv"], (I, taps)), WeightRequest(w["conv_b"], (I,)),
                WeightRequest(w["x"], (R + 2 * N, I)), WeightRequest(w["dt"], (I, R)), WeightRequest(w["dt_b"], (I,)),
                WeightRequest(w["A_log"], (I, N)), WeightRequest(w["D"], (I,)), WeightRequest(w["o"], (d, I))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, names = spec.params, spec.weights
        self.inner, self.N, self.R, self.taps = int(p["inner"]), int(p["state"]), int(p["dt_rank"]), int(p["taps"])
        I, N, R = self.inner, self.N, self.R
        self.w_in = rt.weight(names["in"], weights["in"])
        # the projection of u in two: the rows that feed the step sizes (their product's result is the next product's
        # input, in the compute type) and the rows of B and C (float32 results, they enter the recurrence)
        self.w_r = rt.weight(names["x"] + "|steps", weights["x"][:R].contiguous())
        self.w_bc = rt.weight(names["x"] + "|inout", weights["x"][R:].contiguous())
        self.w_dt = rt.weight(names["dt"], weights["dt"])
        self.w_o = rt.weight(names["o"], weights["o"])
        self.conv = weights["conv"].to(device=rt.device, dtype=torch.float32).contiguous()
        self.conv_b = rt.vector32(names["conv_b"], weights["conv_b"])
        self.dt_b = rt.vector32(names["dt_b"], weights["dt_b"])
        self.D = rt.vector32(names["D"], weights["D"])
        self.scan_floats = K.scan_state_floats(I, N)
        a = torch.zeros(I, self.scan_floats // I, dtype=torch.float32)
        a[:, :N] = -torch.exp(weights["A_log"].to(torch.float32))
        self.A = a.to(rt.device)
        self.state_size = _up4(self.scan_floats + (self.taps - 1) * I)
        K.state_mixers_lib()

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state=StateNeed((self.state_size,), torch.float32))

    def forward(self, x, ctx, cache: LayerCache, out: Optional[torch.Tensor] = None):
        if not cache.writes:
            raise K.KernelError("a selective_scan mixer moves its state on: it cannot read another entry's cache")
        seq = ctx.per_seq
        xz = K.linear(x, self.w_in, out_dtype=torch.float32)
        u32, u = K.conv_silu(xz, self.inner, self.conv, self.conv_b, cache.state, self.scan_floats, ctx.seq_of_token,
                             seq.q_start, seq.q_len, seq.state_slot, self.rt.dtype, max_q_len=ctx.max_q_len)
        dt_pre = K.linear(K.linear(u, self.w_r), self.w_dt, out_dtype=torch.float32)
        bc = K.linear(u, self.w_bc, out_dtype=torch.float32)
        y = K.selective_scan(dt_pre, self.dt_b, u32, xz, self.inner, bc, self.A, self.D, cache.state, seq.q_start, seq.q_len,
                             seq.state_slot, self.N, self.rt.dtype, max_q_len=ctx.max_q_len)
        return K.linear(y, self.w_o, out_dtype=torch.float32, out=out)
