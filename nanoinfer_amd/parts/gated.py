"""Parts around a stream whose sublayers are normed on both sides: attention whose values are its keys, attention
over a low-rank latent that layers may share, a matrix memory with exponential gates, a feed-forward whose activation
is a polynomial of normed powers, the block with a norm before and behind each sublayer, and the mix of all earlier
states of the stream that takes a layer's result's place.

Kinds registered here: mixer ``keyed_attention``, ``latent_attention`` and ``gated_memory``; feed_forward
``poly_norm_mlp``; block ``sandwich``; stream_mix ``depth_average``.  Every size and constant is a parameter of the
part's spec.
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .. import kernels as K
from ..registry import register_part
from .base import Block, CacheNeed, KVNeed, LayerCache, Part, StateNeed, WeightRequest, pending_for
from .hybrid import PagedSoftmax
from .stateful import WindowAttention


# ------------------------------------------------------------------ softmax attention whose values are its keys

@register_part("mixer", "keyed_attention")
class KeyedAttention(WindowAttention):
    """Causal softmax attention with grouped heads and no value projection: the keys as projected, before their
    norm, are the values.  In float32: an RMS norm over a token's whole query projection and one over its whole key
    projection; a query factor ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)`` at position p;
    ``score = q . k * scale - r1[h] * ln(1 + r2[h] * (i - j))``; a window of ``window`` keys (the query's own among them;
    None: every earlier key, for which ``max_positions`` bounds the distances).

    params: hidden_size, num_heads, num_kv_heads, key_dim, scale, window, eps, temp_coef and temp_every (None: no
    factor), penalty (True: the weights r1, r2), max_positions.
    weights: q [H*dk, d], k [G*dk, d], o [d, H*dk], q_norm [H*dk], k_norm [G*dk], r1 [H], r2 [H]."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, H, G, dk = p["hidden_size"], p["num_heads"], p["num_kv_heads"], p["key_dim"]
        out = [WeightRequest(w["q"], (H * dk, d)), WeightRequest(w["k"], (G * dk, d)), WeightRequest(w["o"], (d, H * dk)),
               WeightRequest(w["q_norm"], (H * dk,)), WeightRequest(w["k_norm"], (G * dk,))]
        if p.get("penalty"):
            out += [WeightRequest(w["r1"], (H,)), WeightRequest(w["r2"], (H,))]
        return out

    def __init__(self, spec, weights, rt):
        p = dict(spec.params)
        p.update(value_dim=p["key_dim"], qk_norm=True, keep_first=0, position=None)
        super().__init__(type(spec)(spec.kind, p, spec.weights), weights, rt)

    def _stacked_projection(self, names, weights, rt):
        return rt.weight("|".join((names["q"], names["k"])), torch.cat([weights["q"], weights["k"]], dim=0))

    def _bias_table(self, p, names, weights, rt) -> Optional[torch.Tensor]:
        if not p.get("penalty"):
            return None
        # the penalty at every distance a query can see, worked out once in float64: the kernel looks it up
        distances = int(p["window"]) if p.get("window") is not None else int(p["max_positions"])
        dist = torch.arange(distances, dtype=torch.float64)[:, None]
        r1, r2 = weights["r1"].to(torch.float64)[None, :], weights["r2"].to(torch.float64)[None, :]
        return (-r1 * torch.log1p(r2 * dist)).to(torch.float32).to(rt.device).contiguous()

    def forward(self, x, ctx, cache: LayerCache, out: Optional[torch.Tensor] = None):
        proj = K.linear(x, self.w_qkv, out_dtype=torch.float32)
        q = torch.empty(x.shape[0], self.H * self.dk, dtype=self.rt.dtype, device=proj.device)
        K.qk_norm_rope_store(proj, ctx.positions, cache.slot_mapping if cache.writes else None, self.q_norm, self.k_norm, self.eps,
                             None, 1.0, q, cache.kpool, cache.vpool, self.H, values_are_keys=True)
        attended = self.attend(q, ctx, cache, self.window, 0, 1.0)
        return K.linear(attended, self.w_o, out_dtype=torch.float32, out=out)


# ------------------------------------------------------------------ softmax attention over a low-rank latent

# the longest portion of a step from which on a latent attention writes keys and values of every head out for the step
# (None: never): below it the products over all visible latents cost more than attention over the latents themselves saves
LATENT_EXPAND_FROM = 256
# the most channels a token's row in the pages may have for attention over the rows themselves (the attention kernels'
# value channels); a wider row is only ever read through the written-out way
LATENT_ROW_MAX = 256


@register_part("mixer", "latent_attention")
class LatentAttention(Part):
    """Causal softmax attention whose keys and values of every head are projections of one latent ``c`` of ``rank``
    numbers a token, the only thing kept in the pages:

        ``c_q = rmsnorm(W_dq x) * w_dq;  q = W_uq c_q;  c = rmsnorm(W_dkv x) * w_dkv``
        ``k_h = W_uk[h] c,  v_h = W_uv[h] c;  score = q_h . k_h * scale``      (no positions)
        ``out = W_o (concat_h(softmax(score) v_h) * sigmoid(W_g x))``

    The key projection is taken to the query's side and the value projection behind the softmax: ``q_h . (W_uk[h] c) =
    (W_uk[h]^T q_h) . c`` and ``sum_j p_j W_uv[h] c_j = W_uv[h] sum_j p_j c_j``, so the kernel runs H query heads of
    ``rank`` channels on one key/value head whose keys and values are the same pool.  A part without ``dkv`` in its
    weights reads the latents that another entry of the order wrote (``LayerRun.writes_cache`` False), with its own
    W_uk, W_uv, queries and window.

    With ``rot_dim`` r > 0 positions enter through r more channels: ``W_dkv`` has ``rank + r`` rows, of which the last r,
    not normed, are rotated (``position``: a PartSpec of family ``position``; ``adjacent_pairs``: channel 2i turns with
    channel 2i + 1) and kept in the pages behind the latent, one key part for all heads; a query head is ``key_dim``
    channels that meet ``W_uk[h] c`` and r rotated ones that meet that part; the two dot products are summed before the
    scale.  The kernel's key is then the whole row ``[c | k_rot]`` and a query as the row sees it ``[W_uk[h]^T q_h |
    q_rot]``; the r extra value channels meet zero rows of W_uv.

    Steps whose longest portion has ``expand_from`` tokens or more (and that are not recorded) take the other way:
    ``k_h`` and ``v_h`` of every latent the step can see are written out once for the step, and attention runs over H
    heads of ``key_dim + rot_dim`` and ``value_dim`` channels, a fraction of the products where the latent is wider than a head.

    params: hidden_size, num_heads, key_dim, value_dim, q_rank (None: the queries are ``W_q x``, no latent of their own),
    rank, scale, window (None: every earlier key), eps, rot_dim (default 0), position, adjacent_pairs, gate ("channel", the
    default: a gate a value channel; "head": one a head), expand_from (default ``LATENT_EXPAND_FROM``; None: never; it is
    never taken where ``rank + rot_dim < key_dim + rot_dim + value_dim``, and always where ``rank + rot_dim`` is more than
    ``LATENT_ROW_MAX``: such a part reads the host lists in every step and is not ``graph_safe``).
    weights: dq [q_rank, d], dq_norm [q_rank], uq [H*(dk+r), q_rank] (or q [H*(dk+r), d]), dkv [rank + r, d] and dkv_norm
    [rank] (both or neither), uk [H*dk, rank], uv [H*dv, rank], g [H*dv, d] (or [H, d]), o [d, H*dv], sink [H] (absent:
    none; one more term ``exp(sink[h])`` in the softmax's denominator)."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, H, dk, dv, rq, r = p["hidden_size"], p["num_heads"], p["key_dim"], p["value_dim"], p.get("q_rank"), p["rank"]
        dr = int(p.get("rot_dim", 0))
        gates = H if p.get("gate", "channel") == "head" else H * dv
        out = [WeightRequest(w["uk"], (H * dk, r)), WeightRequest(w["uv"], (H * dv, r)), WeightRequest(w["g"], (gates, d)),
               WeightRequest(w["o"], (d, H * dv))]
        if rq is None:
            out.append(WeightRequest(w["q"], (H * (dk + dr), d)))
        else:
            out += [WeightRequest(w["dq"], (rq, d)), WeightRequest(w["dq_norm"], (rq,)), WeightRequest(w["uq"], (H * (dk + dr), rq))]
        if "dkv" in w:
            out += [WeightRequest(w["dkv"], (r + dr, d)), WeightRequest(w["dkv_norm"], (r,))]
        if "sink" in w:
            out.append(WeightRequest(w["sink"], (H,)))
        if p.get("position") is not None:
            from .standard import requests_of
            out += requests_of("position", p["position"])
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, names = spec.params, spec.weights
        self.H, self.dk, self.dv = int(p["num_heads"]), int(p["key_dim"]), int(p["value_dim"])
        self.q_rank = None if p.get("q_rank") is None else int(p["q_rank"])
        self.rank, self.dr = int(p["rank"]), int(p.get("rot_dim", 0))
        self.row, self.dq = self.rank + self.dr, self.dk + self.dr       # what a token keeps; a query head
        self.window = None if p.get("window") is None else int(p["window"])
        self.eps = float(p["eps"])
        self.own = "dkv" in names
        gate = p.get("gate", "channel")
        if gate not in ("channel", "head"):
            raise ValueError(f"gate {gate!r} is not 'channel' or 'head'")
        self.gate_per_head = gate == "head"
        H, dk, dv, dr, rank, row = self.H, self.dk, self.dv, self.dr, self.rank, self.row
        # rows of more channels than the attention kernels take as values: every step writes the heads' keys and values
        # out, which reads the step's host lists, so no step of such a model is recorded
        self.always_expand = row > LATENT_ROW_MAX
        if self.always_expand:
            self.graph_safe = False
        self.freq, self.amplitude, self.adjacent = None, 1.0, bool(p.get("adjacent_pairs", False))
        if dr:
            from .standard import build_part
            if p.get("position") is None:
                raise ValueError("rotated channels need a position part")
            self.freq, self.amplitude = build_part("position", p["position"], getattr(weights, "checkpoint", {}), rt).frequencies()
            if 2 * self.freq.shape[0] != dr:
                raise ValueError(f"{2 * self.freq.shape[0]} rotated channels, rot_dim is {dr}")
        # one product for everything that reads the layer's input: the queries (or their latent), the latent of keys and
        # values with its rotated part if this layer makes its own, and the gate; float32 out (norms, rotation and the
        # gate read the accumulators)
        first = ["q" if self.q_rank is None else "dq"] + (["dkv"] if self.own else []) + ["g"]
        self.latent_col = int(weights[first[0]].shape[0])
        self.gate_col = self.latent_col + (row if self.own else 0)
        self.w_in = rt.weight("|".join(names[k] for k in first), torch.cat([weights[k] for k in first], dim=0))
        self.dkv_norm = rt.vector32(names["dkv_norm"], weights["dkv_norm"]) if self.own else None
        self.dq_norm = self.w_uq = None
        if self.q_rank is not None:
            self.dq_norm = rt.vector32(names["dq_norm"], weights["dq_norm"])
            self.w_uq = rt.weight(names["uq"], weights["uq"])
        self.w_o = rt.weight(names["o"], weights["o"])
        self.sink = rt.vector32(names["sink"], weights["sink"]) if "sink" in names else None
        # per head: [dk + dr, rank + dr] for the queries' side (W_uk[h], and an identity that hands the rotated channels
        # on), [rank + dr, dv] behind the softmax (W_uv[h]^T over zero rows)
        uk = torch.zeros(H, self.dq, row, dtype=weights["uk"].dtype)
        uk[:, :dk, :rank] = weights["uk"].view(H, dk, rank)
        uv = torch.zeros(H, dv, row, dtype=weights["uv"].dtype)
        uv[:, :, :rank] = weights["uv"].view(H, dv, rank)
        if dr:
            uk[:, dk:, rank:] = torch.eye(dr, dtype=uk.dtype)
        self.uk = rt.matrix(names["uk"] + "|row", uk.view(H * self.dq, row)).view(H, self.dq, row)
        self.uv_t = rt.matrix(names["uv"] + "|row", uv.view(H * dv, row)).view(H, dv, row).transpose(1, 2)
        self.core = PagedSoftmax(H, 1, row, row, float(p["scale"]), one_pool=True, sink=self.sink)
        # steps with long portions: keys and values of every head are made of the latents the step can see, once,
        # and attention runs at the heads' own sizes
        self.expand_from = p.get("expand_from", LATENT_EXPAND_FROM)
        if row < self.dq + dv and not self.always_expand:      # attention over the latents is then the smaller sum of products already
            self.expand_from = None
        if self.expand_from is not None:
            self.expand_from = max(2, int(self.expand_from))
        self.eager_portion_from = self.expand_from        # that way reads the step's host lists
        self.heads = PagedSoftmax(H, H, self.dq, dv, float(p["scale"]), sink=self.sink)
        self.uk_rows = self.uk.view(H * self.dq, row)
        self.uv_rows = self.uv_t.transpose(1, 2).view(H * dv, row)
        K.stream_lib()

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv=KVNeed(1, self.row, None, 0))       # one pool: the latents are keys and values

    def _queries(self, x, proj, ctx, cache: LayerCache) -> torch.Tensor:
        """The queries [T, H * (dk + dr)] in the compute type, rotated where they have rotated channels; a layer that
        makes its own latents also puts them into the pages here: normed, their rotated part turned."""
        T, H = x.shape[0], self.H
        direct = self.q_rank is None
        if self.own and not (direct and self.dr):
            K.qk_norm_rope_store(proj, ctx.positions, cache.slot_mapping, None, self.dkv_norm, self.eps, self.freq, self.amplitude,
                                 None, cache.kpool, cache.vpool, 0, col=self.latent_col, per_head=True, adjacent=self.adjacent,
                                 rot_at_k=self.rank, k_normed=self.rank)
        if not direct:
            q = K.rmsnorm_cols(proj, 0, self.dq_norm, self.eps, self.rt.dtype)
            if not self.dr:
                return K.linear(q, self.w_uq)
            proj = K.linear(q, self.w_uq, out_dtype=torch.float32)
        q = torch.empty(T, H * self.dq, dtype=self.rt.dtype, device=x.device)
        if direct and self.own and self.dr:
            # queries and latents lie side by side in the product's rows: one pass turns both and stores the latents
            K.qk_norm_rope_store(proj, ctx.positions, cache.slot_mapping, None, self.dkv_norm, self.eps, self.freq, self.amplitude,
                                 q, cache.kpool, cache.vpool, H, per_head=True, adjacent=self.adjacent, q_dim=self.dq,
                                 rot_at_q=self.dk, rot_at_k=self.rank, k_normed=self.rank)
        else:
            K.qk_norm_rope_store(proj, ctx.positions, None, None, None, self.eps, self.freq, self.amplitude, q, None, None, H,
                                 adjacent=self.adjacent, q_dim=self.dq, rot_at_q=self.dk, queries_only=True)
        return q

    def _gated(self, y, proj):
        return K.gate_rows(y, proj, self.gate_col, every=self.dv if self.gate_per_head else 1)

    def forward(self, x, ctx, cache: LayerCache, out: Optional[torch.Tensor] = None):
        T, H = x.shape[0], self.H
        if cache.writes != self.own:
            raise K.KernelError("a latent_attention part writes the latents it makes, and only those")
        proj = K.linear(x, self.w_in, out_dtype=torch.float32)
        q = self._queries(x, proj, ctx, cache)
        if self.always_expand or (self.expand_from is not None and not ctx.recording and ctx.max_q_len >= self.expand_from):
            return K.linear(self._gated(self._over_heads(q, ctx, cache), proj), self.w_o, out_dtype=torch.float32, out=out)
        # the queries as the rows of the pages see them, [T, H * row]: a product per head, read and written in place
        seen = torch.empty(T, H * self.row, dtype=self.rt.dtype, device=x.device)
        torch.bmm(q.view(T, H, self.dq).transpose(0, 1), self.uk, out=seen.view(T, H, self.row).transpose(0, 1))
        K.note_library_call()
        mixed = self.core(seen, ctx, cache.kpool, cache.kpool, cache.block_table, self.window)
        per_head = mixed.view(T, H, self.row).transpose(0, 1)
        heads = torch.bmm(per_head, self.uv_t) if mixed.dtype == torch.float32 else torch.bmm(per_head, self.uv_t, out_dtype=torch.float32)
        K.note_library_call()
        y = K.gate_heads(heads, proj, self.gate_col, self.rt.dtype, per_head=self.gate_per_head)
        return K.linear(y, self.w_o, out_dtype=torch.float32, out=out)

    def _over_heads(self, q, ctx, cache: LayerCache) -> torch.Tensor:
        """Attention with keys and values of every head written out: the pages that hold a key some token of the step
        can see are picked out of the pool, ``k = W_uk c`` (beside the rotated channels, the same for every head) and
        ``v = W_uv c`` are two products over them, laid out as pools of H heads, and the kernels walk them through a
        block table of their own that holds nothing else.  A tile of queries starts at the tile of 64 keys in which its
        first token's window starts; the picked pages start there."""
        ps, window = int(cache.kpool.shape[2]), self.window
        B, width = cache.block_table.shape
        pairs, table, at = [], np.full((B, width), -1, dtype=np.int32), 0
        for b, (n, total) in enumerate(zip(ctx.q_len, ctx.context_len)):
            first = 0 if window is None else max(total - n - window + 1, 0) // 64 * 64
            p0, p1 = first // ps, -(-total // ps)
            pairs.append(np.stack([np.full(p1 - p0, b, dtype=np.int32), np.arange(p0, p1, dtype=np.int32)], axis=1))
            table[b, p0:p1] = np.arange(at, at + p1 - p0, dtype=np.int32)
            at += p1 - p0
        flat = np.concatenate([np.concatenate(pairs).reshape(-1), table.reshape(-1)])
        dev = ctx.upload_ints(flat)
        pairs_dev, table_dev = dev[: 2 * at].view(at, 2), dev[2 * at:].view(B, width)
        latents = K.gather_pages(cache.kpool, cache.block_table, pairs_dev).view(at * ps, self.row)
        keys = K.rows_to_pages(K.linear(latents, self.uk_rows), ps, self.H, self.dq)
        values = K.rows_to_pages(K.linear(latents, self.uv_rows), ps, self.H, self.dv)
        return self.heads(q, ctx, keys, values, table_dev, window)


# ------------------------------------------------------------------ matrix memory with exponential gates

@register_part("mixer", "gated_memory")
class GatedMemory(Part):
    """A matrix memory per head whose input and forget gates are exponentials kept in range by a running maximum.
    Per head, with ``S`` [key channel, value channel], ``n`` [key channel] and ``m``, all float32, zero at the start and
    carried from token to token:

        ``li = cap tanh((W_i x + b_i) / cap);  lf = logsigmoid(cap tanh((W_f x + b_f) / cap));  m' = max(lf + m, li)``
        ``S <- exp(lf + m - m') S + exp(li - m') k v^T;  n likewise with k alone;  m <- m'``
        ``o = S^T q / (max(|n . q|, exp(-m)) + 1e-6)``          q = W_q x * key_dim^-1/2, k = W_k x, v = W_v x

    Every head's ``o`` is divided by its root mean square; the heads together times ``norm``, times ``sigmoid(W_g x)``,
    then ``W_o``.  S, n and m are the per-request state.

    params: hidden_size, num_heads, key_dim, value_dim, gate_cap, eps.
    weights: q, k [H*dk, d], v, g [H*dv, d], i, f [H, d], i_b, f_b [H], norm [H*dv], o [d, H*dv]."""

    graph_safe = True
    idempotent = False        # a step moves the memory on

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, H, dk, dv = p["hidden_size"], p["num_heads"], p["key_dim"], p["value_dim"]
        return [WeightRequest(w["q"], (H * dk, d)), WeightRequest(w["k"], (H * dk, d)), WeightRequest(w["v"], (H * dv, d)),
                WeightRequest(w["g"], (H * dv, d)), WeightRequest(w["i"], (H, d)), WeightRequest(w["f"], (H, d)),
                WeightRequest(w["i_b"], (H,)), WeightRequest(w["f_b"], (H,)), WeightRequest(w["norm"], (H * dv,)),
                WeightRequest(w["o"], (d, H * dv))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, names = spec.params, spec.weights
        self.H, self.dk, self.dv = int(p["num_heads"]), int(p["key_dim"]), int(p["value_dim"])
        self.cap, self.eps = float(p["gate_cap"]), float(p["eps"])
        H, dk, dv = self.H, self.dk, self.dv
        # one product, float32 out (everything but the gate's rows enters the recurrence); every block of rows starts
        # at a whole 16-byte piece of the result
        blocks, self.cols, at = [], {}, 0
        for key in ("q", "k", "v", "g", "i", "f"):
            if key != "f":                      # f follows i directly: the kernel reads zi [H] | zf [H]
                pad = (-at) % 4
                if pad:
                    blocks.append(torch.zeros(pad, weights[key].shape[1], dtype=weights[key].dtype))
                    at += pad
            self.cols[key] = at
            blocks.append(weights[key])
            at += weights[key].shape[0]
        pad = (-at) % 16
        if pad:
            blocks.append(torch.zeros(pad, weights["q"].shape[1], dtype=weights["q"].dtype))
        order = ("q", "k", "v", "g", "i", "f")
        self.w_in = rt.weight("|".join(names[k] for k in order) + "|pieces", torch.cat(blocks, dim=0))
        self.gate_bias = torch.cat([weights["i_b"].to(torch.float32), weights["f_b"].to(torch.float32)]).to(rt.device).contiguous()
        self.norm = rt.vector32(names["norm"], weights["norm"])
        self.w_o = rt.weight(names["o"], weights["o"])
        self.state_size = K.memory_state_floats(H, dk, dv)
        K.state_mixers_lib()

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state=StateNeed((self.state_size,), torch.float32))

    def forward(self, x, ctx, cache: LayerCache, out: Optional[torch.Tensor] = None):
        if not cache.writes:
            raise K.KernelError("a gated_memory mixer moves its memory on: it cannot read another entry's cache")
        c, seq = self.cols, ctx.per_seq
        proj = K.linear(x, self.w_in, out_dtype=torch.float32)
        raw, m = K.gated_memory(proj, c["q"], c["k"], c["v"], c["i"], self.gate_bias, self.cap, self.dk ** -0.5, cache.state,
                                seq.q_start, seq.q_len, seq.state_slot, self.H, self.dk, self.dv, max_q_len=ctx.max_q_len)
        y = K.memory_norm(raw, m, proj, c["g"], self.norm, self.eps, cache.state, ctx.seq_of_token, seq.q_start, seq.q_len,
                          seq.state_slot, self.dk, self.rt.dtype)
        return K.linear(y, self.w_o, out_dtype=torch.float32, out=out)


# ------------------------------------------------------------------ feed-forward

@register_part("feed_forward", "poly_norm_mlp")
class PolyNormMLP(Part):
    """``W_down act(W_up x)`` with ``act(z) = a N(z) + b N(z^2) + c N(z^3) + e``: powers element by element, ``N`` the
    division of a token's hidden row by its root mean square, in float32 on the product's accumulators.
    params: hidden_size, intermediate_size, eps.  weights: up [I, d], down [d, I], act [4] = (a, b, c, e)."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        p, w = spec.params, spec.weights
        d, i = p["hidden_size"], p["intermediate_size"]
        return [WeightRequest(w["up"], (i, d)), WeightRequest(w["down"], (d, i)), WeightRequest(w["act"], (4,))]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        names = spec.weights
        self.eps = float(spec.params["eps"])
        self.w_up = rt.weight(names["up"], weights["up"])
        self.w_down = rt.weight(names["down"], weights["down"])
        self.coef = rt.vector32(names["act"], weights["act"])

    def forward(self, x, ctx):
        z = K.linear(x, self.w_up, out_dtype=torch.float32)
        return K.linear(K.poly_norm(z, self.coef, self.eps, self.rt.dtype), self.w_down, out_dtype=torch.float32)


# ------------------------------------------------------------------ block

@register_part("block", "sandwich")
class SandwichBlock(Block):
    """``h += post1(mixer(norm1(h))); h += post2(ffn(norm2(h)))``: a norm before and a norm behind each sublayer, the
    one behind applied to the sublayer's float32 output before it is added to the float32 stream.  ``ffn_norm``,
    ``ffn`` and ``ffn_post`` may be absent together: the block is its first sublayer alone."""

    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "mixer_post": "norm", "ffn_norm": "norm", "ffn": "feed_forward",
             "ffn_post": "norm"}
    OPTIONAL = ("ffn_norm", "ffn", "ffn_post")

    @classmethod
    def _roles(cls, spec):
        missing = [r for r in cls.ROLES if r not in spec.parts and r not in cls.OPTIONAL]
        extra = [r for r in spec.parts if r not in cls.ROLES]
        have = [r for r in cls.OPTIONAL if r in spec.parts]
        if have and len(have) != len(cls.OPTIONAL):
            missing += [r for r in cls.OPTIONAL if r not in spec.parts]
        if missing or extra:
            raise ValueError(f"a block of kind {spec.kind!r} has the parts {sorted(cls.ROLES)}; "
                             f"missing: {missing}, not known: {extra}")
        return [(r, f) for r, f in cls.ROLES.items() if r in spec.parts]

    @staticmethod
    def _add_normed(h, y, post):
        if y.dtype != torch.float32:
            y = y.to(torch.float32)
        return K.add_rmsnormed(h, y.contiguous(), post.weight, post.eps)

    def forward(self, h, pending, ctx, cache: LayerCache):
        x = self.mixer_norm.forward(h, pending_for(self.mixer_norm, pending, self.rt.dtype))
        self._add_normed(h, self.mixer.forward(x, ctx, cache), self.mixer_post)
        if "ffn" in self.roles:
            x = self.ffn_norm.forward(h, None)
            self._add_normed(h, self.ffn.forward(x, ctx), self.ffn_post)
        return h, None


# ------------------------------------------------------------------ the mix of all earlier states of the stream

@register_part("stream_mix", "depth_average")
class DepthAverage(Part):
    """With ``X_0`` the embedding's output and ``X_(i+1)`` the result of entry i of the order, what goes on behind
    entry i is ``sum_(j <= i+1) w_i[j] X_j``.  params: entries, size.  weights: ``w<i>`` [i + 2] for every entry i."""

    graph_safe = True

    @classmethod
    def weight_requests(cls, spec):
        return [WeightRequest(spec.weights[f"w{i}"], (i + 2,)) for i in range(spec.params["entries"])]

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.weights = [rt.vector32(spec.weights[f"w{i}"], weights[f"w{i}"]) for i in range(int(spec.params["entries"]))]
        K.stream_lib()

    def settle(self, h: torch.Tensor, pending: Optional[torch.Tensor]) -> torch.Tensor:
        """``h`` with an addend it has not received yet."""
        return h if pending is None else K.stream_add(h, pending.contiguous())

    def forward(self, history: torch.Tensor, entry: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``history`` float32 [entries + 1, T, size] whose rows 0 .. entry + 1 are filled; the mix goes to ``out``."""
        if out is None:
            out = torch.empty(history.shape[1], history.shape[2], dtype=torch.float32, device=history.device)
        return K.depth_mix(history[: entry + 2], self.weights[entry], out)
