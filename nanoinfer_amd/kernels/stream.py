"""Python face of the kernels in ``csrc/stream_ops.hip``, ``csrc/delta_rule.hip`` and
``csrc/bias_attention.hip``: sums onto the residual stream, a scaled embedding with position rows, a
token's side input, the router and its experts, the gated delta rule, and attention with a bias by
distance.  Shapes, types and devices are checked here, on the host, before a kernel is launched.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..csrc import build as _build
from . import KernelError, _check, _gpu, _load, _need, _ptr, _stream, dtype_code


def stream_lib() -> ctypes.CDLL:
    return _load(_build.STREAM_OPS)


def bias_attention_lib() -> ctypes.CDLL:
    return _load(_build.BIAS_ATTENTION)


def delta_rule_lib(key_size: int) -> ctypes.CDLL:
    return _load(_build.delta_rule_target(key_size))


_size_t = ctypes.c_size_t
_float = ctypes.c_float


# ------------------------------------------------------------------ the residual stream

def embed_scaled(ids: torch.Tensor, positions: torch.Tensor, table: torch.Tensor, pos_table: Optional[torch.Tensor],
                 scale: float, out: torch.Tensor) -> torch.Tensor:
    """``out[t] = table[ids[t]] * scale + pos_table[positions[t]]`` as float32 (no position rows: the first term)."""
    T = ids.shape[0]
    vocab, d = table.shape
    _gpu(ids, "ids", torch.int32, (T,))
    _gpu(positions, "positions", torch.int32, (T,))
    _gpu(table, "table")
    _gpu(out, "out", torch.float32, (T, d))
    max_pos = 0
    if pos_table is not None:
        max_pos = pos_table.shape[0]
        _gpu(pos_table, "pos_table", table.dtype, (max_pos, d))
    _check(stream_lib().ni_embed_scaled(_ptr(ids), _ptr(positions), _ptr(table), _ptr(pos_table), _ptr(out), T, d, vocab,
                                        max_pos, _float(scale), dtype_code(table.dtype), _stream()), "embed_scaled")
    return out


def add_vector(h: torch.Tensor, vec: torch.Tensor) -> torch.Tensor:
    """``h[t] += vec`` for every row of the float32 stream."""
    T, d = h.shape
    _gpu(h, "h", torch.float32)
    _gpu(vec, "vec", torch.float32, (d,))
    _check(stream_lib().ni_add_vector(_ptr(h), _ptr(vec), T, d, _stream()), "add_vector")
    return h


def embed_pair_hash(ids: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor, q_start: torch.Tensor,
                    q_len: torch.Tensor, state_slot: torch.Tensor, last_token: torch.Tensor, table: torch.Tensor,
                    pairs: Optional[torch.Tensor], buckets: int, mul_prev: int, mul_cur: int, scale: float, out: torch.Tensor,
                    freq: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t] = table[ids[t]] * scale + pairs[(prev * mul_prev + ids[t] * mul_cur) mod buckets]`` as float32, ``prev``
    the token before ``ids[t]`` in its sequence; a sequence's first token (position 0) takes row ``buckets``.
    ``last_token`` int32 [slots, 1] holds, per state slot, the last token of the sequence so far: it serves the first
    row of a portion and is moved on by this call.  ``pairs`` None: no second table.  ``freq`` float32 [(d + 1) // 2]:
    a sinusoid of the position is added, column 2i ``sin(position * freq[i])`` and column 2i + 1 the cosine."""
    T = ids.shape[0]
    B = q_start.shape[0]
    vocab, d = table.shape
    for name, t in (("ids", ids), ("positions", positions), ("seq_of_token", seq_of_token)):
        _gpu(t, name, torch.int32, (T,))
    for name, t in (("q_start", q_start), ("q_len", q_len), ("state_slot", state_slot)):
        _gpu(t, name, torch.int32, (B,))
    _need(last_token.is_cuda and last_token.dtype == torch.int32 and last_token.is_contiguous() and last_token.dim() == 2
          and last_token.shape[1] == 1, "last_token must be int32 [slots, 1] on the GPU")
    _gpu(table, "table")
    if pairs is not None:
        _gpu(pairs, "pairs", table.dtype, (buckets + 1, d))
    if freq is not None:
        _gpu(freq, "freq", torch.float32, ((d + 1) // 2,))
    _gpu(out, "out", torch.float32, (T, d))
    _check(stream_lib().ni_embed_pair_hash(_ptr(ids), _ptr(positions), _ptr(seq_of_token), _ptr(q_start), _ptr(q_len),
                                           _ptr(state_slot), _ptr(last_token), _ptr(table), _ptr(pairs), _ptr(out), T, B, d, vocab,
                                           int(buckets), ctypes.c_longlong(mul_prev), ctypes.c_longlong(mul_cur), _float(scale),
                                           _ptr(freq), dtype_code(table.dtype), _stream()), "embed_pair_hash")
    return out


def add_rows_vector(h: torch.Tensor, extra: Optional[torch.Tensor], vec: torch.Tensor) -> torch.Tensor:
    """``h[t] = (h[t] + extra[t]) + vec`` for every row of the float32 stream (``extra`` may be absent)."""
    T, d = h.shape
    _gpu(h, "h", torch.float32)
    if extra is not None:
        _gpu(extra, "extra", torch.float32, (T, d))
    _gpu(vec, "vec", torch.float32, (d,))
    _check(stream_lib().ni_add_rows_vector(_ptr(h), _ptr(extra), _ptr(vec), T, d, _stream()), "add_rows_vector")
    return h


def stream_add(h: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None,
               x_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``h += (a + b)`` in float32 (``b`` may be absent); ``x_out``, if given, takes the new stream in its own
    type.  ``a`` and ``b`` are float32 or bfloat16 [T, d]."""
    T, d = h.shape
    _gpu(h, "h", torch.float32)
    _gpu(a, "a", None, (T, d))
    if b is not None:
        _gpu(b, "b", None, (T, d))
    if x_out is not None:
        _gpu(x_out, "x_out", None, (T, d))
    _check(stream_lib().ni_stream_add(_ptr(h), _ptr(a), dtype_code(a.dtype), _ptr(b), dtype_code(b.dtype) if b is not None else 0,
                                      _ptr(x_out), dtype_code(x_out.dtype) if x_out is not None else 0, T, d, _stream()),
           "stream_add")
    return h


def gated_side(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, first: int, size: int, out: torch.Tensor) -> torch.Tensor:
    """``out[t, c] = gelu_tanh(z[t, c]) * table[ids[t], first + c]`` for c < size, zero in the padding columns."""
    T, width = z.shape
    vocab, cols = table.shape
    _gpu(z, "z", torch.float32)
    _gpu(table, "table")
    _gpu(ids, "ids", torch.int32, (T,))
    _gpu(out, "out", table.dtype, (T, width))
    _need(0 <= first and first + size <= cols and size <= width, "the side rows do not lie inside the table")
    _check(stream_lib().ni_gated_side(_ptr(z), _ptr(table), _ptr(ids), _ptr(out), T, width, size, cols, first, vocab,
                                      dtype_code(table.dtype), _stream()), "gated_side")
    return out


def add_rmsnormed(h: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``h += y / sqrt(mean(y^2) + eps) * weight`` row by row, all float32."""
    T, d = h.shape
    _gpu(h, "h", torch.float32)
    _gpu(y, "y", torch.float32, (T, d))
    _gpu(weight, "weight", torch.float32, (d,))
    _check(stream_lib().ni_add_rmsnormed(_ptr(h), _ptr(y), _ptr(weight), T, d, _float(eps), _stream()), "add_rmsnormed")
    return h


def post_norm(h: torch.Tensor, addends: Optional[torch.Tensor], alpha: float, weight: torch.Tensor, eps: float,
              x: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``h <- rmsnorm(alpha * h + sum of addends) * weight`` in place, all float32: the stream of a block whose norm stands
    behind the sum.  ``addends`` float32 [T, d] or [S, T, d] (summed in their order), or None; ``x`` [T, d] in a compute
    type takes a copy of the result for the products that read it next."""
    T, d = h.shape
    _gpu(h, "h", torch.float32)
    _gpu(weight, "weight", torch.float32, (d,))
    n = 0
    if addends is not None:
        _gpu(addends, "addends", torch.float32)
        _need(addends.shape[-2:] == (T, d) and addends.dim() in (2, 3), "addends are float32 [T, d] or [S, T, d]")
        n = 1 if addends.dim() == 2 else addends.shape[0]
    if x is not None:
        _gpu(x, "x", None, (T, d))
    _check(stream_lib().ni_post_norm(_ptr(h), _ptr(addends), n, _float(alpha), _ptr(weight), _float(eps), _ptr(x),
                                     0 if x is None else dtype_code(x.dtype), T, d, _stream()), "post_norm")
    return h


def rmsnorm_cols(rows: torch.Tensor, col: int, weight: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * weight`` over the columns ``col .. col + len(weight)`` of ``rows`` float32 [T, wide]
    (some of a stacked product's accumulators); [T, len(weight)] in ``out_dtype``."""
    T, wide = rows.shape
    n = weight.shape[0]
    _gpu(rows, "rows", torch.float32)
    _gpu(weight, "weight", torch.float32, (n,))
    _need(0 <= col and col + n <= wide, "the columns lie outside the rows")
    y = torch.empty(T, n, dtype=out_dtype, device=rows.device)
    src = ctypes.c_void_p(rows.data_ptr() + 4 * col)
    _check(stream_lib().ni_rmsnorm_cols(src, wide, _ptr(weight), _ptr(y), T, n, _float(eps), dtype_code(out_dtype), _stream()), "rmsnorm_cols")
    return y


def depth_mix(history: torch.Tensor, weights: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out[t] = sum_j weights[j] * history[j, t]``: a weighted sum of earlier states of the stream.  ``history``
    float32 [n, T, d] (contiguous), ``weights`` float32 [n], ``out`` float32 [T, d]."""
    n, T, d = history.shape
    _gpu(history, "history", torch.float32)
    _gpu(weights, "weights", torch.float32, (n,))
    _gpu(out, "out", torch.float32, (T, d))
    _check(stream_lib().ni_depth_mix(_ptr(history), _ptr(weights), _ptr(out), n, T, d, _stream()), "depth_mix")
    return out


def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """``a N(z) + b N(z^2) + c N(z^3) + e`` row by row, ``N(u) = u / sqrt(mean(u^2) + eps)``, powers element by element;
    ``z`` float32 [T, n], ``coef`` float32 [4] = (a, b, c, e); the result in ``out_dtype``."""
    T, n = z.shape
    _gpu(z, "z", torch.float32)
    _gpu(coef, "coef", torch.float32, (4,))
    y = torch.empty(T, n, dtype=out_dtype, device=z.device)
    _check(stream_lib().ni_poly_norm(_ptr(z), _ptr(coef), _ptr(y), T, n, _float(eps), dtype_code(out_dtype), _stream()), "poly_norm")
    return y


def scale_(x: torch.Tensor, factor: float) -> torch.Tensor:
    """``x *= factor`` in place (float32)."""
    _gpu(x, "x", torch.float32)
    _check(stream_lib().ni_scale(_ptr(x), _float(factor), _size_t(x.numel()), _stream()), "scale")
    return x


def gate_heads(o: torch.Tensor, gate_rows: torch.Tensor, gate_col: int, out_dtype: torch.dtype, per_head: bool = False) -> torch.Tensor:
    """``y[t, h * dv + c] = o[h, t, c] * sigmoid(gate[t, h * dv + c])``: ``o`` float32 [H, T, dv] (head by head), the
    gate's pre-activations the columns ``gate_col ..`` of ``gate_rows`` float32 [T, wide]; y [T, H * dv] in ``out_dtype``.
    ``per_head``: one gate a head, ``gate[t, h]``."""
    H, T, dv = o.shape
    per = dv if per_head else 1
    _gpu(o, "o", torch.float32)
    _gpu(gate_rows, "gate_rows", torch.float32)
    _need(gate_rows.shape[0] == T and 0 <= gate_col and gate_col + H * dv // per <= gate_rows.shape[1], "the gate's columns lie outside its rows")
    y = torch.empty(T, H * dv, dtype=out_dtype, device=o.device)
    gate = ctypes.c_void_p(gate_rows.data_ptr() + 4 * gate_col)
    _check(stream_lib().ni_gate_heads(_ptr(o), gate, gate_rows.shape[1], _ptr(y), T, H, dv, per, dtype_code(out_dtype), _stream()), "gate_heads")
    return y


def gate_rows(x: torch.Tensor, gate_rows_: torch.Tensor, gate_col: int, out: Optional[torch.Tensor] = None, every: int = 1) -> torch.Tensor:
    """``y[t, j] = x[t, j] * sigmoid(gate[t, j // every])``: ``x`` [T, n] in the compute type, the gate's pre-activations
    the columns ``gate_col ..`` of ``gate_rows_`` float32 [T, wide]; y like x.  ``every`` 1: a gate a channel; a head's
    channels: a gate a head."""
    T, n = x.shape
    _gpu(x, "x")
    _gpu(gate_rows_, "gate_rows", torch.float32)
    _need(every >= 1 and n % every == 0, "whole groups of channels share a gate")
    _need(gate_rows_.shape[0] == T and 0 <= gate_col and gate_col + n // every <= gate_rows_.shape[1], "the gate's columns lie outside its rows")
    y = torch.empty_like(x) if out is None else out
    gate = ctypes.c_void_p(gate_rows_.data_ptr() + 4 * gate_col)
    _check(stream_lib().ni_gate_rows(_ptr(x), gate, gate_rows_.shape[1], _ptr(y), T, n, int(every), dtype_code(x.dtype), _stream()), "gate_rows")
    return y


def gather_pages(pool: torch.Tensor, block_table: torch.Tensor, pairs: torch.Tensor) -> torch.Tensor:
    """Pages of ``pool`` [pages, ...] picked through ``block_table`` int32 [B, width]: ``pairs`` int32 [n, 2] rows of
    (sequence, index of the page in the sequence's table); [n, ...] like the pool's pages, zeros where the table holds
    no page."""
    _gpu(pool, "pool")
    _gpu(block_table, "block_table", torch.int32)
    _gpu(pairs, "pairs", torch.int32)
    _need(pairs.dim() == 2 and pairs.shape[1] == 2 and block_table.dim() == 2, "pairs are rows of (sequence, page index)")
    n = pairs.shape[0]
    out = torch.empty((n,) + tuple(pool.shape[1:]), dtype=pool.dtype, device=pool.device)
    page_elems = pool[0].numel()
    _check(stream_lib().ni_gather_pages(_ptr(pool), _ptr(block_table), block_table.shape[1], _ptr(pairs), _ptr(out), n, page_elems,
                                        dtype_code(pool.dtype), _stream()), "gather_pages")
    return out


def rows_to_pages(x: torch.Tensor, page: int, H: int, n: int) -> torch.Tensor:
    """``y[p, h, s, c] = x[p * page + s, h * n + c]``: rows [pages * page, H * n] of heads side by side as a pool of
    keys or values, [pages, H, page, n]."""
    rows, wide = x.shape
    _gpu(x, "x")
    _need(wide == H * n and rows % page == 0, "the rows are not whole pages of these heads")
    y = torch.empty(rows // page, H, page, n, dtype=x.dtype, device=x.device)
    _check(stream_lib().ni_rows_to_pages(_ptr(x), _ptr(y), rows // page, page, H, n, dtype_code(x.dtype), _stream()), "rows_to_pages")
    return y


def heads_apart(x: torch.Tensor, H: int, n: int) -> torch.Tensor:
    """``y[h, t, c] = x[t, h * n + c]`` for the first ``H * n`` columns of ``x`` [T, wide]: every head's rows together,
    as a product per head reads them."""
    T, wide = x.shape
    _gpu(x, "x")
    _need(H * n <= wide, "more heads than the rows hold")
    y = torch.empty(H, T, n, dtype=x.dtype, device=x.device)
    _check(stream_lib().ni_heads_apart(_ptr(x), wide, _ptr(y), T, H, n, dtype_code(x.dtype), _stream()), "heads_apart")
    return y


# ------------------------------------------------------------------ router and experts

ROUTE_SCORINGS = {"softmax_chosen": 0, "softmax_all": 1, "sigmoid": 2}


def route_top(z: torch.Tensor, top: int, mix_all: bool, over_all: bool = False, groups: int = 1, keep: int = 1,
              scoring: Optional[str] = None, correction: Optional[torch.Tensor] = None, group_top: int = 1, scale: float = 1.0):
    """The ``top`` experts of every row of ``z`` float32 [T, E] and their weights.  ``scoring``: "softmax_chosen" (an
    expert's value is its logit, the weights the softmax among the chosen; the default), "softmax_all" (``over_all``:
    the softmax over all E experts, not renormalised) or "sigmoid" (the value is ``sigmoid(logit)``, the weights the
    values themselves); every weight times ``scale``.  ``correction`` float32 [E] is added to the values that choose,
    never to the weights.  With ``groups`` > 1 the experts form that many equal groups of neighbours, a group counts as
    much as the sum of its ``group_top`` largest choosing values, and only experts of the ``keep`` best groups can be
    chosen.  ``(chosen int32 [T, top], mix float32 [T, top], mix over all experts float32 [T, E] or None)``."""
    T, E = z.shape
    _gpu(z, "z", torch.float32)
    if scoring is None:
        scoring = "softmax_all" if over_all else "softmax_chosen"
    _need(scoring in ROUTE_SCORINGS, f"scoring {scoring!r} is not one of {sorted(ROUTE_SCORINGS)}")
    _need(1 <= top <= E, f"{top} of {E} experts cannot be chosen")
    _need(1 <= groups <= 64 and E % groups == 0 and 1 <= keep <= groups and top <= E // groups * keep,
          f"{top} experts cannot be chosen from {keep} of {groups} groups of {E} experts")
    _need(group_top >= 1, "a group counts by at least one of its experts")
    if correction is not None:
        _gpu(correction, "correction", torch.float32, (E,))
    chosen = torch.empty(T, top, dtype=torch.int32, device=z.device)
    mix = torch.empty(T, top, dtype=torch.float32, device=z.device)
    dense = torch.empty(T, E, dtype=torch.float32, device=z.device) if mix_all else None
    _check(stream_lib().ni_route_top(_ptr(z), _ptr(correction), _ptr(chosen), _ptr(mix), _ptr(dense), T, E, top,
                                     ROUTE_SCORINGS[scoring], int(groups), int(keep), int(group_top), _float(scale), _stream()), "route_top")
    return chosen, mix, dense


EXPERT_FORMS = {"relu2": 0, "swiglu": 1, "capped_glu": 2}


def _expert_form(gated) -> int:
    """The number the kernels know an expert's activation by; ``gated`` may be a bool (relu2 / swiglu) or a name."""
    if isinstance(gated, str):
        _need(gated in EXPERT_FORMS, f"expert activation {gated!r} is not one of {sorted(EXPERT_FORMS)}")
        return EXPERT_FORMS[gated]
    return int(bool(gated))


def experts_act(up: torch.Tensor, mix_all: Optional[torch.Tensor], ff: int, gated=False, limit: float = 0.0,
                slope: float = 1.0) -> torch.Tensor:
    """``mix_all[t, e] * relu(up[t, e * ff + i])^2`` in the type of ``up``; ``gated`` (True or "swiglu"): an expert's
    columns of ``up`` are [gate: ff | up: ff] and the result is ``mix_all[t, e] * silu(gate) * up``, [T, E * ff];
    "capped_glu": ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``, ``mix * g * sigmoid(slope * g) * (u + 1)``.
    ``mix_all`` None (gated forms): every expert counts once."""
    T, width = up.shape
    form = _expert_form(gated)
    _gpu(up, "up")
    if mix_all is None:
        _need(form != 0 and width % (2 * ff) == 0, "without a mix the rows are whole gated experts")
        E = width // (2 * ff)
    else:
        E = mix_all.shape[1]
        _gpu(mix_all, "mix_all", torch.float32, (T, E))
    _need(width == E * ff * (2 if form else 1), "the experts' hidden rows do not match the router")
    act = torch.empty(T, E * ff, dtype=up.dtype, device=up.device)
    _check(stream_lib().ni_experts_act(_ptr(up), _ptr(mix_all), _ptr(act), T, E, ff, form, _float(limit), _float(slope),
                                       dtype_code(up.dtype), _stream()), "experts_act")
    return act


EXPERTS_FEW_ROWS = 16       # up to here only the chosen experts' matrices are read, row by row


def experts_few(x: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, chosen: torch.Tensor, mix: torch.Tensor,
                ff: int, gated=False, out: Optional[torch.Tensor] = None, limit: float = 0.0, slope: float = 1.0) -> torch.Tensor:
    """The weighted sum of the chosen experts for a few rows: ``w_up`` [E * ff, d] (``gated``: [E * 2 ff, d], an
    expert's gate rows and then its up rows; the hidden row is then ``silu(gate) * up`` instead of ``relu(up)^2``, or,
    "capped_glu", the capped form of :func:`experts_act`), ``w_down`` [d, E * ff]; returns float32 [T, d] (``out``, if given)."""
    T, d = x.shape
    top = chosen.shape[1]
    form = _expert_form(gated)
    per = ff * (2 if form else 1)
    E = w_up.shape[0] // per
    _gpu(x, "x", w_up.dtype)
    _gpu(w_up, "w_up", None, (E * per, d))
    _gpu(w_down, "w_down", w_up.dtype, (d, E * ff))
    _gpu(chosen, "chosen", torch.int32, (T, top))
    _gpu(mix, "mix", torch.float32, (T, top))
    hid = torch.empty(T * top, ff, dtype=torch.float32, device=x.device)
    if out is None:
        out = torch.empty(T, d, dtype=torch.float32, device=x.device)
    else:
        _gpu(out, "out", torch.float32, (T, d))
    _check(stream_lib().ni_experts_few(_ptr(x), _ptr(w_up), _ptr(w_down), _ptr(chosen), _ptr(mix), _ptr(hid), _ptr(out),
                                       T, d, ff, E, top, form, _float(limit), _float(slope), dtype_code(x.dtype), _stream()),
           "experts_few")
    return out


# ------------------------------------------------------------------ gated delta rule

DELTA_RUN_FROM = 16      # a step whose longest portion has this many tokens goes in runs of sixteen


def delta_rule(proj: torch.Tensor, low: torch.Tensor, conv: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
               norm_w: torch.Tensor, state: torch.Tensor, seq_of_token: torch.Tensor, q_start: torch.Tensor,
               q_len: torch.Tensor, state_slot: torch.Tensor, G: int, H: int, dk: int, dv: int, taps: int, eps: float,
               out_dtype: torch.dtype, max_q_len: int = 0, runs: Optional[bool] = None) -> torch.Tensor:
    """One step of the gated delta rule with a decay per key channel for all sequences of the step.

    ``proj`` float32 [T, >= C + H] holds q [G*dk] | k [G*dk] | v [H*dv] | b [H] as projected (C the first
    three); ``low`` float32 [T, H*dk + H*dv] the decay's and the output gate's pre-activations; ``conv``
    float32 [C, taps]; ``state`` float32 [slots, H*dv*dk + (taps-1)*C]: the memory of every head (stored
    [head, value channel, key channel]) and the convolutions' last inputs, both moved on by this call.
    Returns the normalised, gated read-out [T, H*dv] in ``out_dtype``.

    ``max_q_len`` is the longest portion of the step (a host number; 0: not known).  From ``DELTA_RUN_FROM``
    tokens on, and where the key size is a multiple of 16, the step goes sixteen tokens at a time on the matrix
    cores (in float32 as well); otherwise token by token (``runs`` = True / False asks for one of the two).
    Both compute the same recurrence and differ by rounding.  A step of single tokens (``max_q_len`` 1) moves
    the convolutions' inputs on in its first kernel."""
    T, proj_cols = proj.shape
    B = q_start.shape[0]
    C = 2 * G * dk + H * dv
    _gpu(proj, "proj", torch.float32)
    _need(proj_cols >= C + H, "proj is too narrow")
    _gpu(low, "low", torch.float32, (T, H * dk + H * dv))
    _gpu(conv, "conv", torch.float32, (C, taps))
    _gpu(a_log, "a_log", torch.float32, (H,))
    _gpu(dt_bias, "dt_bias", torch.float32, (H * dk,))
    _gpu(norm_w, "norm_w", torch.float32, (dv,))
    _need(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous(), "state must be float32 [slots, n] on the GPU")
    conv_off = H * dv * dk
    _need(state.shape[1] == conv_off + (taps - 1) * C, "state has the wrong size")
    _gpu(seq_of_token, "seq_of_token", torch.int32, (T,))
    for name, t in (("q_start", q_start), ("q_len", q_len), ("state_slot", state_slot)):
        _need(t.is_cuda and t.dtype == torch.int32 and t.shape == (B,), f"{name} must be int32 [{B}] on the GPU")
    _need(H % G == 0 and taps >= 1, "heads and taps")
    lib = delta_rule_lib(dk)
    prep = torch.empty(T, C + H + H * dk + H * dv, dtype=torch.float32, device=proj.device)
    stride = state.shape[1]
    _need(0 <= max_q_len <= T, "max_q_len is larger than the step")
    _need(max_q_len != 1 or T == B, "a step of single tokens has one row a sequence")
    in_runs = max_q_len >= DELTA_RUN_FROM if runs is None else bool(runs)
    run_floats = int(lib.ni_delta_run_floats()) if in_runs else 0
    _need(run_floats > 0 or not runs, f"the delta rule has no runs of sixteen for keys of {dk} channels")
    chunks = None
    if run_floats:
        max_q_len = max_q_len or T
        chunks = torch.empty((T // 16 + B + 1) * H * run_floats, dtype=torch.float32, device=proj.device)
    _check(lib.ni_delta_prepare(_ptr(proj), _ptr(low), _ptr(conv), _ptr(a_log), _ptr(dt_bias), _ptr(state), _ptr(seq_of_token),
                                _ptr(q_start), _ptr(q_len), _ptr(state_slot), _ptr(prep), T, B, G, H, dk, dv, taps, proj_cols,
                                _size_t(stride), _size_t(conv_off), int(chunks is not None), int(max_q_len), _stream()), "delta_prepare")
    o = torch.empty(T, H * dv, dtype=torch.float32, device=proj.device)
    y = torch.empty(T, H * dv, dtype=out_dtype, device=proj.device)
    _check(lib.ni_delta_rule(_ptr(prep), _ptr(chunks), _ptr(state), _ptr(q_start), _ptr(q_len), _ptr(state_slot), _ptr(o),
                             _ptr(norm_w), _ptr(y), T, B, int(max_q_len), G, H, dk, dv, _float(eps), _size_t(stride),
                             dtype_code(out_dtype), _stream()),
           "delta_rule")
    return y


# ------------------------------------------------------------------ attention with a bias by distance

RUN_KEYS = 128      # a run of keys is at least this long


def bias_attention_runs(n_tiles: int, kv_heads: int, head_chunks: int, max_keys: int, waves: int = 4) -> int:
    """Into how many runs the keys of a tile are cut: none while the tiles alone fill the chip's 256 compute
    units or the keys are few, else towards 2,048 wavefronts, a run being at least ``RUN_KEYS`` keys."""
    blocks = max(1, n_tiles * kv_heads * head_chunks)
    if blocks >= 256 or max_keys < 2 * RUN_KEYS:
        return 1
    # a step of very few rows (a single token of a model with few kv heads) takes runs of one tile of 64 keys: a run is
    # a chain of tiles, each a round trip to memory (a decode step at batch 1 over 1,028 keys 0.896 -> 0.877 ms; at
    # batch 8, where the chip is busier, the longer runs win, 1.337 : 1.358 ms)
    run_keys = min(RUN_KEYS, 64) if blocks * waves <= 16 else RUN_KEYS
    return max(1, min(64, 2048 // (blocks * waves), max_keys // run_keys))


def bias_attention_rows() -> int:
    """Rows of (token, head) that one workgroup of the kernel takes."""
    return 16


def kv_store(qkv: torch.Tensor, k_off: int, v_off: int, slot_mapping: torch.Tensor, kpool: torch.Tensor,
             vpool: torch.Tensor) -> None:
    """Keys (columns from ``k_off``) and values (from ``v_off``) of the rows of ``qkv`` into their page slots."""
    T, width = qkv.shape
    pages, G, ps, dk = kpool.shape
    dv = vpool.shape[3]
    _gpu(qkv, "qkv")
    _gpu(kpool, "kpool", qkv.dtype)
    _gpu(vpool, "vpool", qkv.dtype, (pages, G, ps, dv))
    _gpu(slot_mapping, "slot_mapping", torch.int32, (T,))
    _need(k_off + G * dk <= width and v_off + G * dv <= width, "keys or values lie outside the rows")
    _check(bias_attention_lib().ni_kv_store(_ptr(qkv), width, k_off, v_off, _ptr(slot_mapping), _ptr(kpool), _ptr(vpool),
                                            T, G, dk, dv, ps, dtype_code(qkv.dtype), _stream()), "kv_store")


def qk_norm_rope_store(proj: torch.Tensor, positions: torch.Tensor, slot_mapping: Optional[torch.Tensor],
                       q_norm: Optional[torch.Tensor], k_norm: Optional[torch.Tensor], eps: float, freq: Optional[torch.Tensor],
                       amplitude: float, q_out: Optional[torch.Tensor], kpool: Optional[torch.Tensor], vpool: Optional[torch.Tensor],
                       H: int, values_are_keys: bool = False, col: int = 0, per_head: bool = False, adjacent: bool = False,
                       q_dim: Optional[int] = None, rot_at_q: int = 0, rot_at_k: int = 0, k_normed: Optional[int] = None,
                       queries_only: bool = False) -> Optional[torch.Tensor]:
    """From ``proj`` float32 [T, H*dq + G*dk + G*dv] (q | k | v as projected): the RMS norm over a token's WHOLE
    query projection and over its whole key projection (weights ``q_norm`` [H*dq], ``k_norm`` [G*dk]; None: no norm),
    then the rotation of the first ``2 * len(freq)`` channels of every head, channel c with channel c + len(freq), by
    ``position * freq[c]`` with cos and sin times ``amplitude`` (``freq`` None: no rotation), all in float32.  Queries
    go to ``q_out`` [T, H*dq], keys and values into their page slots (``slot_mapping`` None: nothing is stored).
    ``values_are_keys``: ``proj`` is q | k alone and the keys as projected, before their norm, are stored as the values.
    ``H`` may be 0 (``q_out`` None): keys alone, and values may have no channels.  ``col``: the projections are the
    columns from ``col`` on of wider rows.

    ``per_head``: every head is normed on its own, with one weight shared by the heads (``q_norm`` [dq], ``k_norm``
    [k_normed]); of a key head only the first ``k_normed`` channels are normed then (default: all), the others pass as
    projected.  ``adjacent``: the rotation pairs channel 2p with channel 2p + 1.  ``rot_at_q``, ``rot_at_k``: the first
    rotated channel of a query head and of a key head.  ``q_dim``: a query head's size where it differs from a key
    head's.  ``queries_only``: ``proj`` holds the queries alone (the pools only say the sizes, or are None)."""
    T, wide = proj.shape
    if queries_only:
        G, dk, dv, ps = 0, 0, 0, 1
        _need(slot_mapping is None, "queries alone leave nothing to store")
    else:
        pages, G, ps, dk = kpool.shape
        dv = vpool.shape[3]
    dq = dk if q_dim is None else int(q_dim)
    _need(not queries_only or q_dim is not None, "queries alone need their head size")
    width = H * dq + G * dk + (0 if values_are_keys else G * dv)
    _need(0 <= col and col + width <= wide, "the projections lie outside the rows")
    _gpu(proj, "proj", torch.float32)
    _need(not values_are_keys or dv == dk, "values that are the keys have the keys' size")
    _gpu(positions, "positions", torch.int32, (T,))
    if slot_mapping is not None:
        _gpu(slot_mapping, "slot_mapping", torch.int32, (T,))
    normed = dk if k_normed is None else int(k_normed)
    _need(0 <= normed <= dk and (per_head or normed == dk), "only norms a head keep some of a key's channels out")
    if q_norm is not None:
        _gpu(q_norm, "q_norm", torch.float32, (dq,) if per_head else (H * dq,))
    if k_norm is not None:
        _gpu(k_norm, "k_norm", torch.float32, (normed,) if per_head else (G * dk,))
    rot = 0
    if freq is not None:
        rot = 2 * freq.shape[0]
        _gpu(freq, "freq", torch.float32, (rot // 2,))
        _need(rot > 0 and (H == 0 or rot_at_q + rot <= dq) and (G == 0 or rot_at_k + rot <= dk) and rot_at_q >= 0 and rot_at_k >= 0,
              f"{rot} rotated channels do not fit the heads")
    dtype = q_out.dtype if queries_only else kpool.dtype
    if not queries_only:
        _gpu(kpool, "kpool")
        _gpu(vpool, "vpool", kpool.dtype, (pages, G, ps, dv))
    if H > 0 or q_out is not None:
        _gpu(q_out, "q_out", dtype, (T, H * dq))
    src = ctypes.c_void_p(proj.data_ptr() + 4 * col)
    _check(bias_attention_lib().ni_qk_norm_rope_store(src, wide, _ptr(positions), _ptr(slot_mapping), _ptr(q_norm),
                                                      _ptr(k_norm), _float(eps), _ptr(freq), rot, _float(amplitude), _ptr(q_out),
                                                      _ptr(None if queries_only else kpool), _ptr(None if queries_only else vpool),
                                                      T, H, G, dq, dk, dv, ps, int(bool(values_are_keys)), int(bool(per_head)),
                                                      normed, int(rot_at_q), int(rot_at_k), int(bool(adjacent)),
                                                      dtype_code(dtype), _stream()), "qk_norm_rope_store")
    return q_out


def bias_attention(qkv: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_table: torch.Tensor,
                   tiles: torch.Tensor, positions: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, H: int, scale: float,
                   temp_coef: float, temp_every: int, heads_per_chunk: int, n_runs: int = 1,
                   workspace: Optional[torch.Tensor] = None, waves: int = 4, window: Optional[int] = None, keep_first: int = 0,
                   out_scale: float = 1.0, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of the query heads in the first ``H * dk`` columns of ``qkv`` over the paged cache.
    ``tiles`` int32 [n, 4]: (sequence, first row, tokens, -) with tokens * heads of a chunk <= 16, the tokens of a
    tile being consecutive ones of one sequence; ``positions`` int32 [T] the position of every row;
    ``bias`` float32 [distances, H] or None; ``out`` [T, H * dv].  With ``n_runs`` > 1 the keys of every tile are
    cut into that many runs, which meet in ``workspace`` (float32, at least T * H * n_runs * (dv + 2)) and are merged
    by a second kernel.  ``waves`` (1 to 4): wavefronts of a workgroup, four rows each; fewer than four only where no
    tile has more rows than they take.  ``window`` n: a query sees its last n keys (its own among them) and the first
    ``keep_first`` keys of its sequence; ``out_scale`` multiplies the output.  ``sink`` float32 [H]: one more term
    ``exp(sink[head])`` in every row's denominator, with no key and no value."""
    T, width = qkv.shape
    pages, G, ps, dk = kpool.shape
    dv = vpool.shape[3]
    _gpu(qkv, "qkv")
    _gpu(kpool, "kpool", qkv.dtype)
    _gpu(vpool, "vpool", qkv.dtype, (pages, G, ps, dv))
    _need(block_table.is_cuda and block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be int32 [B, pages] on the GPU")
    _need(tiles.is_cuda and tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous(),
          "tiles must be int32 [n, 4] on the GPU")
    _gpu(out, "out", qkv.dtype, (T, H * dv))
    _gpu(positions, "positions", torch.int32, (T,))
    _need(H % G == 0 and H * dk <= width, "heads")
    distances = 0
    if bias is not None:
        distances = bias.shape[0]
        _gpu(bias, "bias", torch.float32, (distances, H))
        _need(distances >= 1, "an empty bias table")
    _need(dv <= 256, "values of more than 256 channels are not compiled")
    _need(1 <= heads_per_chunk <= 16, "heads_per_chunk")
    _need(1 <= n_runs <= 64, "n_runs")
    _need(1 <= waves <= 4, "waves")
    if sink is not None:
        _gpu(sink, "sink", torch.float32, (H,))
    if n_runs > 1:
        _need(workspace is not None and workspace.is_cuda and workspace.dtype == torch.float32 and workspace.is_contiguous()
              and workspace.numel() >= T * H * n_runs * (dv + 2), "the runs need a float32 workspace of T * H * n_runs * (dv + 2)")
    err = bias_attention_lib().ni_bias_attention(_ptr(qkv), width, _ptr(kpool), _ptr(vpool), _ptr(block_table),
                                                 block_table.shape[1], _ptr(tiles), tiles.shape[0], _ptr(positions), _ptr(bias), distances,
                                                 _ptr(out), H, G, dk, dv, ps, _float(scale), _float(temp_coef), int(temp_every),
                                                 heads_per_chunk, n_runs, _ptr(workspace if n_runs > 1 else None), T, waves,
                                                 int(window or 0), int(keep_first), _float(out_scale), _ptr(sink),
                                                 dtype_code(qkv.dtype), _stream())
    if err == -2:
        raise KernelError(f"keys of {dk} and values of {dv} channels do not fit the kernel's staging memory")
    _check(err, "bias_attention")
    return out


BIAS_ATTENTION_MFMA_FROM = 8      # a step whose longest portion has this many tokens takes the matrix-core kernel


def bias_attention_mfma_rows(dk: int, dv: int, one_pool: bool = False) -> int:
    """Rows of (token, head) of a tile of the matrix-core kernel for prompt portions; 0 where it does not take
    these sizes (both multiples of 16, small enough for its staging memory).  ``one_pool``: keys and values are the
    same pool, which is staged once and so may be larger."""
    return int(bias_attention_lib().ni_bias_attention_mfma_rows(int(dk), int(dv), int(bool(one_pool))))


def bias_attention_mfma(qkv: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_table: torch.Tensor,
                        tiles: torch.Tensor, positions: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, H: int,
                        scale: float, temp_coef: float, temp_every: int, heads_per_chunk: int, window: Optional[int] = None,
                        keep_first: int = 0, out_scale: float = 1.0, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """:func:`bias_attention` for steps with portions of prompts: tiles of up to 64 rows (tokens * heads of a chunk),
    both products on the float32 matrix instructions, the same formula and the same 32-bit softmax; no runs."""
    T, width = qkv.shape
    pages, G, ps, dk = kpool.shape
    dv = vpool.shape[3]
    _gpu(qkv, "qkv")
    _gpu(kpool, "kpool", qkv.dtype)
    _gpu(vpool, "vpool", qkv.dtype, (pages, G, ps, dv))
    _need(block_table.is_cuda and block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be int32 [B, pages] on the GPU")
    _need(tiles.is_cuda and tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous(),
          "tiles must be int32 [n, 4] on the GPU")
    _gpu(out, "out", qkv.dtype, (T, H * dv))
    _gpu(positions, "positions", torch.int32, (T,))
    _need(H % G == 0 and H * dk <= width, "heads")
    _need(bias_attention_mfma_rows(dk, dv, kpool.data_ptr() == vpool.data_ptr()) > 0,
          f"keys of {dk} and values of {dv} channels are not taken by the matrix-core kernel")
    _need(1 <= heads_per_chunk <= 64, "heads_per_chunk")
    if sink is not None:
        _gpu(sink, "sink", torch.float32, (H,))
    distances = 0
    if bias is not None:
        distances = bias.shape[0]
        _gpu(bias, "bias", torch.float32, (distances, H))
        _need(distances >= 1, "an empty bias table")
    _check(bias_attention_lib().ni_bias_attention_mfma(_ptr(qkv), width, _ptr(kpool), _ptr(vpool), _ptr(block_table),
                                                       block_table.shape[1], _ptr(tiles), tiles.shape[0], _ptr(positions),
                                                       _ptr(bias), distances, _ptr(out), H, G, dk, dv, ps, _float(scale),
                                                       _float(temp_coef), int(temp_every), heads_per_chunk,
                                                       int(window or 0), int(keep_first), _float(out_scale), _ptr(sink),
                                                       dtype_code(qkv.dtype), _stream()), "bias_attention_mfma")
    return out
