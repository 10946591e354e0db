"""Python face of the kernels in ``csrc/state_mixers.hip``: linear attention with one decay a head, and the
selective scan with its short convolution.  Their memory of the past is a float32 row of the cache manager's
state slots.  Shapes, types and devices are checked here, on the host, before a kernel is launched.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..csrc import build as _build
from . import _check, _gpu, _load, _need, _ptr, _stream, dtype_code

_size_t = ctypes.c_size_t
_float = ctypes.c_float


def state_mixers_lib() -> ctypes.CDLL:
    return _load(_build.STATE_MIXERS)


def _per_seq(q_start, q_len, state_slot) -> int:
    B = q_start.shape[0]
    for name, t in (("q_start", q_start), ("q_len", q_len), ("state_slot", state_slot)):
        _need(t.is_cuda and t.dtype == torch.int32 and tuple(t.shape) == (B,), f"{name} must be int32 [{B}] on the GPU")
    return B


def _state(state: torch.Tensor) -> int:
    _need(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous(),
          "state must be float32 [slots, n] on the GPU")
    return state.shape[1]


def _pow2_parts(n: int, per: int) -> int:
    parts = 1
    while parts * per < n:
        parts *= 2
    return parts


def decay_state_floats(heads: int, dk: int, dv: int) -> int:
    """Floats of one request's state of :func:`decay_attention`: [heads][dv][dk rounded up to 8 * a power of two]."""
    parts = _pow2_parts(dk, 8)
    _need(parts <= 64, f"keys of {dk} channels are more than the kernel's 512")
    return heads * dv * parts * 8


def scan_state_floats(inner: int, n: int) -> int:
    """Floats of one request's recurrent state of :func:`selective_scan`: [inner][n rounded up to 4 * a power of two]."""
    parts = _pow2_parts(n, 4)
    _need(parts <= 64, f"{n} numbers a channel are more than the kernel's 256")
    return inner * parts * 4


STATE_RUNS_FROM = 64      # a step whose longest portion has this many tokens goes in runs of tokens, all runs at once


def run_tokens(T: int, columns: int) -> int:
    """Tokens of a run for a step of T tokens whose token-by-token kernel has ``columns`` workgroups a sequence: 64, or
    less (a power of two, at least 16) where runs of 64 would leave the launches under about 2,048 workgroups: a run is
    a chain of dependent steps, and only many runs at once hide their round trips to memory."""
    run = 64
    while run > 16 and (T // run) * max(columns, 1) < 2048:
        run //= 2
    return run


def _in_runs(max_q_len: int, T: int, runs) -> bool:
    _need(0 <= max_q_len <= T, "max_q_len is larger than the step")
    return max_q_len >= STATE_RUNS_FROM if runs is None else bool(runs)


def decay_in_runs(max_q_len: int, T: int) -> bool:
    """Whether :func:`decay_attention` and :func:`selective_scan` take a step of T tokens whose longest portion has
    ``max_q_len`` in runs."""
    return _in_runs(max_q_len, T, None)


def silu_rows(x: torch.Tensor, n: int) -> torch.Tensor:
    """``silu`` of the first ``n`` columns of every row of ``x`` float32 [T, >= n], as float32 [T, n]."""
    T, width = x.shape
    _gpu(x, "x", torch.float32)
    _need(0 < n <= width, "more columns than the rows have")
    out = torch.empty(T, n, dtype=torch.float32, device=x.device)
    _check(state_mixers_lib().ni_silu_rows(_ptr(x), width, _ptr(out), T, n, _stream()), "silu_rows")
    return out


def decay_attention(act: torch.Tensor, decay: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor,
                    state_slot: torch.Tensor, H: int, dk: int, dv: int, max_q_len: int = 0, runs=None, raw: bool = False,
                    run_len: Optional[int] = None) -> torch.Tensor:
    """Per head ``S <- decay[h] S + k v^T; o = S^T q`` over the rows of every sequence of the step, in order.
    ``act`` float32 [T, 2 H dk + H dv]: q | k | v after their activation; ``state`` float32 [slots, >=
    decay_state_floats(H, dk, dv)], moved on by this call.  Returns ``o`` float32 [T, H dv].

    ``max_q_len`` is the longest portion of the step (a host number; 0: not known).  From ``STATE_RUNS_FROM`` tokens on
    the portions go in runs of :func:`run_tokens` tokens (``run_len``: of that many) that are worked out side by side
    and then chained (``runs`` = True / False asks for one of the two ways); otherwise token by token.  Both compute the same recurrence and differ by rounding.
    ``raw`` (token by token only, see :func:`decay_in_runs`): ``act`` holds the projections themselves, possibly as the
    first columns of wider rows, and silu is applied as they are read."""
    T, width = act.shape
    _gpu(act, "act", torch.float32)
    _need(width >= 2 * H * dk + H * dv if raw else width == 2 * H * dk + H * dv, "act is not q | k | v of these sizes")
    _need(not (raw and _in_runs(max_q_len, T, runs)), "the runs take their operands with silu applied")
    _gpu(decay, "decay", torch.float32, (H,))
    stride = _state(state)
    _need(stride >= decay_state_floats(H, dk, dv), "the state is too small")
    B = _per_seq(q_start, q_len, state_slot)
    out = torch.empty(T, H * dv, dtype=torch.float32, device=act.device)
    lib = state_mixers_lib()
    scratch, run = None, 0
    if _in_runs(max_q_len, T, runs):
        max_q_len = max_q_len or T
        parts = _pow2_parts(dk, 8)
        run = run_tokens(T, H * -(-dv // (4 * (64 // parts)))) if run_len is None else int(run_len)
        scratch = torch.empty((T // run + B) * decay_state_floats(H, dk, dv), dtype=torch.float32, device=act.device)
    _check(lib.ni_decay_attention(_ptr(act), width, _ptr(decay), _ptr(state), _size_t(stride), _ptr(q_start), _ptr(q_len),
                                  _ptr(state_slot), _ptr(out), T, B, H, dk, dv, int(max_q_len), _ptr(scratch), run, int(bool(raw)), _stream()),
           "decay_attention")
    return out


def gated_rmsnorm(o: torch.Tensor, gate_rows: torch.Tensor, gate_col: int, weight: torch.Tensor, eps: float, out_scale: float,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """``o / sqrt(mean(o^2) + eps) * weight * sigmoid(gate) * out_scale`` row by row; the gate's pre-activations are
    the columns ``gate_col ..`` of ``gate_rows`` float32 [T, wide]."""
    T, n = o.shape
    _gpu(o, "o", torch.float32)
    _gpu(gate_rows, "gate_rows", torch.float32)
    _need(gate_rows.shape[0] == T and 0 <= gate_col and gate_col + n <= gate_rows.shape[1], "the gate's columns lie outside its rows")
    _gpu(weight, "weight", torch.float32, (n,))
    y = torch.empty(T, n, dtype=out_dtype, device=o.device)
    gate = ctypes.c_void_p(gate_rows.data_ptr() + 4 * gate_col)
    _check(state_mixers_lib().ni_gated_rmsnorm(_ptr(o), gate, gate_rows.shape[1], _ptr(weight), _ptr(y), T, n, _float(eps),
                                               _float(out_scale), dtype_code(out_dtype), _stream()), "gated_rmsnorm")
    return y


def conv_silu(xz: torch.Tensor, inner: int, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, tail_off: int,
              seq_of_token: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, state_slot: torch.Tensor,
              out_dtype: torch.dtype, max_q_len: int = 0):
    """``u[t, c] = silu(bias[c] + sum_j weight[c, j] * x[t - (taps - 1 - j), c])`` over the first ``inner`` columns of
    ``xz`` float32 [T, wide], the inputs before a portion's first row taken from the state's tail (per slot, from
    float ``tail_off`` on: [(taps - 1)][inner], the oldest first), which this call moves on.  Returns ``(u as
    float32, u in out_dtype)`` (the same tensor when ``out_dtype`` is float32).  ``max_q_len`` 1 (a step of single
    tokens, one row a sequence) moves the tail on in the same kernel."""
    T, wide = xz.shape
    _gpu(xz, "xz", torch.float32)
    taps = weight.shape[1]
    _gpu(weight, "weight", torch.float32, (inner, taps))
    if bias is not None:
        _gpu(bias, "bias", torch.float32, (inner,))
    _need(inner <= wide, "more channels than the rows have")
    stride = _state(state)
    _need(stride >= tail_off + (taps - 1) * inner, "the state is too small")
    _gpu(seq_of_token, "seq_of_token", torch.int32, (T,))
    B = _per_seq(q_start, q_len, state_slot)
    u32 = torch.empty(T, inner, dtype=torch.float32, device=xz.device)
    uc = None if out_dtype == torch.float32 else torch.empty(T, inner, dtype=out_dtype, device=xz.device)
    _check(state_mixers_lib().ni_conv_silu(_ptr(xz), wide, _ptr(weight), _ptr(bias), _ptr(state), _size_t(stride), _size_t(tail_off),
                                           _ptr(seq_of_token), _ptr(q_start), _ptr(q_len), _ptr(state_slot), _ptr(u32), _ptr(uc),
                                           T, B, inner, taps, int(max_q_len == 1 and T == B), dtype_code(out_dtype), _stream()),
           "conv_silu")
    return u32, (u32 if uc is None else uc)


def selective_scan(dt_pre: torch.Tensor, dt_bias: torch.Tensor, u: torch.Tensor, xz: torch.Tensor, z_col: int, bc: torch.Tensor,
                   A: torch.Tensor, D: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor,
                   state_slot: torch.Tensor, N: int, out_dtype: torch.dtype, max_q_len: int = 0, runs=None,
                   run_len: Optional[int] = None) -> torch.Tensor:
    """``dt = softplus(dt_pre + dt_bias); S <- exp(dt A) S + dt u B; y = (S . C + D u) * silu(z)`` over the rows of
    every sequence of the step, in order.  ``dt_pre``, ``u`` float32 [T, inner]; ``z``: the columns ``z_col ..`` of
    ``xz`` float32 [T, wide]; ``bc`` float32 [T, 2 N]: B | C; ``A`` float32 [inner, n padded] as
    :func:`scan_state_floats` lays a channel out (negative, padding zero); ``state`` float32 [slots, >=
    scan_state_floats(inner, N)], moved on.  Returns y [T, inner] in ``out_dtype``.  ``max_q_len`` and ``runs`` as for
    :func:`decay_attention`."""
    T, inner = u.shape
    _gpu(u, "u", torch.float32)
    _gpu(dt_pre, "dt_pre", torch.float32, (T, inner))
    _gpu(dt_bias, "dt_bias", torch.float32, (inner,))
    _gpu(D, "D", torch.float32, (inner,))
    _gpu(xz, "xz", torch.float32)
    _need(xz.shape[0] == T and 0 <= z_col and z_col + inner <= xz.shape[1], "the gate's columns lie outside its rows")
    _gpu(bc, "bc", torch.float32, (T, 2 * N))
    floats = scan_state_floats(inner, N)
    _gpu(A, "A", torch.float32, (inner, floats // inner))
    stride = _state(state)
    _need(stride >= floats, "the state is too small")
    B = _per_seq(q_start, q_len, state_slot)
    y = torch.empty(T, inner, dtype=out_dtype, device=u.device)
    z = ctypes.c_void_p(xz.data_ptr() + 4 * z_col)
    lib = state_mixers_lib()
    scratch = y_local = dt_sum = None
    run = 0
    if _in_runs(max_q_len, T, runs):
        max_q_len = max_q_len or T
        run = run_tokens(T, -(-floats // 4 // 256)) if run_len is None else int(run_len)
        scratch = torch.empty((T // run + B) * floats, dtype=torch.float32, device=u.device)
        y_local = torch.empty(2, T, inner, dtype=torch.float32, device=u.device)
        y_local, dt_sum = y_local[0], y_local[1]
    _check(lib.ni_selective_scan(_ptr(dt_pre), _ptr(dt_bias), _ptr(u), z, xz.shape[1], _ptr(bc), 2 * N, _ptr(A), _ptr(D), _ptr(state),
                                 _size_t(stride), _ptr(q_start), _ptr(q_len), _ptr(state_slot), _ptr(y), T, B, inner, N, int(max_q_len),
                                 _ptr(scratch), _ptr(y_local), _ptr(dt_sum), run, dtype_code(out_dtype), _stream()), "selective_scan")
    return y


def memory_state_floats(heads: int, dk: int, dv: int) -> int:
    """Floats of one request's state of :func:`gated_memory`: [heads][dv + 1][dk rounded up to 8 * a power of two] (the
    normaliser is one more value channel), then the running maximum of every head; rounded up to whole 16 bytes."""
    parts = _pow2_parts(dk, 8)
    _need(parts <= 64, f"keys of {dk} channels are more than the kernel's 512")
    return (heads * (dv + 1) * parts * 8 + heads + 3) // 4 * 4


def gated_memory(proj: torch.Tensor, q_col: int, k_col: int, v_col: int, z_col: int, gate_bias: torch.Tensor, cap: float,
                 q_scale: float, state: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, state_slot: torch.Tensor,
                 H: int, dk: int, dv: int, max_q_len: int = 0, runs=None, run_len: Optional[int] = None):
    """A matrix memory per head with exponential gates, over the rows of every sequence of the step, in order:

        ``li = cap tanh((zi + bi) / cap);  lf = logsigmoid(cap tanh((zf + bf) / cap));  m' = max(lf + m, li)``
        ``S <- exp(lf + m - m') S + exp(li - m') k v^T;  n <- exp(lf + m - m') n + exp(li - m') k;  m <- m'``

    ``proj`` float32 [T, wide] holds q and k [H dk each] from columns ``q_col`` and ``k_col``, v [H dv] from ``v_col``
    and the gates' pre-activations zi [H] | zf [H] from ``z_col``; ``gate_bias`` float32 [2 H] = bi | bf; q is
    multiplied by ``q_scale``.  ``state`` float32 [slots, >= memory_state_floats(H, dk, dv)] holds S, n and (kept by
    :func:`memory_norm`) m; S and n are moved on by this call.  Returns ``(raw float32 [T, H, dv + 1], m float32 [T, H])``:
    ``S^T q`` and, as the last number of a head, ``n . q``, and every token's m.  ``max_q_len``, ``runs`` and ``run_len``
    as for :func:`decay_attention`: long portions go in runs side by side from an empty memory, chained afterwards."""
    T, wide = proj.shape
    _gpu(proj, "proj", torch.float32)
    for col, n in ((q_col, H * dk), (k_col, H * dk), (v_col, H * dv), (z_col, 2 * H)):
        _need(0 <= col and col + n <= wide, "the operands' columns lie outside the rows")
    _gpu(gate_bias, "gate_bias", torch.float32, (2 * H,))
    _need(cap > 0, "the gates' cap must be positive")
    stride = _state(state)
    floats = memory_state_floats(H, dk, dv)
    _need(stride >= floats, "the state is too small")
    B = _per_seq(q_start, q_len, state_slot)
    raw = torch.empty(T, H, dv + 1, dtype=torch.float32, device=proj.device)
    m = torch.empty(T, H, dtype=torch.float32, device=proj.device)
    scratch = scalars = None
    run = 0
    if _in_runs(max_q_len, T, runs):
        max_q_len = max_q_len or T
        parts = _pow2_parts(dk, 8)
        run = run_tokens(T, H * -(-(dv + 1) // (4 * (64 // parts)))) if run_len is None else int(run_len)
        n_runs = T // run + B
        scratch = torch.empty(n_runs * H * (dv + 1) * parts * 8, dtype=torch.float32, device=proj.device)
        scalars = torch.empty(2 * T * H + 3 * n_runs * H, dtype=torch.float32, device=proj.device)
    _check(state_mixers_lib().ni_gated_memory(_ptr(proj), wide, int(q_col), int(k_col), int(v_col), int(z_col), _ptr(gate_bias),
                                              _float(cap), _float(q_scale), _ptr(state), _size_t(stride), _ptr(q_start), _ptr(q_len),
                                              _ptr(state_slot), _ptr(raw), _ptr(m), T, B, H, dk, dv, int(max_q_len), _ptr(scratch),
                                              _ptr(scalars), run, _stream()), "gated_memory")
    return raw, m


def memory_norm(raw: torch.Tensor, m: torch.Tensor, gate_rows: torch.Tensor, gate_col: int, weight: torch.Tensor, eps: float,
                state: torch.Tensor, seq_of_token: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor,
                state_slot: torch.Tensor, dk: int, out_dtype: torch.dtype) -> torch.Tensor:
    """What :func:`gated_memory` left, finished: ``o = raw[..., :dv] / (max(|raw[..., dv]|, exp(-m)) + 1e-6)``, every head
    divided by its root mean square (``eps``), times ``weight`` [H dv], times ``sigmoid`` of the gate's pre-activations
    (columns ``gate_col ..`` of ``gate_rows`` float32 [T, wide]); [T, H dv] in ``out_dtype``.  The m of every sequence's
    last token is kept in ``state`` for the next step."""
    T, H, dvn = raw.shape
    dv = dvn - 1
    _gpu(raw, "raw", torch.float32)
    _gpu(m, "m", torch.float32, (T, H))
    _gpu(gate_rows, "gate_rows", torch.float32)
    _need(gate_rows.shape[0] == T and 0 <= gate_col and gate_col + H * dv <= gate_rows.shape[1], "the gate's columns lie outside its rows")
    _gpu(weight, "weight", torch.float32, (H * dv,))
    stride = _state(state)
    floats = memory_state_floats(H, dk, dv)
    _need(stride >= floats, "the state is too small")
    m_off = H * dvn * _pow2_parts(dk, 8) * 8
    _gpu(seq_of_token, "seq_of_token", torch.int32, (T,))
    _per_seq(q_start, q_len, state_slot)
    y = torch.empty(T, H * dv, dtype=out_dtype, device=raw.device)
    gate = ctypes.c_void_p(gate_rows.data_ptr() + 4 * gate_col)
    _check(state_mixers_lib().ni_memory_norm(_ptr(raw), _ptr(m), gate, gate_rows.shape[1], _ptr(weight), _ptr(y), _ptr(state),
                                             _size_t(stride), _size_t(m_off), _ptr(seq_of_token), _ptr(q_start), _ptr(q_len),
                                             _ptr(state_slot), T, H, dv, _float(eps), dtype_code(out_dtype), _stream()), "memory_norm")
    return y
