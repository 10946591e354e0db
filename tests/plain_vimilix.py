"""A plain, slow implementation of the Vimilix design in float64 numpy: one function per mechanism, written from
the equations, sharing no code with the engine.  It runs one whole sequence at a time and keeps nothing between
calls; the tests compare the engine's logits, layer outputs and kernels with it.

Notation: ``d`` width, ``T`` tokens of the sequence, weights as stored ([out, in], applied as ``W x``); ``w`` maps
tensor names to arrays, ``pre`` is a layer's prefix (``l3.``).
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional

import numpy as np

F = np.float64
GLU_SLOPE = 1.702          # the slope inside the experts' sigmoid


def rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


# ------------------------------------------------------------------ embedding

def embed(tokens: List[int], cfg: dict, w: Dict[str, np.ndarray]) -> np.ndarray:
    """The token's row, normed."""
    return rms(w["embed"][tokens].astype(F), cfg["norm"]["eps"]) * w["embed.norm"]


# ------------------------------------------------------------------ rotation

def rotation_frequencies(rot: dict) -> np.ndarray:
    """f_i = base^(-2i / dims) for the dims / 2 pairs, stretched where ``rot`` has a ``scaling``: waves shorter than
    original / high are kept, waves longer than original / low are divided by ``factor``, and between the two the
    frequency moves linearly (in original / wavelength) from the one to the other."""
    dims = rot["dims"]
    f = np.array([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    s = rot.get("scaling")
    if s is None:
        return f
    out = f.copy()
    for i, fi in enumerate(f):
        wave = 2.0 * math.pi / fi
        if wave < s["original"] / s["high"]:
            continue
        if wave > s["original"] / s["low"]:
            out[i] = fi / s["factor"]
        else:
            t = (s["original"] / wave - s["low"]) / (s["high"] - s["low"])
            out[i] = (1.0 - t) * fi / s["factor"] + t * fi
    return out


def rotate_pairs(x: np.ndarray, positions: np.ndarray, freqs: np.ndarray) -> np.ndarray:
    """x [T, ..., 2 n]: neighbours (2i, 2i + 1) are turned by the angle position * f_i."""
    out = np.array(x, dtype=F)
    angle = positions.astype(F)[:, None] * freqs[None, :]                  # [T, n]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (freqs.shape[0],)
    c, s = np.cos(angle).reshape(shape), np.sin(angle).reshape(shape)
    a, b = x[..., 0::2], x[..., 1::2]
    out[..., 0::2] = a * c - b * s
    out[..., 1::2] = b * c + a * s
    return out


# ------------------------------------------------------------------ softmax with a sink

def sink_softmax(scores: np.ndarray, sink: float, size: Optional[int]) -> np.ndarray:
    """scores [T, T] (query, key): weights over the keys j with 0 <= i - j < size (None: every j <= i) whose
    denominator also holds exp(sink), a term without a key: a row's weights sum to less than one."""
    T = scores.shape[-1]
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    seen = (j <= i) if size is None else ((j <= i) & (i - j < size))
    s = np.where(seen, scores, -np.inf)
    top = np.maximum(s.max(axis=-1, keepdims=True), sink)
    e = np.exp(s - top)
    return e / (e.sum(axis=-1, keepdims=True) + np.exp(sink - top))


# ------------------------------------------------------------------ mixer: attention in a window

def attention_keys_values(h: np.ndarray, m: dict, w: Dict[str, np.ndarray], pre: str, eps: float):
    """What an attention layer with projections of its own keeps of every token: keys after norm and rotation
    [T, G, dim] and values [T, G, vdim]."""
    T = h.shape[0]
    G, dk, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = rms((h @ w[pre + "mix.k"].T).reshape(T, G, dk), eps) * w[pre + "mix.k.norm"]
    n = m["rot"]["dims"]
    k[..., :n] = rotate_pairs(k[..., :n], np.arange(T), rotation_frequencies(m["rot"]))
    return k, (h @ w[pre + "mix.v"].T).reshape(T, G, dv)


def attention(h: np.ndarray, kv, m: dict, w: Dict[str, np.ndarray], pre: str, eps: float) -> np.ndarray:
    """``kv``: this layer's own keys and values (``attention_keys_values``), or those of the layer ``kv_from`` names."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    keys, values = kv
    q = rms((h @ w[pre + "mix.q"].T).reshape(T, H, dk), eps) * w[pre + "mix.q.norm"]
    n = m["rot"]["dims"]
    q[..., :n] = rotate_pairs(q[..., :n], np.arange(T), rotation_frequencies(m["rot"]))
    size = (m.get("mask") or {}).get("size")
    out = np.zeros((T, H, dv), dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        p = sink_softmax(q[:, hd] @ keys[:, g].T * m["scale"], float(w[pre + "mix.sink"][hd]), size)
        out[:, hd] = p @ values[:, g]
    out = out * sigmoid(h @ w[pre + "mix.g"].T)[:, :, None]                # one gate a head
    return out.reshape(T, H * dv) @ w[pre + "mix.o"].T


# ------------------------------------------------------------------ mixer: attention over a latent

def latent_attention(h: np.ndarray, m: dict, w: Dict[str, np.ndarray], pre: str, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, dk, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    freqs = rotation_frequencies(dict(m["rot"], dims=dr))
    q = (h @ w[pre + "mix.q"].T).reshape(T, H, dk + dr)
    q_plain, q_turned = q[..., :dk], rotate_pairs(q[..., dk:], np.arange(T), freqs)
    down = h @ w[pre + "mix.dkv"].T
    c = rms(down[:, :rank], eps) * w[pre + "mix.dkv.norm"]                 # the latent
    k_turned = rotate_pairs(down[:, rank:], np.arange(T), freqs)           # one for all heads
    k_plain = (c @ w[pre + "mix.uk"].T).reshape(T, H, dk)
    v = (c @ w[pre + "mix.uv"].T).reshape(T, H, dv)
    size = (m.get("mask") or {}).get("size")
    out = np.zeros((T, H, dv), dtype=F)
    for hd in range(H):
        scores = (q_plain[:, hd] @ k_plain[:, hd].T + q_turned[:, hd] @ k_turned.T) * m["scale"]
        out[:, hd] = sink_softmax(scores, float(w[pre + "mix.sink"][hd]), size) @ v[:, hd]
    out = out * sigmoid(h @ w[pre + "mix.g"].T)[:, :, None]
    return out.reshape(T, H * dv) @ w[pre + "mix.o"].T


# ------------------------------------------------------------------ feed-forward: routed experts

def expert(h: np.ndarray, w: Dict[str, np.ndarray], pre: str, limit: float) -> np.ndarray:
    """``pre``: the expert's prefix (``l0.mlp.e3.``)."""
    g = np.minimum(h @ w[pre + "gate"].T, limit)
    u = np.clip(h @ w[pre + "up"].T, -limit, limit)
    return (g * sigmoid(GLU_SLOPE * g) * (u + 1.0)) @ w[pre + "down"].T


def route(h: np.ndarray, mlp: dict, w: Dict[str, np.ndarray], pre: str, margins: Optional[np.ndarray] = None):
    """(chosen [T, top], weights [T, top]).  Experts are chosen by sigmoid(z) + correction, within the ``keep`` groups
    whose two best such scores sum highest; the weights are sigmoid(z) alone, times ``scale``.  ``margins`` [T], if
    given, is lowered to the smallest gap by which a token's choice was made here (between the last group kept and the
    first one left out, and between the last expert chosen and the first one left out): a choice made by less than
    rounding moves the scores may fall the other way in an implementation that rounds."""
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    s = sigmoid(h @ w[pre + "mlp.router"].T)
    choice = s + w[pre + "mlp.correction"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    per = E // groups["count"]
    chosen = np.zeros((h.shape[0], top), dtype=np.int64)
    for t in range(h.shape[0]):
        by_group = choice[t].reshape(groups["count"], per)
        group_score = np.sort(by_group, axis=1)[:, -2:].sum(axis=1)
        ranked = np.argsort(-group_score, kind="stable")
        kept = ranked[: groups["keep"]]
        allowed = np.full(E, -np.inf)
        for g in kept:
            allowed[g * per:(g + 1) * per] = choice[t, g * per:(g + 1) * per]
        order = np.argsort(-allowed, kind="stable")
        chosen[t] = order[:top]
        if margins is not None:
            if groups["keep"] < groups["count"]:
                margins[t] = min(margins[t], group_score[ranked[groups["keep"] - 1]] - group_score[ranked[groups["keep"]]])
            if top < E and np.isfinite(allowed[order[top]]):
                margins[t] = min(margins[t], allowed[order[top - 1]] - allowed[order[top]])
    return chosen, np.take_along_axis(s, chosen, axis=1) * r["scale"]


def feed_forward(h: np.ndarray, mlp: dict, w: Dict[str, np.ndarray], pre: str, margins: Optional[np.ndarray] = None) -> np.ndarray:
    chosen, weights = route(h, mlp, w, pre, margins)
    out = np.zeros((h.shape[0], w[pre + "mlp.e0.down"].shape[0]), dtype=F)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], weights[t]):
            out[t] += a * expert(h[t:t + 1], w, f"{pre}mlp.e{e}.", mlp["expert"]["limit"])[0]
    if mlp.get("shared") is not None:
        out = out + expert(h, w, pre + "mlp.shared.", mlp["shared"]["limit"])
    return out


# ------------------------------------------------------------------ the model

def forward(cfg: dict, w: Dict[str, np.ndarray], tokens: List[int], layers_out: Optional[list] = None,
            margins: Optional[np.ndarray] = None) -> np.ndarray:
    """Logits [T, vocab] of one whole sequence.  ``layers_out``, if a list, gets the stream behind every layer;
    ``margins`` [T] (start it at infinity) the smallest gap by which any router chose for each token (see ``route``)."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    w = {k: np.asarray(v, dtype=F) for k, v in w.items()}
    x = embed(tokens, cfg, w)
    kept: Dict[int, tuple] = {}
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = attention_keys_values(x, m, w, pre, eps)
            y = attention(x, kept[i if m.get("kv_from") is None else m["kv_from"]], m, w, pre, eps)
        elif layer["type"] == "latent_attention":
            y = latent_attention(x, m, w, pre, eps)
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        x = rms(alpha * x + y, eps) * w[pre + "norm1"]
        if layer.get("mlp") is not None:
            x = rms(alpha * x + feed_forward(x, layer["mlp"], w, pre, margins), eps) * w[pre + "norm2"]
        if layers_out is not None:
            layers_out.append(x)
    return (rms(x, eps) * w["final.norm"]) @ w["head"].T


def argmax(row: np.ndarray) -> int:
    return int(np.argmax(row))


# ------------------------------------------------------------------ reading a model folder

def read_safetensors(path: str) -> Dict[str, np.ndarray]:
    out = {}
    with open(path, "rb") as fh:
        (n,) = struct.unpack("<Q", fh.read(8))
        header = json.loads(fh.read(n))
        data = fh.read()
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        a, b = meta["data_offsets"]
        raw = data[a:b]
        if meta["dtype"] == "BF16":
            arr = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32)
        elif meta["dtype"] == "F32":
            arr = np.frombuffer(raw, dtype="<f4")
        elif meta["dtype"] == "I32":
            arr = np.frombuffer(raw, dtype="<i4")
        else:
            raise ValueError(f"{name}: stored type {meta['dtype']}")
        out[name] = arr.reshape(meta["shape"]).astype(F)
    return out


def read_model_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))
