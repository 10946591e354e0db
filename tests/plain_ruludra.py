"""A plain, slow implementation of the Ruludra design in float64 numpy: one function per mechanism, written
from the equations, sharing no code with the engine.  It runs one whole sequence at a time and keeps nothing
between calls; the tests compare the engine's logits, layer outputs and kernels with it.

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


def rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------ embedding

def pair_rows(tokens: List[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Row of the pair table for every token: a hash of (token before, token); the first token takes the row behind
    the buckets."""
    return [buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets for t, tok in enumerate(tokens)]


def sinusoid(positions: np.ndarray, d: int, base: float = 10000.0) -> np.ndarray:
    """[T, d]: column 2i is sin(p * base^(-2i/d)), column 2i + 1 the cosine of the same angle."""
    out = np.zeros((len(positions), d), dtype=F)
    for c in range(d):
        angle = positions.astype(F) * base ** (-(c - c % 2) / d)
        out[:, c] = np.sin(angle) if c % 2 == 0 else np.cos(angle)
    return out


def embed(tokens: List[int], cfg: dict, w: Dict[str, np.ndarray]) -> np.ndarray:
    x = w["embed"][tokens].astype(F)
    pair = (cfg.get("embedding") or {}).get("bigram")
    if pair is not None:
        x = x + w["bigram"][pair_rows(tokens, pair["buckets"], pair["mul_prev"], pair["mul_cur"])]
    return x + sinusoid(np.arange(len(tokens)), cfg["width"])


# ------------------------------------------------------------------ softmax over a window

def window_softmax(scores: np.ndarray, size: Optional[int]) -> np.ndarray:
    """scores [..., T, T] (query, key): softmax over the keys j with 0 <= i - j < size (None: every j <= i)."""
    T = scores.shape[-1]
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    seen = (j <= i) if size is None else ((j <= i) & (i - j < size))
    s = np.where(seen, scores, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=-1, keepdims=True)


def query_factor(positions: np.ndarray, temp: Optional[dict]) -> np.ndarray:
    """1 + coef * ln(floor((p + 1) / every) + 1) for every position (no entry: ones)."""
    if temp is None:
        return np.ones(len(positions), dtype=F)
    return 1.0 + temp["coef"] * np.log(np.floor((positions + 1) / temp["every"]) + 1.0)


def distance_penalty(T: int, r1: np.ndarray, r2: np.ndarray) -> np.ndarray:
    """[heads, T, T]: r1_h * ln(1 + r2_h * (i - j)) where j <= i (zero elsewhere)."""
    dist = np.maximum(np.arange(T)[:, None] - np.arange(T)[None, :], 0).astype(F)
    return r1[:, None, None] * np.log1p(r2[:, None, None] * dist[None])


# ------------------------------------------------------------------ mixer: attention whose values are its keys

def attention(h: np.ndarray, m: dict, w: Dict[str, np.ndarray], pre: str, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, G, dk = m["heads"], m["kv_heads"], m["dim"]
    q = h @ w[pre + "mix.q"].T
    k_raw = h @ w[pre + "mix.k"].T
    values = k_raw.reshape(T, G, dk)                                   # the keys as projected are the values
    q = rms(q, eps) * w[pre + "mix.q.norm"]                            # one norm over all heads' channels together
    k = (rms(k_raw, eps) * w[pre + "mix.k.norm"]).reshape(T, G, dk)
    q = q.reshape(T, H, dk) * query_factor(np.arange(T), m.get("q_temp"))[:, None, None]
    penalty = distance_penalty(T, w[pre + "mix.r1"].astype(F), w[pre + "mix.r2"].astype(F))
    size = (m.get("mask") or {}).get("size")
    out = np.zeros((T, H, dk), dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        p = window_softmax(q[:, hd] @ k[:, g].T * m["scale"] - penalty[hd], size)
        out[:, hd] = p @ values[:, g]
    return out.reshape(T, H * dk) @ w[pre + "mix.o"].T


# ------------------------------------------------------------------ mixer: attention over a shared low-rank latent

def latent_of(h: np.ndarray, w: Dict[str, np.ndarray], pre: str, eps: float) -> np.ndarray:
    """What a layer with a down-projection of its own keeps of every token: [T, kv_rank]."""
    return rms(h @ w[pre + "mix.dkv"].T, eps) * w[pre + "mix.dkv.norm"]


def latent_attention(h: np.ndarray, latent: np.ndarray, m: dict, w: Dict[str, np.ndarray], pre: str, eps: float) -> np.ndarray:
    """``latent``: this layer's own (``latent_of``), or the one of the layer that ``kv_from`` names."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    cq = rms(h @ w[pre + "mix.dq"].T, eps) * w[pre + "mix.dq.norm"]
    q = (cq @ w[pre + "mix.uq"].T).reshape(T, H, dk)
    k = (latent @ w[pre + "mix.uk"].T).reshape(T, H, dk)
    v = (latent @ w[pre + "mix.uv"].T).reshape(T, H, dv)
    size = (m.get("mask") or {}).get("size")
    out = np.zeros((T, H, dv), dtype=F)
    for hd in range(H):
        out[:, hd] = window_softmax(q[:, hd] @ k[:, hd].T * m["scale"], size) @ v[:, hd]
    gate = sigmoid(h @ w[pre + "mix.g"].T)
    return (out.reshape(T, H * dv) * gate) @ w[pre + "mix.o"].T


# ------------------------------------------------------------------ mixer: matrix memory with exponential gates

def capped(z, cap: float):
    return cap * np.tanh(z / cap)


def matrix_memory(h: np.ndarray, m: dict, w: Dict[str, np.ndarray], pre: str, eps: float, state=None):
    """Token by token.  ``state``: None (a new sequence) or (S [H, dk, dv], n [H, dk], m [H]) as an earlier call
    returned it.  Returns (output [T, d], state)."""
    T = h.shape[0]
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[pre + "mix.q"].T).reshape(T, H, dk) * dk ** -0.5
    k = (h @ w[pre + "mix.k"].T).reshape(T, H, dk)
    v = (h @ w[pre + "mix.v"].T).reshape(T, H, dv)
    log_in = capped(h @ w[pre + "mix.i"].T + w[pre + "mix.i.b"], cap)
    log_keep = log_sigmoid(capped(h @ w[pre + "mix.f"].T + w[pre + "mix.f.b"], cap))
    if state is None:
        S, n, run_max = np.zeros((H, dk, dv), dtype=F), np.zeros((H, dk), dtype=F), np.zeros(H, dtype=F)
    else:
        S, n, run_max = (np.array(a, dtype=F) for a in state)
    out = np.zeros((T, H, dv), dtype=F)
    for t in range(T):
        for hd in range(H):
            new_max = max(log_keep[t, hd] + run_max[hd], log_in[t, hd])
            keep = math.exp(log_keep[t, hd] + run_max[hd] - new_max)
            take = math.exp(log_in[t, hd] - new_max)
            S[hd] = keep * S[hd] + take * np.outer(k[t, hd], v[t, hd])
            n[hd] = keep * n[hd] + take * k[t, hd]
            run_max[hd] = new_max
            out[t, hd] = (S[hd].T @ q[t, hd]) / (max(abs(n[hd] @ q[t, hd]), math.exp(-new_max)) + 1e-6)
    y = rms(out, eps).reshape(T, H * dv) * w[pre + "mix.norm"] * sigmoid(h @ w[pre + "mix.g"].T)
    return y @ w[pre + "mix.o"].T, (S, n, run_max)


# ------------------------------------------------------------------ feed-forward

def poly_norm(z: np.ndarray, coef: np.ndarray, eps: float) -> np.ndarray:
    """a N(z) + b N(z^2) + c N(z^3) + e with N = division by the root mean square over the row."""
    a, b, c, e = (float(x) for x in coef)
    return a * rms(z, eps) + b * rms(z ** 2, eps) + c * rms(z ** 3, eps) + e


def feed_forward(h: np.ndarray, w: Dict[str, np.ndarray], pre: str, eps: float) -> np.ndarray:
    return poly_norm(h @ w[pre + "mlp.up"].T, w[pre + "mlp.act"], eps) @ w[pre + "mlp.down"].T


# ------------------------------------------------------------------ the model

def forward(cfg: dict, w: Dict[str, np.ndarray], tokens: List[int], layers_out: Optional[list] = None) -> np.ndarray:
    """Logits [T, vocab] of one whole sequence.  ``layers_out``, if a list, gets the stream as every layer hands it on."""
    eps = cfg["norm"]["eps"]
    w = {k: np.asarray(v, dtype=F) for k, v in w.items()}
    x = embed(tokens, cfg, w)
    results = [x]                                   # the embedding's output, then every layer's own result
    latents: Dict[int, np.ndarray] = {}
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        n = rms(x, eps) * w[pre + "norm1"]
        if layer["type"] == "attention":
            y = attention(n, m, w, pre, eps)
        elif layer["type"] == "latent_attention":
            if m.get("kv_from") is None:
                latents[i] = latent_of(n, w, pre, eps)
            y = latent_attention(n, latents[i if m.get("kv_from") is None else m["kv_from"]], m, w, pre, eps)
        elif layer["type"] == "mlstm":
            y, _ = matrix_memory(n, m, w, pre, eps)
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        x = x + rms(y, eps) * w[pre + "norm1b"]
        if layer.get("mlp") is not None:
            y = feed_forward(rms(x, eps) * w[pre + "norm2"], w, pre, eps)
            x = x + rms(y, eps) * w[pre + "norm2b"]
        results.append(x)
        x = sum(w[pre + "dwa"][j] * results[j] for j in range(len(results)))     # what the next layer reads
        if layers_out is not None:
            layers_out.append(x)
    x = rms(x, eps) * w["final.norm"]
    return x @ w["head"].T * cfg.get("logit_scale", 1.0)


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
