"""Typed configuration of the Ruludra family, read from the keys of its ``config.json``.

Every size and every constant that one model of the design may choose differently from another comes from the
file: ``layers`` lists the layers, each with its ``type`` (which mixer), the mixer's sizes and constants and its
feed-forward (``mlp``; null: the layer has none).  A key the file must give and does not is an error that names it;
an absent block (``embedding.bigram``, a mixer's ``q_temp`` or ``mask``, ``logit_scale``) switches its mechanism off.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .fusavik_config import BigramConfig, _need, _positive
from .model_config import ConfigError

LAYER_TYPES = ("attention", "latent_attention", "mlstm")


def _window(d: Dict[str, Any], where: str) -> Optional[int]:
    mask = d.get("mask")
    if mask is None:
        return None
    size = int(_need(mask, "size", where + ".mask"))
    if size < 1:
        raise ConfigError(f"{where}.mask.size must be at least 1")
    return size


def _with_window(d: Dict[str, Any], window: Optional[int]) -> Dict[str, Any]:
    if window is not None:
        d["mask"] = {"size": window}
    return d


@dataclass(frozen=True)
class KeyValueAttentionConfig:
    """Softmax attention with grouped heads whose values are its keys as projected (``vdim`` = ``dim``): a norm over
    the whole query and key projections, a query factor that grows with the position (``temp`` = (coef, every)), a
    penalty on the scores that grows with the logarithm of the distance, a window of ``window`` keys."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]
    temp: Optional[Tuple[float, int]]

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> "KeyValueAttentionConfig":
        temp = d.get("q_temp")
        if temp is not None:
            temp = (float(_need(temp, "coef", where + ".q_temp")), int(_need(temp, "every", where + ".q_temp")))
            _positive(temp[1], f"{where}.q_temp.every")
        out = KeyValueAttentionConfig(int(_need(d, "heads", where)), int(_need(d, "kv_heads", where)), int(_need(d, "dim", where)),
                                      int(d.get("vdim", d["dim"])), float(_need(d, "scale", where)), _window(d, where), temp)
        for name in ("heads", "kv_heads", "dim"):
            _positive(getattr(out, name), f"{where}.{name}")
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: {out.heads} heads do not divide into {out.kv_heads} kv heads")
        if out.vdim != out.dim:
            raise ConfigError(f"{where}: the values are the keys, so vdim {out.vdim} must equal dim {out.dim}")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.temp is not None:
            d["q_temp"] = {"coef": self.temp[0], "every": self.temp[1]}
        return _with_window(d, self.window)


@dataclass(frozen=True)
class LatentAttentionConfig:
    """Softmax attention whose keys and values of every head are projections of one latent of ``kv_rank`` numbers a
    token, the only thing cached; queries go through a latent of ``q_rank``.  ``kv_from``: the layer whose latents this
    one reads instead of making its own."""

    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: Optional[int]
    kv_from: Optional[int]

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> "LatentAttentionConfig":
        out = LatentAttentionConfig(int(_need(d, "heads", where)), int(_need(d, "dim", where)), int(_need(d, "vdim", where)),
                                    int(_need(d, "q_rank", where)), int(_need(d, "kv_rank", where)), float(_need(d, "scale", where)),
                                    _window(d, where), None if d.get("kv_from") is None else int(d["kv_from"]))
        for name in ("heads", "dim", "vdim", "q_rank", "kv_rank"):
            _positive(getattr(out, name), f"{where}.{name}")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "q_rank": self.q_rank, "kv_rank": self.kv_rank,
                             "scale": self.scale}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return _with_window(d, self.window)


@dataclass(frozen=True)
class MatrixMemoryConfig:
    """A matrix memory per head with exponential input and forget gates whose pre-activations are capped at
    ``gate_cap``."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> "MatrixMemoryConfig":
        out = MatrixMemoryConfig(int(_need(d, "heads", where)), int(_need(d, "dim", where)), int(_need(d, "vdim", where)),
                                 float(_need(d, "gate_cap", where)))
        for name in ("heads", "dim", "vdim", "gate_cap"):
            _positive(getattr(out, name), f"{where}.{name}")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


_MIXERS = {"attention": KeyValueAttentionConfig, "latent_attention": LatentAttentionConfig, "mlstm": MatrixMemoryConfig}


@dataclass(frozen=True)
class RuludraLayer:
    type: str
    mixer: Any
    ff: Optional[int]          # hidden size of the dense feed-forward; None: the layer has none


@dataclass(frozen=True)
class RuludraConfig:
    architecture: str
    vocab: int
    width: int
    bigram: Optional[BigramConfig]
    norm_eps: float
    logit_scale: float
    layers: Tuple[RuludraLayer, ...]
    torch_dtype: str = "bfloat16"

    @staticmethod
    def from_dict(d: Dict[str, Any]) -> "RuludraConfig":
        name = d.get("architecture") or (d.get("architectures") or [None])[0]
        if not name:
            raise ConfigError("config.json lacks 'architecture'")
        layers = []
        for i, entry in enumerate(_need(d, "layers", "")):
            where = f"layers[{i}]"
            kind = str(_need(entry, "type", where))
            if kind not in _MIXERS:
                raise ConfigError(f"{where}: layer type {kind!r} is not one of {LAYER_TYPES}")
            mixer = _MIXERS[kind].from_dict(_need(entry, "mixer", where), where + ".mixer")
            mlp, ff = entry.get("mlp"), None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}.mlp.kind {mlp.get('kind')!r} is not 'dense'")
                ff = _positive(int(_need(mlp, "ff", where + ".mlp")), f"{where}.mlp.ff")
            layers.append(RuludraLayer(kind, mixer, ff))
        if not layers:
            raise ConfigError("config.json lists no layers")
        for i, layer in enumerate(layers):
            src = getattr(layer.mixer, "kv_from", None)
            if src is None:
                continue
            where = f"layers[{i}].mixer.kv_from"
            if not 0 <= src < i or layers[src].type != "latent_attention" or layers[src].mixer.kv_from is not None:
                raise ConfigError(f"{where} = {src} does not name an earlier latent_attention layer with latents of its own")
            if layers[src].mixer.kv_rank != layer.mixer.kv_rank:
                raise ConfigError(f"{where}: layer {src} keeps latents of {layers[src].mixer.kv_rank}, this layer reads {layer.mixer.kv_rank}")
        bigram = (d.get("embedding") or {}).get("bigram")
        if bigram is not None:
            bigram = BigramConfig(int(_need(bigram, "buckets", "embedding.bigram")), int(_need(bigram, "mul_prev", "embedding.bigram")),
                                  int(_need(bigram, "mul_cur", "embedding.bigram")))
            _positive(bigram.buckets, "embedding.bigram.buckets")
        cfg = RuludraConfig(architecture=str(name), vocab=int(_need(d, "vocab", "")), width=int(_need(d, "width", "")), bigram=bigram,
                            norm_eps=float(_need(_need(d, "norm", ""), "eps", "norm")), logit_scale=float(d.get("logit_scale", 1.0)),
                            layers=tuple(layers), torch_dtype=str(d.get("torch_dtype", "bfloat16")))
        _positive(cfg.vocab, "vocab")
        _positive(cfg.width, "width")
        _positive(cfg.norm_eps, "norm.eps")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        emb: Dict[str, Any] = {}
        if self.bigram is not None:
            emb["bigram"] = {"buckets": self.bigram.buckets, "mul_prev": self.bigram.mul_prev, "mul_cur": self.bigram.mul_cur}
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "embedding": emb,
                "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale,
                "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.ff is None else {"kind": "dense", "ff": l.ff}}
                           for l in self.layers]}
