"""Typed configuration of the Vimilix family, read from the keys of its ``config.json``.

Every size and every constant that one model of the design may choose differently from another comes from the
file: ``layers`` lists the layers, each with its ``type`` (which mixer), the mixer's sizes and constants and its
feed-forward (``mlp``; null: the layer has none).  A key the file must give and does not is an error that names it;
an absent block (a mixer's ``mask``, a rotation's ``scaling``, a router's ``groups``, an ``mlp.shared``) switches its
mechanism off.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .fusavik_config import _need, _positive
from .model_config import ConfigError

LAYER_TYPES = ("attention", "latent_attention")


@dataclass(frozen=True)
class PairRotationConfig:
    """Rotation of ``dims`` channels of a head, channel 2i with channel 2i + 1, by ``position * base^(-2i / dims)``;
    ``scaling`` (factor, low, high, original) divides the frequencies of long waves by ``factor``, keeps short ones and
    blends between."""

    dims: int
    base: float
    scaling: Optional[Tuple[float, float, float, float]] = None      # (factor, low, high, original)

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str, dims: Optional[int] = None) -> "PairRotationConfig":
        sc = d.get("scaling")
        if sc is not None:
            sc = tuple(float(_need(sc, k, where + ".scaling")) for k in ("factor", "low", "high", "original"))
            if sc[2] == sc[1]:
                raise ConfigError(f"{where}.scaling: high and low must differ")
        out = PairRotationConfig(int(_need(d, "dims", where)) if dims is None else int(d.get("dims", dims)),
                                 float(_need(d, "base", where)), sc)
        if out.dims <= 0 or out.dims % 2:
            raise ConfigError(f"{where}.dims must be positive and even, got {out.dims}")
        if dims is not None and out.dims != dims:
            raise ConfigError(f"{where}.dims is {out.dims}, the rotated part of a head has {dims} channels")
        _positive(out.base, f"{where}.base")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            factor, low, high, original = self.scaling
            d["scaling"] = {"factor": factor, "high": high, "low": low,
                            "original": int(original) if float(original).is_integer() else original}
        return d


def _window(d: Dict[str, Any], where: str) -> Optional[int]:
    mask = d.get("mask")
    if mask is None:
        return None
    size = int(_need(mask, "size", where + ".mask"))
    if size < 1:
        raise ConfigError(f"{where}.mask.size must be at least 1")
    return size


@dataclass(frozen=True)
class SinkAttentionConfig:
    """Softmax attention with grouped heads in a window of ``window`` keys: a norm a head on queries and keys, a
    rotation of the first ``rot.dims`` channels, a sink in the denominator and a gate a head.  ``kv_from``: the layer
    whose keys and values this one reads instead of making its own."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]
    rot: PairRotationConfig
    kv_from: Optional[int]

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> "SinkAttentionConfig":
        out = SinkAttentionConfig(int(_need(d, "heads", where)), int(_need(d, "kv_heads", where)), int(_need(d, "dim", where)),
                                  int(_need(d, "vdim", where)), float(_need(d, "scale", where)), _window(d, where),
                                  PairRotationConfig.from_dict(_need(d, "rot", where), where + ".rot"),
                                  None if d.get("kv_from") is None else int(d["kv_from"]))
        for name in ("heads", "kv_heads", "dim", "vdim"):
            _positive(getattr(out, name), f"{where}.{name}")
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: {out.heads} heads do not divide into {out.kv_heads} kv heads")
        if out.rot.dims > out.dim:
            raise ConfigError(f"{where}.rot.dims {out.rot.dims} is more than a head's {out.dim} channels")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "rot": self.rot.to_dict(),
                             "scale": self.scale, "vdim": self.vdim}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d


@dataclass(frozen=True)
class RotaryLatentConfig:
    """Softmax attention whose keys and values of every head are projections of one latent of ``kv_rank`` numbers a
    token; beside it every token keeps ``rot_dim`` rotated key channels that all heads share.  A query head has ``dim``
    channels that meet the projected keys and ``rot_dim`` rotated ones."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: Optional[int]
    rot: PairRotationConfig

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> "RotaryLatentConfig":
        rot_dim = int(_need(d, "rot_dim", where))
        out = RotaryLatentConfig(int(_need(d, "heads", where)), int(_need(d, "dim", where)), rot_dim, int(_need(d, "vdim", where)),
                                 int(_need(d, "kv_rank", where)), float(_need(d, "scale", where)), _window(d, where),
                                 PairRotationConfig.from_dict(_need(d, "rot", where), where + ".rot", dims=rot_dim))
        for name in ("heads", "dim", "rot_dim", "vdim", "kv_rank"):
            _positive(getattr(out, name), f"{where}.{name}")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "rot": self.rot.to_dict(),
                             "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d


@dataclass(frozen=True)
class CappedExpertsConfig:
    """Routed experts chosen by ``sigmoid(logit) + correction`` within the best groups, weighed by ``sigmoid(logit) *
    scale``; an expert's hidden units are capped at ``limit``.  ``shared`` (ff, limit): one more expert every token uses."""

    experts: int
    top: int
    ff: int
    limit: float
    scale: float
    group_count: int
    group_keep: int
    shared: Optional[Tuple[int, float]]

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> "CappedExpertsConfig":
        kind = d.get("kind", "moe")
        if kind != "moe":
            raise ConfigError(f"{where}.kind {kind!r} is not 'moe'")
        router, expert = _need(d, "router", where), _need(d, "expert", where)
        groups = router.get("groups")
        count, keep = (1, 1) if groups is None else (int(_need(groups, "count", where + ".router.groups")),
                                                     int(_need(groups, "keep", where + ".router.groups")))
        shared = d.get("shared")
        if shared is not None:
            shared = (int(_need(shared, "ff", where + ".shared")), float(_need(shared, "limit", where + ".shared")))
            _positive(shared[0], f"{where}.shared.ff")
        out = CappedExpertsConfig(int(_need(router, "experts", where + ".router")), int(_need(router, "top", where + ".router")),
                                  int(_need(expert, "ff", where + ".expert")), float(_need(expert, "limit", where + ".expert")),
                                  float(router.get("scale", 1.0)), count, keep, shared)
        for name in ("experts", "top", "ff", "group_count", "group_keep"):
            _positive(getattr(out, name), f"{where}.{name}")
        if out.experts % out.group_count or out.group_keep > out.group_count:
            raise ConfigError(f"{where}: {out.experts} experts do not form {out.group_count} equal groups of which {out.group_keep} are kept")
        if out.top > out.experts // out.group_count * out.group_keep:
            raise ConfigError(f"{where}: {out.top} experts cannot be chosen from {out.group_keep} groups of {out.experts // out.group_count}")
        return out

    def to_dict(self) -> Dict[str, Any]:
        router: Dict[str, Any] = {"experts": self.experts, "scale": self.scale, "top": self.top}
        if (self.group_count, self.group_keep) != (1, 1):
            router["groups"] = {"count": self.group_count, "keep": self.group_keep}
        d: Dict[str, Any] = {"expert": {"ff": self.ff, "limit": self.limit}, "kind": "moe", "router": router}
        if self.shared is not None:
            d["shared"] = {"ff": self.shared[0], "limit": self.shared[1]}
        return d


_MIXERS = {"attention": SinkAttentionConfig, "latent_attention": RotaryLatentConfig}


@dataclass(frozen=True)
class VimilixLayer:
    type: str
    mixer: Any
    mlp: Optional[CappedExpertsConfig]


@dataclass(frozen=True)
class VimilixConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    postln_alpha: float
    layers: Tuple[VimilixLayer, ...]
    torch_dtype: str = "bfloat16"

    @staticmethod
    def from_dict(d: Dict[str, Any]) -> "VimilixConfig":
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
            mlp = entry.get("mlp")
            layers.append(VimilixLayer(kind, mixer, None if mlp is None else CappedExpertsConfig.from_dict(mlp, where + ".mlp")))
        if not layers:
            raise ConfigError("config.json lists no layers")
        for i, layer in enumerate(layers):
            src = getattr(layer.mixer, "kv_from", None)
            if src is None:
                continue
            where = f"layers[{i}].mixer.kv_from"
            if not 0 <= src < i or layers[src].type != "attention" or layers[src].mixer.kv_from is not None:
                raise ConfigError(f"{where} = {src} does not name an earlier attention layer with keys and values of its own")
            a, b = layers[src].mixer, layer.mixer
            if (a.kv_heads, a.dim, a.vdim, a.rot) != (b.kv_heads, b.dim, b.vdim, b.rot):
                raise ConfigError(f"{where}: layer {src} keeps {a.kv_heads} heads of {a.dim} + {a.vdim} channels rotated by {a.rot}, "
                                  f"this layer reads {b.kv_heads} of {b.dim} + {b.vdim} rotated by {b.rot}")
        cfg = VimilixConfig(architecture=str(name), vocab=int(_need(d, "vocab", "")), width=int(_need(d, "width", "")),
                            norm_eps=float(_need(_need(d, "norm", ""), "eps", "norm")),
                            postln_alpha=float(_need(d, "postln_alpha", "")), layers=tuple(layers),
                            torch_dtype=str(d.get("torch_dtype", "bfloat16")))
        _positive(cfg.vocab, "vocab")
        _positive(cfg.width, "width")
        _positive(cfg.norm_eps, "norm.eps")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "postln_alpha": self.postln_alpha,
                "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                           for l in self.layers]}
