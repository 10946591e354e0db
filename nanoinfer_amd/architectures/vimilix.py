"""``Vimilix``: its configuration keys, its model as a list of parts, its tensor names.

A decoder whose stream is normed behind every sum: ``x <- norm1(alpha x + mixer(x))``, then, where the layer has a
feed-forward, ``x <- norm2(alpha x + ff(x))``; the sublayers read the stream itself.  The embedding's row is normed
before the first layer.  A mixer is softmax attention in a window (grouped heads, a norm a head on queries and keys, a
rotation of neighbouring channel pairs stretched for long contexts, a sink in the softmax's denominator, a gate a head),
whose keys and values a later layer may read again (``kv_from``), or attention over a low-rank latent beside which
every token keeps a few rotated key channels that all heads share.  The feed-forward is a set of routed experts with
capped hidden units, chosen by ``sigmoid(logit) + correction`` within the groups whose two best scores sum highest and
weighed by ``sigmoid(logit) * scale``, plus one expert every token uses.
Tensor names: ``embed``, ``embed.norm``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
``final.norm``, ``head``.
"""
from __future__ import annotations

from typing import Optional

from ..config.spec import BlockSpec, LayerRun, ModelSpec, PartSpec
from ..config.vimilix_config import PairRotationConfig, RotaryLatentConfig, SinkAttentionConfig, VimilixConfig
from ..registry import Architecture, register_architecture
from ..weights.random_init import InitRule

POSITIONS = 1 << 24          # beyond it a float32 no longer holds every position
GLU_SLOPE = 1.702            # the slope inside the sigmoid of an expert's hidden units
GROUP_TOP = 2                # a group of experts counts as much as its two best scores together


def _position(rot: PairRotationConfig) -> PartSpec:
    scaling = None
    if rot.scaling is not None:
        factor, low, high, original = rot.scaling
        scaling = {"kind": "llama3", "factor": factor, "low_freq_factor": low, "high_freq_factor": high,
                   "original_max_position_embeddings": original}
    return PartSpec("rope", {"rotary_dim": rot.dims, "theta": rot.base, "max_positions": None, "scaling": scaling, "exact": True})


def _mixer(i: int, cfg: VimilixConfig, cache_window: Optional[int]) -> PartSpec:
    m = cfg.layers[i].mixer
    d, pre = cfg.width, f"l{i}.mix."
    if isinstance(m, SinkAttentionConfig):
        names = {k: pre + k for k in ("q", "sink", "g", "o")}
        names["q_norm"] = pre + "q.norm"
        if m.kv_from is None:
            names.update(k=pre + "k", v=pre + "v", k_norm=pre + "k.norm")
        return PartSpec("sink_attention",
                        {"hidden_size": d, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim, "value_dim": m.vdim,
                         "scale": m.scale, "window": m.window, "cache_window": cache_window, "eps": cfg.norm_eps,
                         "position": _position(m.rot), "adjacent_pairs": True, "shares_kv": m.kv_from is not None}, names)
    assert isinstance(m, RotaryLatentConfig)
    names = {k: pre + k for k in ("q", "dkv", "uk", "uv", "sink", "g", "o")}
    names["dkv_norm"] = pre + "dkv.norm"
    return PartSpec("latent_attention",
                    {"hidden_size": d, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "q_rank": None, "rank": m.kv_rank,
                     "rot_dim": m.rot_dim, "scale": m.scale, "window": m.window, "eps": cfg.norm_eps, "position": _position(m.rot),
                     "adjacent_pairs": True, "gate": "head"}, names)


def _feed_forward(i: int, cfg: VimilixConfig) -> Optional[PartSpec]:
    mlp = cfg.layers[i].mlp
    if mlp is None:
        return None
    d, pre = cfg.width, f"l{i}.mlp."
    names = {"router": pre + "router", "correction": pre + "correction"}
    for e in range(mlp.experts):
        names.update({f"gate{e}": f"{pre}e{e}.gate", f"up{e}": f"{pre}e{e}.up", f"down{e}": f"{pre}e{e}.down"})
    shared = None
    if mlp.shared is not None:
        shared = PartSpec("capped_glu", {"hidden_size": d, "intermediate_size": mlp.shared[0], "limit": mlp.shared[1], "slope": GLU_SLOPE},
                          {"gate": pre + "shared.gate", "up": pre + "shared.up", "down": pre + "shared.down"})
    return PartSpec("routed_experts", {"hidden_size": d, "expert_size": mlp.ff, "experts": mlp.experts, "top": mlp.top,
                                       "activation": "capped_glu", "limit": mlp.limit, "slope": GLU_SLOPE, "mix": "sigmoid",
                                       "mix_scale": mlp.scale, "groups": mlp.group_count, "keep": mlp.group_keep,
                                       "group_top": GROUP_TOP, "shared": shared}, names)


def build_spec(cfg: VimilixConfig) -> ModelSpec:
    d, L = cfg.width, len(cfg.layers)

    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": d, "eps": cfg.norm_eps}, {"weight": name})

    # the pages of an attention layer keep what the longest window among the layers that read them wants
    source = [getattr(l.mixer, "kv_from", None) for l in cfg.layers]
    reach = {}
    for i, layer in enumerate(cfg.layers):
        if isinstance(layer.mixer, SinkAttentionConfig):
            j = i if source[i] is None else source[i]
            w = layer.mixer.window
            reach[j] = None if (w is None or (j in reach and reach[j] is None)) else max(w, reach.get(j, 0))
    blocks, order = [], []
    for i, layer in enumerate(cfg.layers):
        j = i if source[i] is None else source[i]
        parts = {"mixer": _mixer(i, cfg, reach.get(j)), "mixer_norm": norm(f"l{i}.norm1")}
        ff = _feed_forward(i, cfg)
        if ff is not None:
            parts.update(ffn=ff, ffn_norm=norm(f"l{i}.norm2"))
        blocks.append(BlockSpec(kind="postnorm", parts=parts, params={"alpha": cfg.postln_alpha}))
        # a layer that reads another's keys and values runs on that layer's cache and writes nothing there
        order.append(LayerRun(block=i, cache=j, writes_cache=source[i] is None))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=d, max_positions=POSITIONS,
        embedding=PartSpec("scaled_table", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": 1.0, "max_positions": POSITIONS,
                                            "eps": cfg.norm_eps}, {"weight": "embed", "norm": "embed.norm"}),
        blocks=blocks, order=order, final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d}, {"weight": "head"}),
        ignorable_suffixes=(".norm2",),      # a layer without a feed-forward has no use for its second norm's weight
    )


VIMILIX = register_architecture(Architecture(
    name="Vimilix",
    config_from_dict=VimilixConfig.from_dict,
    build_spec=build_spec,
    init=InitRule(matrix_std=0.05, vector_mean=1.0, vector_std=0.05,
                  overrides=((".sink", 0.0, 1.0), (".correction", 0.0, 0.1), (".mlp.router", 0.0, 0.3), ("embed", 0.0, 0.5),
                             (".mix.g", 0.0, 0.1))),
))
