"""``Ruludra``: its configuration keys, its model as a list of parts, its tensor names.

A decoder of layers with a norm before and behind each sublayer, ``x += norm1b(mixer(norm1(x)))`` and, where the
layer has one, ``x += norm2b(ff(norm2(x)))``, over a float32 stream.  Behind every layer the stream that goes on is a
weighted sum of the embedding's output and of all layers' results so far (``l<i>.dwa``).  A mixer is softmax attention
in a window whose values are its keys (norms over the whole query and key projections, a query factor that grows with
the position, a penalty by the logarithm of the distance), attention over a low-rank latent that a later layer may
read again (``kv_from``), or a matrix memory with exponential gates.  The feed-forward is dense with a polynomial of
normed powers as activation.  The embedding adds a row of a second table read by a hash of the pair (token before,
token) and a sinusoid of the position; the logits are scaled by ``logit_scale``.
Tensor names: ``embed``, ``bigram``, ``l<i>.norm1``, ``l<i>.norm1b``, ``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``l<i>.dwa``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.ruludra_config import KeyValueAttentionConfig, LatentAttentionConfig, MatrixMemoryConfig, RuludraConfig
from ..config.spec import BlockSpec, LayerRun, ModelSpec, PartSpec
from ..registry import Architecture, register_architecture
from ..weights.random_init import InitRule

POSITIONS = 1 << 24          # beyond it a float32 no longer holds every position
UNBOUNDED_DISTANCES = 1 << 16  # rows of the distance penalty's table of an attention without a window
SINUSOID_BASE = 10000.0


def _mixer(i: int, cfg: RuludraConfig) -> PartSpec:
    m = cfg.layers[i].mixer
    d, pre = cfg.width, f"l{i}.mix."
    if isinstance(m, KeyValueAttentionConfig):
        names = {k: pre + k for k in ("q", "k", "o", "r1", "r2")}
        names.update(q_norm=pre + "q.norm", k_norm=pre + "k.norm")
        return PartSpec("keyed_attention",
                        {"hidden_size": d, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim, "scale": m.scale,
                         "window": m.window, "eps": cfg.norm_eps, "temp_coef": None if m.temp is None else m.temp[0],
                         "temp_every": None if m.temp is None else m.temp[1], "penalty": True,
                         "max_positions": UNBOUNDED_DISTANCES}, names)
    if isinstance(m, LatentAttentionConfig):
        names = {k: pre + k for k in ("dq", "uq", "uk", "uv", "g", "o")}
        names["dq_norm"] = pre + "dq.norm"
        if m.kv_from is None:
            names.update(dkv=pre + "dkv", dkv_norm=pre + "dkv.norm")
        return PartSpec("latent_attention",
                        {"hidden_size": d, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "q_rank": m.q_rank,
                         "rank": m.kv_rank, "scale": m.scale, "window": m.window, "eps": cfg.norm_eps}, names)
    assert isinstance(m, MatrixMemoryConfig)
    names = {k: pre + k for k in ("q", "k", "v", "g", "i", "f", "norm", "o")}
    names.update(i_b=pre + "i.b", f_b=pre + "f.b")
    return PartSpec("gated_memory", {"hidden_size": d, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim,
                                     "gate_cap": m.gate_cap, "eps": cfg.norm_eps}, names)


def build_spec(cfg: RuludraConfig) -> ModelSpec:
    d, L = cfg.width, len(cfg.layers)

    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": d, "eps": cfg.norm_eps}, {"weight": name})

    blocks, order, bounded = [], [], True
    for i, layer in enumerate(cfg.layers):
        parts = {"mixer_norm": norm(f"l{i}.norm1"), "mixer": _mixer(i, cfg), "mixer_post": norm(f"l{i}.norm1b")}
        if layer.ff is not None:
            pre = f"l{i}.mlp."
            parts.update(ffn_norm=norm(f"l{i}.norm2"), ffn_post=norm(f"l{i}.norm2b"),
                         ffn=PartSpec("poly_norm_mlp", {"hidden_size": d, "intermediate_size": layer.ff, "eps": cfg.norm_eps},
                                      {"up": pre + "up", "down": pre + "down", "act": pre + "act"}))
        blocks.append(BlockSpec(kind="sandwich", parts=parts))
        # a layer that reads another's latents runs on that layer's cache and writes nothing there
        source = getattr(layer.mixer, "kv_from", None)
        order.append(LayerRun(block=i, cache=i if source is None else source, writes_cache=source is None))
        if isinstance(layer.mixer, KeyValueAttentionConfig) and layer.mixer.window is None:
            bounded = False
    if cfg.bigram is not None:
        embedding = PartSpec("pair_hash_table", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": 1.0, "buckets": cfg.bigram.buckets,
                                                 "mul_prev": cfg.bigram.mul_prev, "mul_cur": cfg.bigram.mul_cur,
                                                 "sinusoid_base": SINUSOID_BASE}, {"weight": "embed", "pairs": "bigram"})
    else:
        embedding = PartSpec("pair_hash_table", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": 1.0, "buckets": None,
                                                 "sinusoid_base": SINUSOID_BASE}, {"weight": "embed"})
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=d, max_positions=POSITIONS if bounded else UNBOUNDED_DISTANCES, embedding=embedding,
        blocks=blocks, order=order, final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": cfg.logit_scale}, {"weight": "head"}),
        stream_mix=PartSpec("depth_average", {"entries": L, "size": d}, {f"w{i}": f"l{i}.dwa" for i in range(L)}),
    )


RULUDRA = register_architecture(Architecture(
    name="Ruludra",
    config_from_dict=RuludraConfig.from_dict,
    build_spec=build_spec,
    init=InitRule(matrix_std=0.05, vector_mean=1.0, vector_std=0.05,
                  overrides=((".dwa", 0.3, 0.2), (".mlp.act", 0.5, 0.3), (".r1", 0.5, 0.2), (".r2", 0.3, 0.1), (".i.b", 0.0, 0.5),
                             (".f.b", 2.0, 0.5), (".mix.i", 0.0, 0.3), (".mix.f", 0.0, 0.3), ("bigram", 0.0, 0.5), ("embed", 0.0, 0.5))),
))
