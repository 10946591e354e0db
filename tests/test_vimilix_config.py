"""Vimilix on the CPU: the configuration reader and its refusals, the model as data (which entry reads which cache, what
the pages of a layer keep), the tensors a model asks for, and hand-worked cases of the plain implementation's pieces."""
import copy
import math

import numpy as np
import pytest

import plain_vimilix as P
import vimilix_configs as Z

import nanoinfer_amd  # noqa: F401
from nanoinfer_amd.config.model_config import ConfigError
from nanoinfer_amd.config.vimilix_config import VimilixConfig
from nanoinfer_amd.registry import architecture_of
from nanoinfer_amd.weights.loader import expected_tensors


def spec_of(cfg):
    arch = architecture_of(cfg)
    return arch.build_spec(arch.config_from_dict(cfg))


@pytest.mark.parametrize("name", sorted(Z.ALL))
def test_configuration_round_trip_and_spec(name):
    cfg = Z.ALL[name]
    typed = VimilixConfig.from_dict(cfg)
    assert VimilixConfig.from_dict(typed.to_dict()) == typed
    spec = spec_of(cfg)
    assert len(spec.blocks) == len(spec.order) == len(cfg["layers"])
    for i, (layer, run, block) in enumerate(zip(cfg["layers"], spec.order, spec.blocks)):
        src = layer["mixer"].get("kv_from")
        assert run.block == i and run.cache == (i if src is None else src) and run.writes_cache == (src is None)
        assert ("ffn" in block.parts) == (layer["mlp"] is not None) == ("ffn_norm" in block.parts)
        assert block.kind == "postnorm" and block.params["alpha"] == cfg["postln_alpha"]


def test_the_pages_of_a_layer_keep_the_longest_window_that_reads_them():
    spec = spec_of(Z.SHARED_KV)          # windows 9 (the writer), 50 and 3
    assert [spec.blocks[i].parts["mixer"].params["cache_window"] for i in (0, 2, 3)] == [50, 50, 50]
    assert [spec.blocks[i].parts["mixer"].params["window"] for i in (0, 2, 3)] == [9, 50, 3]
    spec = spec_of(Z.SHARED_OPEN)        # a reader without a window
    assert [spec.blocks[i].parts["mixer"].params["cache_window"] for i in (0, 1)] == [None, None]
    assert spec_of(Z.SINK_ONLY).blocks[0].parts["mixer"].params["cache_window"] == 20


def test_tensors_of_a_model():
    names = expected_tensors(spec_of(Z.SHARED_KV))
    assert names["embed"] == (97, 64) and names["embed.norm"] == (64,) and names["final.norm"] == (64,) and names["head"] == (97, 64)
    assert names["l0.mix.q"] == (64, 64) and names["l0.mix.k"] == (32, 64) and names["l0.mix.v"] == (16, 64)
    assert names["l0.mix.q.norm"] == (16,) and names["l0.mix.k.norm"] == (16,) and names["l0.mix.sink"] == (4,)
    assert names["l0.mix.g"] == (4, 64) and names["l0.mix.o"] == (64, 32)
    for gone in ("l2.mix.k", "l2.mix.v", "l2.mix.k.norm", "l3.mix.k", "l0.norm2", "l0.mlp.router"):
        assert gone not in names
    assert names["l2.mix.q"] == (32, 64) and names["l3.mix.q"] == (96, 64) and names["l3.mix.g"] == (6, 64)
    assert names["l1.mix.q"] == (2 * 12, 64) and names["l1.mix.dkv"] == (16, 64) and names["l1.mix.dkv.norm"] == (12,)
    assert names["l1.mix.uk"] == (16, 12) and names["l1.mix.uv"] == (16, 12) and names["l1.mix.g"] == (2, 64)
    assert names["l2.mlp.router"] == (4, 64) and names["l2.mlp.correction"] == (4,) and names["l2.mlp.e3.down"] == (64, 16)
    assert "l2.mlp.shared.gate" not in names and names["l2.norm2"] == (64,)
    moe = expected_tensors(spec_of(Z.MOE_ONLY))
    assert moe["l0.mlp.shared.gate"] == (40, 56) and moe["l0.mlp.shared.down"] == (56, 40) and moe["l0.mlp.e11.up"] == (24, 56)


def test_refusals():
    def broken(edit, base=Z.MIXED):
        cfg = copy.deepcopy(base)
        edit(cfg)
        with pytest.raises(ConfigError):
            VimilixConfig.from_dict(cfg)

    broken(lambda c: c["layers"][0].update(type="conv"))
    broken(lambda c: c["layers"][1]["mixer"].update(kv_heads=4))             # 6 heads on 4
    broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=18))         # more than a head
    broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7))          # pairs
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=8))          # the latent's rotated part is rot_dim
    broken(lambda c: c["layers"][3]["mixer"].update(kv_from=2))              # not an attention layer
    broken(lambda c: c["layers"][3]["mixer"].update(kv_from=3))              # not an earlier layer
    broken(lambda c: c["layers"][3]["mixer"].update(dim=8))                  # another key size than the layer it reads
    broken(lambda c: c["layers"][3]["mixer"]["rot"].update(base=10.0))       # another rotation
    broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=7))          # 7 of 3 groups of 2
    broken(lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=3))
    broken(lambda c: c["layers"][0]["mlp"].update(kind="dense"))
    broken(lambda c: c["layers"][0]["mlp"]["expert"].pop("limit"))
    broken(lambda c: c["layers"][1]["mixer"]["mask"].update(size=0))
    broken(lambda c: c.pop("postln_alpha"))
    broken(lambda c: c.pop("norm"))
    # a chain of readers: the layer that is read must make its own keys
    chain = copy.deepcopy(Z.SHARED_KV)
    chain["layers"][3]["mixer"]["kv_from"] = 2
    with pytest.raises(ConfigError):
        VimilixConfig.from_dict(chain)


def test_rotation_frequencies_by_hand():
    f = P.rotation_frequencies({"dims": 8, "base": 300.0})
    assert np.allclose(f, [1.0, 300 ** -0.25, 300 ** -0.5, 300 ** -0.75])
    # waves of 2 pi / f = 6.3, 26.1, 108.8 and 452.8 positions against original / high = 21.3 and original / low = 64
    s = P.rotation_frequencies({"dims": 8, "base": 300.0, "scaling": dict(zip(("factor", "low", "high", "original"), Z.LONG_WAVES))})
    assert s[0] == f[0]                                           # short: kept
    assert np.allclose(s[2:], f[2:] / 4.0)                        # long: divided by the factor
    t = (64 / (2 * math.pi / f[1]) - 1.0) / (3.0 - 1.0)           # between: a blend
    assert 0 < t < 1 and math.isclose(s[1], (1 - t) * f[1] / 4.0 + t * f[1])
    # the engine's frequencies are these numbers
    from nanoinfer_amd.parts.standard import rope_inverse_frequencies
    got = rope_inverse_frequencies(8, 300.0, {"kind": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 3.0,
                                              "original_max_position_embeddings": 64.0}, exact=True)
    assert np.allclose(got, s, rtol=1e-6)


def test_rotation_of_neighbouring_pairs_by_hand():
    x = np.arange(1.0, 9.0).reshape(1, 1, 8).repeat(2, axis=0)                # positions 0 and 1
    y = P.rotate_pairs(x, np.array([0, 3]), np.array([0.5, 0.1, 0.0, 2.0]))
    assert np.allclose(y[0], x[0])
    for i, f in enumerate([0.5, 0.1, 0.0, 2.0]):
        a, b = x[1, 0, 2 * i], x[1, 0, 2 * i + 1]
        assert math.isclose(y[1, 0, 2 * i], a * math.cos(3 * f) - b * math.sin(3 * f))
        assert math.isclose(y[1, 0, 2 * i + 1], b * math.cos(3 * f) + a * math.sin(3 * f))


def test_softmax_with_a_sink_by_hand():
    p = P.sink_softmax(np.zeros((4, 4)), 0.0, 2)        # a window of 2: row i sees i - 1 and i; the sink weighs like a key
    assert np.allclose(p, [[.5, 0, 0, 0], [1 / 3, 1 / 3, 0, 0], [0, 1 / 3, 1 / 3, 0], [0, 0, 1 / 3, 1 / 3]])
    p = P.sink_softmax(np.zeros((3, 3)), math.log(2.0), None)
    assert np.allclose(p[2], [1 / 5] * 3) and np.allclose(p[0, 0], 1 / 3)
    assert np.allclose(P.sink_softmax(np.zeros((2, 2)), -1e9, None)[1], [.5, .5])       # a sink far below: a plain softmax
    assert np.allclose(P.sink_softmax(np.full((2, 2), -800.0), 700.0, None), 0.0)       # and far above: nothing is left


def test_the_router_by_hand():
    # six experts in three groups; sigmoid scores (as logits below) plus correction
    s = np.array([0.9, 0.1, 0.6, 0.55, 0.2, 0.8])
    z = np.log(s / (1 - s))
    corr = np.array([0.0, 0.0, 0.0, 0.0, 0.5, -0.3])
    h = np.eye(6)[:1] * 0 + 1.0                                   # one token whose logits are the router's row sums
    w = {"l0.mlp.router": np.diag(z) @ np.ones((6, 6)) / 6.0, "l0.mlp.correction": corr}
    mlp = {"router": {"experts": 6, "top": 2, "scale": 2.0, "groups": {"count": 3, "keep": 2}}}
    chosen, weights = P.route(h, mlp, w, "l0.")
    # choice scores .9 .1 | .6 .55 | .7 .5 -> group sums 1.0, 1.15, 1.2: groups 2 and 1 are kept, expert 0 is not
    assert chosen.tolist() == [[4, 2]]
    assert np.allclose(weights, [[2.0 * 0.2, 2.0 * 0.6]])         # the weights never see the correction
    mlp["router"]["groups"] = {"count": 3, "keep": 3}
    assert P.route(h, mlp, w, "l0.")[0].tolist() == [[0, 4]]
    mlp["router"].pop("groups")
    assert P.route(h, mlp, w, "l0.")[0].tolist() == [[0, 4]]


def test_an_expert_by_hand():
    w = {"e.gate": np.array([[1.0, 0.0], [0.0, 1.0]]), "e.up": np.array([[0.0, 1.0], [1.0, 0.0]]), "e.down": np.array([[1.0, 1.0]])}
    h = np.array([[3.0, -0.5]])                                   # gates 3 -> 2 (capped), -0.5; ups -0.5, 3 -> 2 (capped)
    g0, g1 = 2.0, -0.5
    want = g0 / (1 + math.exp(-1.702 * g0)) * (-0.5 + 1) + g1 / (1 + math.exp(-1.702 * g1)) * (2.0 + 1)
    assert np.allclose(P.expert(h, w, "e.", 2.0), [[want]])
    h = np.array([[-9.0, 0.0]])                                   # a gate far below is not capped, an up far below is
    g0 = -9.0
    assert np.allclose(P.expert(h, w, "e.", 2.0), [[g0 / (1 + math.exp(-1.702 * g0)) * 1.0 + 0.0 * (-2.0 + 1)]])


def test_every_mechanism_weighs_in_the_plain_model():
    """With a tensor of each mechanism at zero (or a switch turned) the plain logits move by far more than any tolerance."""
    rng = np.random.default_rng(0)
    spec = spec_of(Z.MIXED)
    w = {}
    for name, shape in expected_tensors(spec).items():
        std = 0.12 if len(shape) > 1 else 0.05
        centre = 1.0 if len(shape) == 1 and not name.endswith((".sink", ".correction")) else 0.0
        w[name] = rng.normal(size=shape) * std + centre
    toks = [int(t) for t in rng.integers(0, 131, size=90)]
    want = P.forward(Z.MIXED, w, toks)

    def moved(weights=None, cfg=None):
        got = P.forward(cfg or Z.MIXED, weights or w, toks)
        return float(np.abs(got - want).max() / np.abs(want).max())

    for key in ("l0.mix.o", "l1.mix.o", "l3.mix.o", "l2.mix.uv", "l0.mlp.shared.down", "l1.mlp.router", "l3.mix.q", "l1.mix.v"):
        dead = dict(w)
        dead[key] = np.zeros_like(w[key])
        assert moved(dead) > 5e-3, key
    for key, value in (("l1.mix.sink", 3.0), ("l0.mix.sink", 3.0), ("l1.mix.g", 2.0), ("l2.mix.g", 2.0), ("l1.mix.q.norm", 2.0),
                       ("l1.mix.k.norm", 2.0), ("l0.mix.dkv.norm", 2.0), ("embed.norm", 2.0), ("l0.norm1", 2.0)):
        other = dict(w)
        other[key] = w[key] + value * (np.arange(w[key].size).reshape(w[key].shape) % 2)
        assert moved(other) > 1e-3, key
    other = dict(w)
    other["l0.mlp.correction"] = w["l0.mlp.correction"] + np.array([2.0, 0, 0, 0, 0, 0, -2.0, 0])
    assert moved(other) > 1e-3
    for edit in (lambda c: c["layers"][1]["mixer"]["mask"].update(size=34), lambda c: c["layers"][3]["mixer"]["mask"].update(size=20),
                 lambda c: c["layers"][2]["mixer"]["mask"].update(size=9), lambda c: c["layers"][1]["mixer"]["rot"].pop("scaling"),
                 lambda c: c["layers"][0]["mixer"]["rot"].update(base=20.0), lambda c: c["layers"][0]["mlp"]["expert"].update(limit=0.1),
                 lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=2), lambda c: c["layers"][1]["mlp"]["shared"].update(limit=0.05),
                 lambda c: c["layers"][3]["mlp"]["router"].update(scale=1.5), lambda c: c.update(postln_alpha=1.0)):
        cfg = copy.deepcopy(Z.MIXED)
        edit(cfg)
        assert moved(cfg=cfg) > 1e-4
