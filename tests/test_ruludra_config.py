"""Ruludra on the CPU: the configuration reader and its refusals, the model as data (which entry reads which cache),
the tensors a model asks for, and hand-worked cases of the plain implementation's pieces."""
import copy
import math

import numpy as np
import pytest

import plain_ruludra as P
import ruludra_configs as Z

import nanoinfer_amd  # noqa: F401
from nanoinfer_amd.config.model_config import ConfigError
from nanoinfer_amd.config.ruludra_config import RuludraConfig
from nanoinfer_amd.registry import architecture_of
from nanoinfer_amd.weights.loader import expected_tensors


def spec_of(cfg):
    arch = architecture_of(cfg)
    return arch.build_spec(arch.config_from_dict(cfg))


@pytest.mark.parametrize("name", sorted(Z.ALL))
def test_configuration_round_trip_and_spec(name):
    cfg = Z.ALL[name]
    typed = RuludraConfig.from_dict(cfg)
    assert RuludraConfig.from_dict(typed.to_dict()) == typed
    spec = spec_of(cfg)
    assert len(spec.blocks) == len(spec.order) == len(cfg["layers"])
    assert spec.stream_mix.params["entries"] == len(cfg["layers"])
    for i, (layer, run, block) in enumerate(zip(cfg["layers"], spec.order, spec.blocks)):
        src = layer["mixer"].get("kv_from")
        assert run.block == i and run.cache == (i if src is None else src) and run.writes_cache == (src is None)
        assert ("ffn" in block.parts) == (layer["mlp"] is not None) == ("ffn_post" in block.parts)


def test_tensors_of_a_model():
    names = expected_tensors(spec_of(Z.LATENT_SHARED))
    assert names["l0.mix.dkv"] == (16, 64) and names["l0.mix.dkv.norm"] == (16,)
    assert "l2.mix.dkv" not in names and "l3.mix.dkv.norm" not in names          # they read layer 0's latents
    assert names["l2.mix.uk"] == (48, 16) and names["l2.mix.uv"] == (32, 16) and names["l2.mix.uq"] == (48, 12)
    assert names["l1.mix.i.b"] == (2,) and names["l1.mix.norm"] == (16,) and names["l1.dwa"] == (3,) and names["l3.dwa"] == (5,)
    assert "l1.norm2" not in names and names["l2.norm2b"] == (64,) and names["l2.mlp.act"] == (4,)
    assert names["bigram"] == (54, 64)
    keyed = expected_tensors(spec_of(Z.KEYED_PLAIN))
    assert "bigram" not in keyed and "l0.mix.v" not in keyed and keyed["l0.mix.r1"] == (3,) and keyed["l0.mix.k.norm"] == (60,)


def test_refusals():
    def broken(edit):
        cfg = copy.deepcopy(Z.MIXED)
        edit(cfg)
        with pytest.raises(ConfigError):
            RuludraConfig.from_dict(cfg)

    broken(lambda c: c["layers"][0].update(type="conv"))
    broken(lambda c: c["layers"][0]["mixer"].update(vdim=8))                 # the values are the keys
    broken(lambda c: c["layers"][0]["mixer"].update(kv_heads=4))             # 6 heads on 4
    broken(lambda c: c["layers"][4]["mixer"].update(kv_from=3))              # not a latent layer
    broken(lambda c: c["layers"][4]["mixer"].update(kv_from=4))              # not an earlier layer
    broken(lambda c: c["layers"][4]["mixer"].update(kv_rank=16))             # another rank than the layer it reads
    broken(lambda c: c["layers"][2]["mixer"].update(kv_from=2))
    broken(lambda c: c["layers"][1]["mixer"].pop("gate_cap"))
    broken(lambda c: c["layers"][1]["mlp"].update(kind="moe"))
    broken(lambda c: c["layers"][3]["mixer"]["mask"].update(size=0))
    broken(lambda c: c.pop("norm"))


def test_pieces_of_the_plain_implementation_by_hand():
    assert P.pair_rows([3, 4, 5], 10, 7, 2) == [10, (3 * 7 + 4 * 2) % 10, (4 * 7 + 5 * 2) % 10]
    s = P.sinusoid(np.array([0, 3]), 6, 100.0)
    assert np.allclose(s[0], [0, 1, 0, 1, 0, 1])
    assert np.allclose(s[1], [math.sin(3), math.cos(3), math.sin(3 * 100 ** (-2 / 6)), math.cos(3 * 100 ** (-2 / 6)),
                              math.sin(3 * 100 ** (-4 / 6)), math.cos(3 * 100 ** (-4 / 6))])
    # a window of 2: row i sees i - 1 and i
    p = P.window_softmax(np.zeros((4, 4)), 2)
    assert np.allclose(p, [[1, 0, 0, 0], [.5, .5, 0, 0], [0, .5, .5, 0], [0, 0, .5, .5]])
    assert np.allclose(P.window_softmax(np.zeros((3, 3)), None)[2], [1 / 3] * 3)
    assert np.allclose(P.query_factor(np.array([0, 6, 7, 15]), {"coef": 2.0, "every": 8}), [1, 1, 1 + 2 * math.log(2), 1 + 2 * math.log(3)])
    pen = P.distance_penalty(3, np.array([2.0]), np.array([0.5]))
    assert np.allclose(pen[0, 2], [2 * math.log(2.0), 2 * math.log(1.5), 0.0])
    z = np.array([[1.0, -2.0, 3.0]])
    n = lambda u: u / math.sqrt((u * u).mean() + 1e-6)
    assert np.allclose(P.poly_norm(z, np.array([0.5, -1.0, 2.0, 0.25]), 1e-6), 0.5 * n(z[0]) - n(z[0] ** 2) + 2 * n(z[0] ** 3) + 0.25)


def test_the_plain_memory_continues_from_its_state_and_its_first_step_by_hand():
    rng = np.random.default_rng(3)
    m = {"heads": 2, "dim": 3, "vdim": 4, "gate_cap": 5.0}
    d = 6
    w = {"l0.mix." + k: rng.normal(size=s) for k, s in dict(q=(6, d), k=(6, d), v=(8, d), g=(8, d), i=(2, d), f=(2, d), o=(d, 8)).items()}
    w.update({"l0.mix.i.b": rng.normal(size=2), "l0.mix.f.b": rng.normal(size=2), "l0.mix.norm": rng.normal(size=8)})
    h = rng.normal(size=(9, d))
    whole, _ = P.matrix_memory(h, m, w, "l0.", 1e-6)
    first, state = P.matrix_memory(h[:4], m, w, "l0.", 1e-6)
    second, _ = P.matrix_memory(h[4:], m, w, "l0.", 1e-6, state)
    assert np.allclose(np.concatenate([first, second]), whole, rtol=1e-12, atol=1e-12)
    # the first token from an empty memory whose maximum starts at 0
    li = 5.0 * math.tanh((w["l0.mix.i"][0] @ h[0] + w["l0.mix.i.b"][0]) / 5.0)
    lf = P.log_sigmoid(5.0 * math.tanh((w["l0.mix.f"][0] @ h[0] + w["l0.mix.f.b"][0]) / 5.0))
    mx = max(lf + 0.0, li)
    S, n, run_max = state if False else P.matrix_memory(h[:1], m, w, "l0.", 1e-6)[1]
    k0, v0 = (w["l0.mix.k"] @ h[0])[:3], (w["l0.mix.v"] @ h[0])[:4]
    assert math.isclose(run_max[0], mx) and np.allclose(S[0], math.exp(li - mx) * np.outer(k0, v0)) and np.allclose(n[0], math.exp(li - mx) * k0)


def test_every_mechanism_weighs_in_the_plain_model():
    """With a tensor of each mechanism at zero (or a switch turned) the plain logits move by far more than any tolerance."""
    rng = np.random.default_rng(0)
    spec = spec_of(Z.MIXED)
    w = {}
    for name, shape in expected_tensors(spec).items():
        std = 0.12 if len(shape) > 1 else 0.05
        w[name] = rng.normal(size=shape) * std + (1.0 if len(shape) == 1 and not name.endswith((".i.b", ".act")) else 0.0)
    for i in range(6):
        w[f"l{i}.dwa"] = np.abs(w[f"l{i}.dwa"]) * 0.3
        if f"l{i}.mix.r2" in w:
            w[f"l{i}.mix.r2"] = np.abs(w[f"l{i}.mix.r2"]) * 0.3
    toks = [int(t) for t in rng.integers(0, 131, size=90)]
    want = P.forward(Z.MIXED, w, toks)

    def moved(weights=None, cfg=None):
        got = P.forward(cfg or Z.MIXED, weights or w, toks)
        return float(np.abs(got - want).max() / np.abs(want).max())

    for key in ("l0.mix.o", "l1.mix.o", "l2.mix.o", "l4.mix.uv", "l0.mlp.down", "bigram", "l3.mix.r1", "l5.mix.g", "l2.mix.g"):
        dead = dict(w)
        dead[key] = np.zeros_like(w[key])
        assert moved(dead) > 5e-3, key
    for edit in (lambda c: c["layers"][0]["mixer"].pop("q_temp"), lambda c: c["layers"][0]["mixer"]["mask"].update(size=34),
                 lambda c: c["layers"][4]["mixer"]["mask"].update(size=20), lambda c: c["layers"][1]["mixer"].update(gate_cap=2.0),
                 lambda c: c.update(logit_scale=1.0)):
        cfg = copy.deepcopy(Z.MIXED)
        edit(cfg)
        assert moved(cfg=cfg) > 1e-4
    other = dict(w)
    other["l3.dwa"] = w["l3.dwa"][::-1].copy()
    assert moved(other) > 5e-4
