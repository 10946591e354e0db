"""Ruludra configurations drawn at random (the order of layers, head counts and groups, key and value sizes, the ranks
of both latents, windows on either side of each other, of the prompt's portions and of the kernel's tiles, layers that
read an earlier layer's latents, caps of the gates, layers with and without a feed-forward, with and without each
optional block of keys), each replayed in three ways in both compute types against the plain implementation: the whole
prompt, portions of changing size, and a prompt followed by single tokens."""
import os
import random
import shutil
import tempfile

import pytest
import torch

import plain_ruludra as P
import ruludra_configs as Z
from gpu_common import random_tokens
from test_gpu_ruludra import assert_close, cuts, replay, runner_for

pytestmark = pytest.mark.gpu


def draw(seed: int) -> dict:
    r = random.Random(seed)
    width = r.choice([32, 40, 48, 64, 72, 96, 128])
    n = r.randint(1, 6)
    layers, own = [], []           # own: (index, kv_rank) of latent layers that make their latents

    def window():
        return r.choice([1, 2, 7, 16, 33, 64, 65, 100, 200]) if r.random() < 0.85 else None

    for i in range(n):
        kind = r.choice(["attention", "latent_attention", "mlstm"])
        if kind == "attention":
            kv = r.choice([1, 2, 3, 4])
            temp = (r.choice([0.1, 0.5, 1.0]), r.choice([1, 4, 16, 50])) if r.random() < 0.7 else None
            entry = Z.keyed(kv * r.choice([1, 2, 3, 5]), kv, r.choice([8, 16, 20, 24, 32, 48, 64]), r.choice([0.1, 0.25, 0.5]),
                            mask=window(), temp=temp)
        elif kind == "latent_attention":
            source = r.choice(own) if own and r.random() < 0.5 else None
            rank = source[1] if source else r.choice([8, 16, 20, 32, 48, 64])
            entry = Z.latent(r.choice([1, 2, 3, 6]), r.choice([4, 8, 12, 16, 32]), r.choice([4, 8, 12, 16, 48]), r.choice([8, 12, 24, 64]),
                             rank, r.choice([0.5, 1.0, 2.0]), mask=window(), kv_from=source[0] if source else None)
            if source is None:
                own.append((i, rank))
        else:
            entry = Z.memory(r.choice([1, 2, 3, 4]), r.choice([8, 12, 16, 24, 40, 64]), r.choice([8, 9, 16, 20, 32, 64]),
                             r.choice([1.0, 4.0, 12.0, 30.0]))
        layers.append((entry, r.choice([None, 24, 50, 64, 100])))
    bigram = (r.choice([7, 64, 101]), r.choice([1, 31, 1000003]), r.choice([1, 7, 65537])) if r.random() < 0.7 else None
    return Z.model(width, r.choice([33, 64, 100, 257]), layers, bigram=bigram, eps=r.choice([1e-6, 1e-5]),
                   logit_scale=r.choice([0.25, 1.0, 2.0]))


_root = []


def folder_for(cfg, seed):
    import nanoinfer_amd  # noqa: F401
    from nanoinfer_amd.weights.loader import make_random_model
    if not _root:
        _root.append(tempfile.mkdtemp(prefix="ruludra-random-"))
        import atexit
        atexit.register(shutil.rmtree, _root[0], ignore_errors=True)
    return make_random_model(os.path.join(_root[0], f"m{seed}"), cfg, seed, dtype="bfloat16", matrix_std=0.1)


@pytest.mark.parametrize("seed", list(range(1, 15)))
def test_a_configuration_drawn_at_random(seed, monkeypatch):
    if seed % 2:            # portions of sixteen tokens write the heads' keys and values out, where the latents are wide
        from nanoinfer_amd.parts import gated
        monkeypatch.setattr(gated, "LATENT_EXPAND_FROM", 16)
    cfg = draw(seed)
    folder = folder_for(cfg, seed)
    config, w = P.read_model_folder(folder)
    toks = random_tokens(cfg["vocab"], 230 if seed % 3 == 0 else 90, seed)
    want = torch.from_numpy(P.forward(config, w, list(toks)))
    rng = random.Random(seed)
    for dtype in ("float32", "bfloat16"):
        runner = runner_for(folder, dtype, page_size=rng.choice([1, 4, 8, 16, 32]))
        got = replay(runner, {"w": toks}, [{"w": len(toks)}])["w"]
        assert_close(got, want, dtype, f"seed {seed}: whole")
        sizes = [rng.choice([1, 2, 3, 5, 16, 31, 64]) for _ in range(5)]
        got = replay(runner, {"p": toks}, [{"p": c} for c in cuts(len(toks), sizes)])["p"]
        assert_close(got, want, dtype, f"seed {seed}: portions of {sizes}")
        first = rng.randint(1, len(toks) - 20)
        got = replay(runner, {"d": toks}, [{"d": first}] + [{"d": 1}] * (len(toks) - first))["d"]
        assert_close(got, want, dtype, f"seed {seed}: {first} tokens, then one by one")
        assert not runner.cache.live_requests()
