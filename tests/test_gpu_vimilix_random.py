"""Vimilix configurations drawn at random (the order of layers, head counts and groups, key and value sizes, rotated
channels and their stretching, latents and their rotated parts, windows on either side of each other, of the prompt's
portions and of the kernel's tiles, layers that read an earlier layer's keys and values, experts, groups and kept groups,
limits, with and without a feed-forward and each optional block of keys), each replayed in three ways in both compute
types against the plain implementation: the whole prompt, portions of changing size, and a prompt followed by single
tokens."""
import os
import random
import shutil
import tempfile

import pytest

import vimilix_configs as Z
from gpu_common import random_tokens
from test_gpu_vimilix import assert_close, cuts, plain, replay, runner_for

pytestmark = pytest.mark.gpu


def draw(seed: int) -> dict:
    r = random.Random(seed)
    width = r.choice([32, 40, 48, 64, 72, 96, 128])
    n = r.randint(1, 6)
    layers, own = [], []           # own: (index, kv heads, dim, vdim, rotation) of attention layers that make their keys

    def window():
        return r.choice([1, 2, 7, 16, 33, 64, 65, 100, 200]) if r.random() < 0.85 else None

    def scaling():
        return (r.choice([2.0, 8.0, 32.0]), 1.0, r.choice([2.0, 4.0]), r.choice([16, 64, 1024])) if r.random() < 0.6 else None

    def experts():
        if r.random() < 0.3:
            return None
        count = r.choice([1, 2, 3, 4])
        per = r.choice([1, 2, 3, 4])
        keep = r.randint(1, count)
        top = r.randint(1, min(per * keep, 6))
        shared = (r.choice([8, 24, 50]), r.choice([0.5, 1.0, 7.0])) if r.random() < 0.7 else None
        return Z.moe(count * per, top, r.choice([8, 16, 20, 33]), r.choice([0.5, 1.5, 7.0]), scale=r.choice([0.5, 1.0, 2.5]),
                     groups=None if count == 1 and r.random() < 0.5 else (count, keep), shared=shared)

    for i in range(n):
        if r.random() < 0.55:
            source = r.choice(own) if own and r.random() < 0.5 else None
            if source is None:
                kv, dim = r.choice([1, 2, 3, 4]), r.choice([8, 16, 20, 24, 32, 48, 64])
                vdim = r.choice([dim, 8, 16, 24])
                rot_ = Z.rot(r.choice([d for d in (2, 4, 8, 16, dim) if d <= dim]), r.choice([100.0, 10000.0, 250000.0]), scaling())
                own.append((i, kv, dim, vdim, rot_))
            else:
                _, kv, dim, vdim, rot_ = source
            entry = Z.sink(kv * r.choice([1, 2, 3, 5]), kv, dim, vdim, r.choice([0.1, 0.25, 0.5]), rot_, mask=window(),
                           kv_from=source[0] if source else None)
        else:
            entry = Z.latent(r.choice([1, 2, 3, 6]), r.choice([4, 8, 12, 16, 32]), r.choice([2, 4, 8, 16]), r.choice([4, 8, 12, 16, 48]),
                             r.choice([8, 16, 20, 32, 48, 64]), r.choice([0.1, 0.25, 0.5]), base=r.choice([100.0, 50000.0]),
                             mask=window() if r.random() < 0.4 else None, scaling=scaling())
        layers.append((entry, experts()))
    return Z.model(width, r.choice([33, 64, 100, 257]), layers, alpha=r.choice([0.5, 1.0, 2.0, 3.0]), eps=r.choice([1e-6, 1e-5]))


_root = []


def folder_for(cfg, seed):
    import nanoinfer_amd  # noqa: F401
    from nanoinfer_amd.weights.loader import make_random_model
    if not _root:
        _root.append(tempfile.mkdtemp(prefix="vimilix-random-"))
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
    toks = random_tokens(cfg["vocab"], 230 if seed % 3 == 0 else 90, seed)
    want = plain(folder, toks)
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
