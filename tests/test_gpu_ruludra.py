"""Ruludra through the engine against the plain implementation (``plain_ruludra.py``): every mechanism alone and all
together, whole prompts against portions and single tokens, unequal batches against each request alone, pages and
state slots that are used again, keys far back, at the edges of pages and of the kernel's tiles of 64 keys, and just
inside and outside every window, in prompts and in decoding, the first tokens of a sequence, long decoding, and greedy
generation through ``Engine``, the command line and the trace program.

Models are written with the random-weights mode in bfloat16 (so that both compute types see the same numbers as the
plain implementation) with larger matrices than the architecture's rule draws, so that a mixer or feed-forward that
went wrong moves the logits by far more than the tolerance; where random weights would still hide a fault (one key
among hundreds, a window's edge) the test makes the inputs or the constants that show it.
"""
import functools
import json
import math
import os
import shutil
import tempfile

import numpy as np
import pytest
import torch

import plain_ruludra as P
import ruludra_configs as Z
from gpu_common import random_tokens

pytestmark = pytest.mark.gpu

_root = None
_folders = {}


def folder_of(name: str, seed: int = 11) -> str:
    global _root
    key = (name, seed)
    if key not in _folders:
        import nanoinfer_amd  # noqa: F401
        from nanoinfer_amd.weights.loader import make_random_model
        if _root is None:
            _root = tempfile.mkdtemp(prefix="ruludra-tests-")
            import atexit
            atexit.register(shutil.rmtree, _root, ignore_errors=True)
        _folders[key] = make_random_model(os.path.join(_root, f"{name}-{seed}-{len(_folders)}"), Z.ALL[name], seed,
                                          dtype="bfloat16", matrix_std=0.12)
    return _folders[key]


@functools.lru_cache(maxsize=None)
def _model(folder: str):
    return P.read_model_folder(folder)


@functools.lru_cache(maxsize=None)
def plain(folder: str, tokens: tuple) -> torch.Tensor:
    cfg, w = _model(folder)
    return torch.from_numpy(P.forward(cfg, w, list(tokens)))


def runner_for(folder, dtype, **kw):
    from nanoinfer_amd.engine.runner import ModelRunner
    kw.setdefault("page_size", 8)
    kw.setdefault("max_tokens", 2048)
    kw.setdefault("max_requests", 4)
    return ModelRunner(folder, dtype=dtype, **kw)


def replay(runner, requests, steps):
    """Run ``steps`` (each a dict request -> number of its next tokens), asking for every row; returns
    request -> logits [tokens, vocab].  A request ends with its last token."""
    from nanoinfer_amd.engine.runner import StepEntry
    done = {r: 0 for r in requests}
    rows = {r: [] for r in requests}
    for counts in steps:
        entries = [StepEntry(r, list(requests[r][done[r]:done[r] + c]), list(range(c))) for r, c in counts.items()]
        out = runner.step(entries, end=[r for r, c in counts.items() if done[r] + c == len(requests[r])])
        at = 0
        for r, c in counts.items():
            rows[r].append(out[at:at + c].clone())
            at += c
            done[r] += c
    assert all(done[r] == len(requests[r]) for r in requests)
    return {r: torch.cat(v) for r, v in rows.items()}


def cuts(n, sizes):
    out, i = [], 0
    while n > 0:
        c = min(n, sizes[i % len(sizes)])
        out.append(c)
        n -= c
        i += 1
    return out


DTYPES = ["float32", "bfloat16"]

# Float32 is the sharp comparison, row by row against the row's own largest logit: at most one row in fifty beyond
# 2e-5 and none beyond 1e-4.  (A few rows are badly conditioned whatever the schedule: the memory's read-out is divided
# by n . q, a sum that can nearly cancel, and the norm behind a sublayer divides by the size of its output; such a row
# showed 5e-5 token by token, in runs and in portions alike, next to a median of 7e-7.)  bfloat16 is judged row by row by
# the root mean square of the difference over the vocabulary (its mean taken off) against the root mean square of the
# plain logits: the median row within 2.5e-2, at most one row in ten beyond 5e-2, none beyond 0.15.  The models are
# drawn with large matrices on purpose, so rounding weighs more than in a trained model; a fault (a lost state, a key
# too many, a forgotten term) moves many rows by the size of the logits themselves.
F32_ROW, F32_WORST = 2e-5, 1e-4
BF16_MEDIAN, BF16_ROW, BF16_WORST = 2.5e-2, 5e-2, 0.15
worst_row = {"float32": 0.0, "bfloat16": 0.0}


def assert_close(got, want, dtype, what=""):
    assert tuple(got.shape) == tuple(want.shape), what
    diff = got.double().cpu() - want
    if dtype == "float32":
        per_row = diff.abs().max(dim=-1).values / want.abs().max(dim=-1).values
        worst_row[dtype] = max(worst_row[dtype], float(per_row.max()))
        over = int((per_row > F32_ROW).sum())
        assert over <= max(1, per_row.numel() // 50), f"{what}: {over} of {per_row.numel()} rows are off by more than {F32_ROW} (float32)"
        assert float(per_row.max()) <= F32_WORST, f"{what}: row {int(per_row.argmax())} is off by {float(per_row.max()):.3e} (float32)"
        return
    diff = diff - diff.mean(dim=-1, keepdim=True)
    per_row = diff.pow(2).mean(dim=-1).sqrt() / want.pow(2).mean().sqrt()
    worst_row[dtype] = max(worst_row[dtype], float(per_row.max()))
    assert float(per_row.median()) <= BF16_MEDIAN, f"{what}: the median row is off by {float(per_row.median()):.3e} (bfloat16)"
    over = int((per_row > BF16_ROW).sum())
    assert over <= max(1, per_row.numel() // 10), f"{what}: {over} of {per_row.numel()} rows are off by more than {BF16_ROW} (bfloat16)"
    assert float(per_row.max()) <= BF16_WORST, f"{what}: row {int(per_row.argmax())} is off by {float(per_row.max()):.3e} (bfloat16)"


def test_zz_report_worst_rows():
    print(f"worst rows of the Ruludra comparisons: {worst_row}")


# ------------------------------------------------------------------ every mechanism alone

ALONE = ["keyed_only", "keyed_plain", "keyed_open", "latent_only", "latent_open", "memory_only", "memory_wide", "mlp_only"]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ALONE)
def test_one_mechanism_whole_prompt_and_token_by_token(name, dtype):
    """A model of one layer with one mechanism that weighs: a whole prompt, then the same tokens as a short portion
    followed by single tokens, both equal to the plain implementation row by row."""
    folder = folder_of(name)
    toks = random_tokens(Z.ALL[name]["vocab"], 75, 5)
    want = plain(folder, toks)
    runner = runner_for(folder, dtype)
    got = replay(runner, {"w": toks}, [{"w": len(toks)}])["w"]
    assert_close(got, want, dtype, f"{name} whole")
    got = replay(runner, {"d": toks}, [{"d": 3}] + [{"d": 1}] * (len(toks) - 3))["d"]
    assert_close(got, want, dtype, f"{name} token by token")
    assert not runner.cache.live_requests()


def _moved(cfg, w, toks, want):
    return float(np.abs(P.forward(cfg, w, toks) - want).max() / np.abs(want).max())


def test_every_mechanism_matters_in_these_models():
    """The comparisons would pass with a mechanism that does nothing if it weighed nothing: with its tensors or constants
    changed the plain logits move by hundreds of times the float32 tolerance."""
    def case(name, edit_w=None, edit_cfg=None, least=5e-3):
        cfg, w = _model(folder_of(name))
        toks = list(random_tokens(cfg["vocab"], 40, 5))
        want = P.forward(cfg, w, toks)
        cfg2, w2 = json.loads(json.dumps(cfg)), dict(w)
        if edit_w:
            edit_w(w2)
        if edit_cfg:
            edit_cfg(cfg2)
        moved = _moved(cfg2, w2, toks, want)
        assert moved > least, (name, moved)

    def zero(key):
        return lambda w: w.__setitem__(key, np.zeros_like(w[key]))

    def ones(key):
        return lambda w: w.__setitem__(key, np.ones_like(w[key]))

    case("keyed_only", zero("l0.mix.o"))
    case("keyed_only", zero("l0.mix.r1"))                                              # the penalty by distance
    case("keyed_only", lambda w: w.__setitem__("l0.mix.r2", w["l0.mix.r2"] * 3))
    case("keyed_only", edit_cfg=lambda c: c["layers"][0]["mixer"].pop("q_temp"))       # the query factor
    case("keyed_only", edit_cfg=lambda c: c["layers"][0]["mixer"]["q_temp"].update(every=9))
    case("keyed_only", ones("l0.mix.q.norm"))
    case("keyed_only", ones("l0.mix.k.norm"))
    case("keyed_only", edit_cfg=lambda c: c["layers"][0]["mixer"]["mask"].update(size=19))
    case("keyed_only", zero("bigram"))
    case("keyed_only", edit_cfg=lambda c: c.update(logit_scale=1.0))
    case("keyed_only", lambda w: w.__setitem__("l0.dwa", np.array([0.0, 1.0])))        # the depth average
    case("keyed_only", ones("l0.norm1b"))
    case("latent_only", zero("l0.mix.o"))
    case("latent_only", zero("l0.mix.g"))                                              # the output gate
    case("latent_only", ones("l0.mix.dkv.norm"))
    case("latent_only", ones("l0.mix.dq.norm"))
    case("latent_only", edit_cfg=lambda c: c["layers"][0]["mixer"]["mask"].update(size=29))
    case("memory_only", zero("l0.mix.o"))
    case("memory_only", zero("l0.mix.i.b"))
    case("memory_only", zero("l0.mix.f"))
    case("memory_only", ones("l0.mix.norm"))
    case("memory_only", edit_cfg=lambda c: c["layers"][0]["mixer"].update(gate_cap=1.0))
    case("mlp_only", zero("l0.mlp.down"))
    case("mlp_only", lambda w: w.__setitem__("l0.mlp.act", np.array([1.0, 0.0, 0.0, 0.0])))
    case("mlp_only", ones("l0.norm2b"))
    case("latent_shared", zero("l2.mix.o"))                                            # a layer that reads another's latents
    case("latent_shared", edit_cfg=lambda c: c["layers"][3]["mixer"]["mask"].update(size=4))


# ------------------------------------------------------------------ the whole design, every schedule

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "latent_shared", "odd_sizes"])
def test_portions_of_several_sizes_down_to_two_tokens(name, dtype):
    folder = folder_of(name)
    toks = random_tokens(Z.ALL[name]["vocab"], 150, 21)
    want = plain(folder, toks)
    runner = runner_for(folder, dtype)
    for sizes in ([150], [2], [37, 2, 23, 3], [64, 1, 1, 17], [5, 8, 16, 1]):
        got = replay(runner, {"p": toks}, [{"p": c} for c in cuts(len(toks), sizes)])["p"]
        assert_close(got, want, dtype, f"{name} in portions of {sizes}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("graphs", [True, False])
def test_unequal_requests_in_one_batch_equal_each_alone_and_slots_are_used_again(dtype, graphs):
    """Six requests of 1 to 130 tokens through a pool that holds three at a time and too few pages for all: portions
    beside single tokens, requests that pause for a step, pages and state slots that the next request takes over as
    they are.  Every row equals the plain implementation of its request alone."""
    name = "mixed"
    folder = folder_of(name)
    vocab = Z.ALL[name]["vocab"]
    lengths = {"a": 130, "b": 1, "c": 47, "d": 80, "e": 2, "f": 66}
    requests = {r: random_tokens(vocab, n, 40 + i) for i, (r, n) in enumerate(lengths.items())}
    runner = runner_for(folder, dtype, max_tokens=8 * 36, max_requests=3, use_graphs=graphs)
    steps = [{"a": 30}, {"a": 29, "b": 1, "c": 2}, {"a": 1, "c": 16}, {"c": 1, "a": 7}, {"a": 1, "c": 1}, {"a": 1, "c": 27},
             {"a": 61}]
    steps += [{"d": 40, "e": 1}, {"e": 1, "d": 1}, {"d": 39}]
    steps += [{"f": 64}, {"f": 1}, {"f": 1}]
    got = replay(runner, requests, steps)
    for r, toks in requests.items():
        assert_close(got[r], plain(folder, toks), dtype, f"request {r}")
    runner.cache.check()
    assert not runner.cache.live_requests() and runner.cache.free_pages() == runner.cache.num_pages
    assert runner.cache.slots.num_free == 3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "memory_only"])
def test_long_portions_in_runs_beside_short_ones_and_single_tokens(name, dtype):
    """Portions long enough for the matrix memory's runs of tokens (a run and a bit, three runs and a bit, exactly two
    runs) in one step with single tokens and a portion of two, continued from states that earlier steps left."""
    folder = folder_of(name)
    vocab = Z.ALL[name]["vocab"]
    lengths = {"a": 300, "b": 150, "c": 40, "d": 128}
    requests = {r: random_tokens(vocab, n, 900 + i) for i, (r, n) in enumerate(lengths.items())}
    runner = runner_for(folder, dtype, max_tokens=1024)
    steps = [{"a": 200}, {"a": 1, "b": 129, "c": 2}, {"a": 99, "b": 1, "c": 1, "d": 128}, {"b": 20, "c": 37}]
    got = replay(runner, requests, steps)
    for r, toks in requests.items():
        assert_close(got[r], plain(folder, toks), dtype, f"request {r}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_in_a_batch_of_recorded_steps(dtype):
    """Three requests decode 160 tokens each side by side after prompts of unequal length, across many page edges, past
    every window of the model and two edges of the attention's tiles of 64 keys, in recorded steps."""
    name = "mixed"
    folder = folder_of(name)
    vocab = Z.ALL[name]["vocab"]
    prompts = {"x": 5, "y": 61, "z": 30}
    requests = {r: random_tokens(vocab, n + 160, 70 + i) for i, (r, n) in enumerate(prompts.items())}
    runner = runner_for(folder, dtype)
    got = replay(runner, requests, [dict(prompts)] + [{r: 1 for r in prompts}] * 160)
    assert any(key[0] == "d" for key in runner._recorded), "the decode steps were not recorded"
    for r, toks in requests.items():
        assert_close(got[r], plain(folder, toks), dtype, f"request {r}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens_of_a_sequence(dtype):
    """Requests of one and of two tokens, and the first rows of a longer one, on the slot and the pages that a longer
    request has just left: nothing of the request before shows (its memory and running maximum, its latents, its last
    token)."""
    name = "mixed"
    folder = folder_of(name)
    vocab = Z.ALL[name]["vocab"]
    runner = runner_for(folder, dtype, max_requests=1, max_tokens=96)
    long = random_tokens(vocab, 90, 3)
    replay(runner, {"long": long}, [{"long": 90}])
    for n in (1, 2, 5):
        toks = random_tokens(vocab, n, 100 + n)
        got = replay(runner, {"s": toks}, [{"s": 1}] * n)["s"]
        assert_close(got, plain(folder, toks), dtype, f"{n} first tokens")
    toks = random_tokens(vocab, 6, 77)
    assert_close(replay(runner, {"s": toks}, [{"s": 6}])["s"], plain(folder, toks), dtype, "a first portion")


@pytest.mark.parametrize("dtype", DTYPES)
def test_layer_by_layer_against_the_plain_stream(dtype):
    """The stream that every layer hands on (its result mixed with the earlier ones), through ``Model.tap``."""
    folder = folder_of("mixed")
    cfg, w = _model(folder)
    toks = list(random_tokens(cfg["vocab"], 40, 8))
    want = []
    P.forward(cfg, w, toks, layers_out=want)
    runner = runner_for(folder, dtype, use_graphs=False)
    got = []
    runner.model.tap = lambda i, h: got.append(h.detach().double().cpu())
    replay(runner, {"t": tuple(toks)}, [{"t": len(toks)}])
    assert len(got) == len(want) == len(cfg["layers"])
    tol = 2e-5 if dtype == "float32" else 6e-2
    for i, (a, b) in enumerate(zip(got, want)):
        err = float((a - torch.from_numpy(b)).abs().max() / np.abs(b).max())
        assert err <= tol, f"layer {i}: {err:.3e}"


# ------------------------------------------------------------------ the windows' edges and far keys, made to show

def _plain_scores_softmax(q, k, v, scale, window, penalty, factor, H, G):
    """softmax(q . k * scale * factor(i) - penalty[h, i - j]) v over the window, written out in float64."""
    T = q.shape[0]
    q, k, v = q.double().numpy(), k.double().numpy(), v.double().numpy()
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] * factor[:, None]) @ k[:, g].T * scale
        if penalty is not None:
            s = s - penalty[h]
        out[:, h] = P.window_softmax(s, window) @ v[:, g]
    return torch.from_numpy(out.reshape(T, -1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,dk,page,window,shared,temp", [(6, 2, 16, 8, 75, False, (0.5, 16)), (4, 4, 32, 16, 5, False, None),
                                                             (3, 1, 24, 4, 130, True, None), (2, 1, 64, 16, 64, True, None),
                                                             (5, 5, 16, 8, 1, False, (0.3, 7)), (2, 2, 16, 8, None, False, (1.0, 50)),
                                                             (7, 1, 48, 16, 140, True, None), (2, 1, 256, 16, 100, True, None),
                                                             (3, 1, 128, 8, 40, True, None)])
def test_window_edges_far_keys_and_the_distance_penalty_in_both_attention_kernels(H, G, dk, page, window, shared, temp, dtype):
    """The attention alone over scattered pages, with one key a query made to stand out: the key just inside the window,
    the key just outside it, a key far back and keys at the edges of the kernel's tiles of 64.  A key that is wrongly
    seen or wrongly missed takes or loses nearly all the weight.  ``shared``: keys and values are one pool (a latent, or
    values that are the keys); otherwise a penalty ``r1 ln(1 + r2 distance)`` a head is taken off the scores, strong
    enough to move the weights.  Prompt portions (the matrix-core kernel where it takes the sizes, else the vector units)
    and single tokens with the keys cut into runs must both give the written-out softmax."""
    from nanoinfer_amd import kernels as K
    from nanoinfer_amd.kernels import stream
    dev = torch.device("cuda")
    T = 300
    g = torch.Generator().manual_seed(3)
    k = torch.randn(T, G, dk, generator=g) * 0.1
    q = torch.randn(T, H, dk, generator=g) * 0.1
    win = window if window is not None else T + 1
    for i in range(T):
        places = [i - win + 1, i - win, 0, i // 2, i - 63, i - 64, i - 65, i - win + 2, i]
        j = places[i % len(places)]
        if 0 <= j <= i:
            q[i] = k[j, torch.arange(H) // (H // G)] * (160.0 / max(float(k[j].pow(2).sum(-1).max()), 1e-3))
    scale = 0.5
    qd, kd = q.to(dtype), k.to(dtype)
    vd = kd if shared else (torch.randn(T, G, dk, generator=g)).to(dtype)
    penalty = table = None
    if not shared:
        r1 = np.linspace(0.5, 6.0, H)
        r2 = np.linspace(0.05, 2.0, H)
        penalty = P.distance_penalty(T, r1, r2)
        dist = np.arange(win if window is not None else T)[:, None]
        table = torch.from_numpy(-(r1[None] * np.log1p(r2[None] * dist))).to(torch.float32).to(dev).contiguous()
    factor = P.query_factor(np.arange(T), None if temp is None else {"coef": temp[0], "every": temp[1]})
    want = _plain_scores_softmax(qd.float(), kd.float(), vd.float(), scale, window, penalty, factor, H, G)
    n_pages = (T + page - 1) // page
    perm = torch.randperm(n_pages + 5, generator=torch.Generator().manual_seed(1))[:n_pages]
    kpool = torch.full((n_pages + 5, G, page, dk), float("nan"), dtype=dtype)
    vpool = torch.full((n_pages + 5, G, page, dk), float("nan"), dtype=dtype)
    for t in range(T):
        kpool[perm[t // page], :, t % page] = kd[t]
        vpool[perm[t // page], :, t % page] = vd[t]
    kpool = kpool.to(dev)
    vpool = kpool if shared else vpool.to(dev)
    pages = perm.to(torch.int32).view(1, -1).to(dev)
    qrows = qd.reshape(T, H * dk).contiguous().to(dev)
    positions = torch.arange(T, dtype=torch.int32, device=dev)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    group = H // G
    coef, every = temp if temp is not None else (0.0, 0)

    def check(out, rows, what):
        err = float((out.double().cpu() - want[rows]).abs().max() / want.abs().max())
        assert err <= tol, f"{what}: {err:.3e}"

    for first in (0, 100, 203):
        n = T - first
        for wide in (True, False):
            rows_per = stream.bias_attention_mfma_rows(dk, dk, shared) if wide else stream.bias_attention_rows()
            if not rows_per:
                continue
            heads = min(group, rows_per)
            tile_tokens = max(1, rows_per // heads)
            tiles = torch.tensor(K.build_q_tiles([0], [n], [T], tile_tokens), dtype=torch.int32).view(-1, 4).to(dev)
            out = torch.empty(n, H * dk, dtype=dtype, device=dev)
            fn = stream.bias_attention_mfma if wide else stream.bias_attention
            fn(qrows[first:].contiguous(), kpool, vpool, pages, tiles, positions[first:].contiguous(), table, out, H, scale, coef, every,
               heads, window=window, keep_first=0)
            check(out, slice(first, T), f"portion from {first}, {'matrix cores' if wide else 'vector units'}")
    heads = min(group, stream.bias_attention_rows())
    for pos in (0, 1, win - 2, win - 1, win, win + 1, 63, 64, 65, 128, 200, 299):
        if not 0 <= pos < T:
            continue
        tiles = torch.tensor(K.build_q_tiles([0], [1], [pos + 1], 1), dtype=torch.int32).view(-1, 4).to(dev)
        for runs in (1, 3, 8):
            out = torch.empty(1, H * dk, dtype=dtype, device=dev)
            ws = torch.empty(H * runs * (dk + 2), dtype=torch.float32, device=dev) if runs > 1 else None
            stream.bias_attention(qrows[pos:pos + 1].contiguous(), kpool, vpool, pages, tiles, positions[pos:pos + 1].contiguous(), table,
                                  out, H, scale, coef, every, heads, runs, ws, 4, window, 0, 1.0)
            check(out, slice(pos, pos + 1), f"single token at {pos} in {runs} runs")


@pytest.mark.parametrize("dtype", DTYPES)
def test_sharp_windows_in_a_whole_model(dtype):
    """A model whose score factors are raised until single keys decide, with three windows (19, 23, and 66 on the latents
    of the layer with 23): prompts that end, portions that start and single tokens that fall just before, on and just
    behind every window's edge, the edges of pages (8) and of the kernel's tiles of 64 keys."""
    name = "sharp"
    folder = folder_of(name)
    toks = random_tokens(Z.ALL[name]["vocab"], 230, 9)
    want = plain(folder, toks)
    runner = runner_for(folder, dtype)
    for first in (2, 17, 18, 19, 20, 22, 23, 24, 63, 64, 65, 66, 67, 129):
        rest = len(toks) - first
        steps = [{"k": first}] + [{"k": 1}] * 3 + [{"k": c} for c in cuts(rest - 3, [62, 2, 1, 64, 3])]
        got = replay(runner, {"k": toks}, steps)["k"]
        assert_close(got, want, dtype, f"first portion of {first}")
    got = replay(runner, {"k": toks}, [{"k": 10}] + [{"k": 1}] * (len(toks) - 10))["k"]
    assert_close(got, want, dtype, "decoded past every window")
    # the rows do depend on each edge: a window one token longer or shorter moves them
    base, w = _model(folder)
    for layer, delta in ((0, 1), (0, -1), (1, 1), (1, -1), (2, 1), (2, -1)):
        other = json.loads(json.dumps(base))
        other["layers"][layer]["mixer"]["mask"]["size"] += delta
        moved = np.abs(P.forward(other, w, list(toks[:120])) - want[:120].numpy()).max() / np.abs(want.numpy()).max()
        assert moved > 1e-2, (layer, delta, moved)


# ------------------------------------------------------------------ the matrix memory's kernels alone

@pytest.mark.parametrize("runs", [False, True])
@pytest.mark.parametrize("H,dk,dv,cap", [(2, 32, 48, 12.0), (3, 24, 40, 3.0), (1, 8, 8, 30.0), (2, 128, 16, 8.0), (4, 20, 33, 1.5), (1, 40, 72, 15.0)])
def test_matrix_memory_kernels_against_the_plain_recurrence(H, dk, dv, cap, runs):
    """Three sequences of unequal length in one call, continued in a second and a third call from the state the one
    before left, with gates from shut to wide open (pre-activations far beyond the cap on both sides), so that the
    running maximum rises and the floor ``exp(-m)`` of the divisor is at work early and the normaliser later; against the
    recurrence written out in float64.  Token by token, and in runs that are chained afterwards (sequences of one token,
    of a run and a bit, of less than a run).  One size walks a sequence, and one a run, of more tokens than a workgroup
    works the gates out for at a time."""
    from nanoinfer_amd import kernels as K
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(2)
    lens = [37, 1, 300 if dv == 48 else 150] if not runs else [64, 1, 650 if H == 3 else 203]
    pad = 3                                          # columns that belong to nobody, before and between the operands
    q_col, k_col = pad, pad + H * dk + 1
    v_col = k_col + H * dk + 2
    g_col = v_col + H * dv + 4
    z_col = g_col + H * dv + 1
    wide = z_col + 2 * H + 5
    eps = 1e-5
    bias = torch.randn(2 * H, generator=g)
    norm = 1.0 + 0.3 * torch.randn(H * dv, generator=g)
    # the plain mixer reads the same rows through matrices that pick the columns
    eye = np.eye(wide)
    w = {"mix.q": eye[q_col:q_col + H * dk], "mix.k": eye[k_col:k_col + H * dk], "mix.v": eye[v_col:v_col + H * dv],
         "mix.g": eye[g_col:g_col + H * dv], "mix.i": eye[z_col:z_col + H], "mix.f": eye[z_col + H:z_col + 2 * H],
         "mix.i.b": bias[:H].double().numpy(), "mix.f.b": bias[H:].double().numpy(), "mix.norm": norm.double().numpy(),
         "mix.o": np.eye(H * dv)}
    m = {"heads": H, "dim": dk, "vdim": dv, "gate_cap": cap}
    floats = K.memory_state_floats(H, dk, dv)
    state = torch.zeros(5, floats + 4, device=dev)
    state[0] = float("nan")                          # a slot that no sequence of the call owns
    slots = torch.tensor([3, 1, 4], dtype=torch.int32, device=dev)
    plain_state = [None, None, None]
    for call in range(3):
        if call == 2:
            lens = [2, 5, 1]
        T = sum(lens)
        rows = torch.randn(T, wide, generator=g)
        rows[:, z_col:z_col + 2 * H] *= 2.5 * cap       # gates on every side of the cap
        rows[:, z_col:z_col + H] += 0.02 * cap * (call * 100 + torch.arange(T)[:, None])      # the input gate drifts up: m rises
        starts = [0, lens[0], lens[0] + lens[1]]
        q_start = torch.tensor(starts, dtype=torch.int32, device=dev)
        q_len = torch.tensor(lens, dtype=torch.int32, device=dev)
        seq_of = torch.tensor([b for b, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=dev)
        proj = rows.to(dev)
        raw, mx = K.gated_memory(proj, q_col, k_col, v_col, z_col, bias.to(dev), cap, dk ** -0.5, state, q_start, q_len, slots,
                                 H, dk, dv, max_q_len=max(lens), runs=runs and call < 2,
                                 run_len=(64 if H == 2 else 300 if H == 3 else None) if runs and call < 2 else None)
        y = K.memory_norm(raw, mx, proj, g_col, norm.to(dev), eps, state, seq_of, q_start, q_len, slots, dk, torch.float32)
        want = np.zeros((T, H * dv))
        for b, (t0, n) in enumerate(zip(starts, lens)):
            want[t0:t0 + n], plain_state[b] = P.matrix_memory(rows[t0:t0 + n].double().numpy(), m, w, "", eps, plain_state[b])
        err = float(np.abs(y.double().cpu().numpy() - want).max() / np.abs(want).max())
        assert err <= 2e-5, (call, err)
        per_row = np.abs(y.double().cpu().numpy() - want).max(axis=1) / np.maximum(np.abs(want).max(axis=1), 1e-3)
        assert float(per_row.max()) <= 2e-4, (call, int(per_row.argmax()), float(per_row.max()))
    assert bool(torch.isnan(state[0]).all()) and bool(torch.isfinite(state[1:]).all())


# ------------------------------------------------------------------ latents wider than a head: keys and values written out for a step

@pytest.fixture
def written_out(monkeypatch):
    """Portions of four tokens or more take the latent attention's other way; counts its calls."""
    from nanoinfer_amd import kernels as K
    from nanoinfer_amd.parts import gated
    calls = []
    real = K.gather_pages
    monkeypatch.setattr(gated, "LATENT_EXPAND_FROM", 4)
    monkeypatch.setattr(K, "gather_pages", lambda *a, **kw: (calls.append(a[2].shape[0]), real(*a, **kw))[1])
    return calls


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [4, 16])
def test_long_portions_over_written_out_keys_and_values_equal_the_way_over_the_latents(dtype, page_size, written_out):
    """A model whose latents are wider than a head's keys and values together (read again by two later layers, with a
    longer and a shorter window, and one layer without a window): the whole prompt, portions on both sides of the
    threshold in one sequence, and unequal requests in one batch (a long portion beside single tokens and a portion of
    two, on pages that earlier requests left) against the plain implementation of each request alone."""
    name = "latent_wide"
    folder = folder_of(name)
    vocab = Z.ALL[name]["vocab"]
    toks = random_tokens(vocab, 150, 31)
    want = plain(folder, toks)
    runner = runner_for(folder, dtype, page_size=page_size, max_tokens=320, max_requests=3)
    assert_close(replay(runner, {"w": toks}, [{"w": len(toks)}])["w"], want, dtype, "whole")
    assert written_out, "no step took the written-out way"
    for sizes in ([3, 70, 2, 5, 1], [64, 1, 1, 9], [4, 3]):
        got = replay(runner, {"p": toks}, [{"p": c} for c in cuts(len(toks), sizes)])["p"]
        assert_close(got, want, dtype, f"portions of {sizes}")
    lengths = {"a": 120, "b": 9, "c": 47, "d": 75}
    requests = {r: random_tokens(vocab, n, 60 + i) for i, (r, n) in enumerate(lengths.items())}
    steps = [{"a": 40}, {"a": 50, "b": 1, "c": 2}, {"a": 1, "b": 7, "c": 40}, {"c": 1, "a": 29, "b": 1}, {"c": 4}, {"d": 70}, {"d": 5}]
    got = replay(runner, requests, steps)
    for r, t in requests.items():
        assert_close(got[r], plain(folder, t), dtype, f"request {r}")
    assert not runner.cache.live_requests() and runner.cache.free_pages() == runner.cache.num_pages


def test_written_out_keys_and_values_at_a_window_s_edge(written_out):
    """The sharp model's shape with latents wider than its heads: whether the key at the window's edge is seen decides
    the output, also where the step's first visible key lies inside a page and inside a tile of 64 keys."""
    cfg = Z.model(64, 97, [(Z.latent(2, 8, 8, 24, 32, 40.0, mask=23), None), (Z.latent(2, 8, 8, 24, 32, 40.0, mask=66, kv_from=0), None)])
    import nanoinfer_amd  # noqa: F401
    from nanoinfer_amd.weights.loader import make_random_model
    folder = make_random_model(tempfile.mkdtemp(prefix="ruludra-wide-sharp-"), cfg, 5, dtype="bfloat16", matrix_std=0.12)
    config, w = P.read_model_folder(folder)
    toks = random_tokens(97, 230, 9)
    want = torch.from_numpy(P.forward(config, w, list(toks)))
    runner = runner_for(folder, "float32", page_size=8)
    assert_close(replay(runner, {"w": toks}, [{"w": len(toks)}])["w"], want, "float32", "whole")
    got = replay(runner, {"p": toks}, [{"p": c} for c in cuts(len(toks), [100, 7, 90, 33])])["p"]
    assert_close(got, want, "float32", "portions")
    assert len(written_out) >= 2 * 5
    shutil.rmtree(folder, ignore_errors=True)


def test_pages_picked_through_a_table_rows_as_pages_and_the_gate_of_rows():
    from nanoinfer_amd import kernels as K
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(4)
    for dtype in (torch.float32, torch.bfloat16):
        pool = torch.randn(9, 1, 4, 10, generator=g).to(dtype).to(dev)
        table = torch.tensor([[3, -1, 8, 0], [5, 2, -1, -1]], dtype=torch.int32, device=dev)
        pairs = torch.tensor([[1, 0], [0, 2], [0, 1], [1, 1], [0, 0]], dtype=torch.int32, device=dev)
        got = K.gather_pages(pool, table, pairs)
        want = torch.stack([pool[5], pool[8], torch.zeros_like(pool[0]), pool[2], pool[3]])
        assert torch.equal(got, want)
        rows = torch.randn(3 * 4, 5 * 6, generator=g).to(dtype).to(dev)
        assert torch.equal(K.rows_to_pages(rows, 4, 5, 6), rows.view(3, 4, 5, 6).permute(0, 2, 1, 3).contiguous())
        x = torch.randn(7, 33, generator=g).to(dtype).to(dev)
        wide = torch.randn(7, 50, generator=g).to(dev)
        y = K.gate_rows(x, wide, 11)
        ref = (x.float() * torch.sigmoid(wide[:, 11:44])).to(dtype)
        assert torch.allclose(y.float(), ref.float(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-6, atol=1e-6)


# ------------------------------------------------------------------ the small kernels alone

@pytest.mark.parametrize("T,n", [(1, 50), (7, 352), (70, 33), (3, 4096), (130, 8)])
@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16])
def test_the_normed_power_activation(T, n, out):
    from nanoinfer_amd import kernels as K
    g = torch.Generator().manual_seed(T + n)
    z = torch.randn(T, n, generator=g) * 3
    coef = torch.tensor([0.7, -0.4, 0.25, 0.1])
    want = P.poly_norm(z.double().numpy(), coef.double().numpy(), 1e-5)
    got = K.poly_norm(z.cuda(), coef.cuda(), 1e-5, out).double().cpu().numpy()
    tol = 2e-6 if out == torch.float32 else 8e-3
    assert np.abs(got - want).max() / np.abs(want).max() <= tol


@pytest.mark.parametrize("T,d,n", [(1, 40, 2), (9, 176, 9), (70, 33, 5), (300, 64, 1)])
def test_the_depth_weighted_mix_and_the_add_of_a_normed_output(T, d, n):
    from nanoinfer_amd import kernels as K
    g = torch.Generator().manual_seed(T + d)
    hist = torch.randn(n + 1, T, d, generator=g)
    wts = torch.randn(n, generator=g)
    dev_hist = hist.cuda()
    out = torch.empty(T, d, device="cuda")
    K.depth_mix(dev_hist[:n], wts.cuda(), out)
    want = (wts.double()[:, None, None] * hist[:n].double()).sum(0)
    assert float((out.double().cpu() - want).abs().max()) <= 1e-5 * float(want.abs().max())
    # into the row behind the ones it reads, as the model calls it
    K.depth_mix(dev_hist[:n], wts.cuda(), dev_hist[n])
    assert float((dev_hist[n].double().cpu() - want).abs().max()) <= 1e-5 * float(want.abs().max())
    h, y, w = torch.randn(T, d, generator=g), torch.randn(T, d, generator=g) * 5, torch.randn(d, generator=g)
    got = K.add_rmsnormed(h.cuda(), y.cuda(), w.cuda(), 1e-4)
    want = h.double().numpy() + P.rms(y.double().numpy(), 1e-4) * w.double().numpy()
    assert np.abs(got.double().cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()


@pytest.mark.parametrize("T,H,dv,before", [(1, 3, 12, 24), (50, 6, 48, 128), (9, 1, 7, 5), (130, 5, 16, 0)])
def test_norm_of_some_columns_heads_apart_and_the_gate_of_heads(T, H, dv, before):
    from nanoinfer_amd import kernels as K
    g = torch.Generator().manual_seed(T + H)
    wide = before + H * dv + 3
    rows = torch.randn(T, wide, generator=g) * 2
    dev = rows.cuda()
    if before:
        w = torch.randn(before, generator=g)
        got = K.rmsnorm_cols(dev, 0, w.cuda(), 1e-5, torch.float32)
        want = P.rms(rows[:, :before].double().numpy(), 1e-5) * w.double().numpy()
        assert np.abs(got.double().cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()
    w = torch.randn(H * dv, generator=g)
    got = K.rmsnorm_cols(dev, before, w.cuda(), 1e-5, torch.float32)
    want = P.rms(rows[:, before:before + H * dv].double().numpy(), 1e-5) * w.double().numpy()
    assert np.abs(got.double().cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()
    o = torch.randn(H, T, dv, generator=g)
    got = K.gate_heads(o.cuda(), dev, before, torch.float32)
    want = o.double().permute(1, 0, 2).reshape(T, H * dv).numpy() * P.sigmoid(rows[:, before:before + H * dv].double().numpy())
    assert np.abs(got.double().cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()
    apart = K.heads_apart(dev, H, dv) if before == 0 else None
    if apart is not None:
        assert torch.equal(apart.cpu(), rows[:, :H * dv].view(T, H, dv).permute(1, 0, 2).contiguous())


@pytest.mark.parametrize("pairs", [True, False])
@pytest.mark.parametrize("d", [6, 40, 176, 33])
def test_the_embedding_with_a_pair_table_and_a_sinusoid(d, pairs):
    """Two sequences in portions: the token before a portion's first is the state's; positions far out (the angle is a
    float32 product, the plain one float64: the tolerance allows for that rounding of the angle and no more)."""
    from nanoinfer_amd import kernels as K
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(d)
    vocab, buckets, mp, mc = 50, 13, 1000003, 7
    table = torch.randn(vocab, d, generator=g)
    pair = torch.randn(buckets + 1, d, generator=g) if pairs else None
    freq = torch.tensor([10000.0 ** (-2.0 * i / d) for i in range((d + 1) // 2)], dtype=torch.float64).to(torch.float32)
    seqs = [random_tokens(vocab, 30, 1), random_tokens(vocab, 11, 2)]
    state = torch.full((4, 1), -7, dtype=torch.int32, device=dev)
    slots = torch.tensor([2, 0], dtype=torch.int32, device=dev)
    done = [0, 0]
    for portion in ([5, 1], [1, 2], [24, 8]):
        ids, pos, seq_of, starts = [], [], [], []
        for b, n in enumerate(portion):
            starts.append(len(ids))
            ids += seqs[b][done[b]:done[b] + n]
            pos += list(range(done[b], done[b] + n))
            seq_of += [b] * n
        ints = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
        out = torch.empty(len(ids), d, device=dev)
        K.embed_pair_hash(ints(ids), ints(pos), ints(seq_of), ints(starts), ints(portion), slots, state, table.to(dev),
                          None if pair is None else pair.to(dev), buckets if pairs else 0, mp if pairs else 0, mc if pairs else 0,
                          1.0, out, freq=freq.to(dev))
        for b, n in enumerate(portion):
            whole = list(seqs[b][:done[b] + n])
            want = table[whole].double().numpy() + P.sinusoid(np.arange(len(whole)), d)
            if pairs:
                want = want + pair[P.pair_rows(whole, buckets, mp, mc)].double().numpy()
            got = out[starts[b]:starts[b] + n].double().cpu().numpy()
            assert np.abs(got - want[done[b]:]).max() <= 1e-5
            done[b] += n
    # a position of millions: the float32 angle p * freq is off by up to p * 2^-24 of the true one
    p = 3_000_001
    out = torch.empty(1, d, device=dev)
    state.fill_(4)
    K.embed_pair_hash(torch.tensor([3], dtype=torch.int32, device=dev), torch.tensor([p], dtype=torch.int32, device=dev),
                      torch.zeros(1, dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev),
                      torch.ones(1, dtype=torch.int32, device=dev), slots[:1], state, table.to(dev), None, 0, 0, 0, 1.0, out, freq=freq.to(dev))
    angle = (torch.tensor(float(p), dtype=torch.float32) * freq).double()
    want = table[3].double().clone()
    want[0::2] += torch.sin(angle)[: (d + 1) // 2]
    want[1::2] += torch.cos(angle)[: d // 2]
    assert float((out[0].double().cpu() - want).abs().max()) <= 1e-5


# ------------------------------------------------------------------ generation through the engine's own entry point

@pytest.mark.parametrize("name", ["mixed", "latent_shared"])
def test_greedy_generation_through_the_engine_is_the_plain_greedy(name):
    """``Engine.generate`` (scheduler, chunked prompts, recorded decode runs, preemption on a pool that is too small)
    gives the tokens that the plain implementation's argmax gives, wherever the plain logits leave no doubt."""
    from nanoinfer_amd.engine.llm import Engine
    from nanoinfer_amd.engine.scheduler import EngineConfig
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = folder_of(name)
    cfg, w = _model(folder)
    prompts = [list(random_tokens(cfg["vocab"], n, 300 + n)) for n in (3, 26, 11, 40, 1)]
    new = 20
    eng = Engine(folder, EngineConfig(dtype="float32", block_size=8, num_cache_blocks=10, max_sequences=3, admission_headroom=0,
                                      prefill_chunk_size=16, max_num_batched_tokens=40), ignore_eos=True)
    results = eng.generate(prompts, max_new_tokens=new, params=SamplingParams.greedy())
    assert eng.scheduler.num_preemptions > 0, "the pool was meant to be too small for all"
    checked = 0
    for prompt, res in zip(prompts, results):
        toks = list(prompt)
        assert len(res.tokens) == new
        for t in res.tokens:
            row = P.forward(cfg, w, toks)[-1]
            top = np.sort(row)[-2:]
            if float(top[1] - top[0]) > 1e-3 * float(np.abs(row).max()):
                assert t == int(row.argmax()), (len(prompt), len(toks))
                checked += 1
            toks.append(t)
    assert checked >= len(prompts) * new * 3 // 4
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.num_pages


def test_sampling_with_temperature_runs_and_respects_the_seed():
    from nanoinfer_amd.engine.llm import Engine
    from nanoinfer_amd.engine.scheduler import EngineConfig
    from nanoinfer_amd.sampling.params import SamplingParams
    folder = folder_of("mixed")
    prompts = [list(random_tokens(Z.MIXED["vocab"], n, 500 + n)) for n in (9, 20)]
    outs = []
    for _ in range(2):
        eng = Engine(folder, EngineConfig(dtype="bfloat16", block_size=8, num_cache_blocks=64, max_sequences=4), ignore_eos=True)
        outs.append([r.tokens for r in eng.generate(prompts, max_new_tokens=10,
                                                    params=SamplingParams(temperature=0.8, top_k=20, top_p=0.9, seed=5))])
    assert outs[0] == outs[1] and all(len(t) == 10 for t in outs[0])


def test_the_command_line_generates_from_a_ruludra_folder(tmp_path, capsys):
    """``bin/nanoinfer``'s program with a Ruludra ``config.json``: the random-weights mode writes the folder, the engine
    generates greedily from two prompts, and the tokens are the plain implementation's."""
    from nanoinfer_amd import cli
    cfg_path, folder = str(tmp_path / "config.json"), str(tmp_path / "model")
    with open(cfg_path, "w") as fh:
        json.dump(Z.LATENT_SHARED, fh)
    rc = cli.main(["--random-config", cfg_path, "--save-random-model", folder, "--random-seed", "3", "--dtype", "fp32",
                   "--prompt-ids", "5,9,77,3,90", "--prompt-len", "19", "--max-tokens", "6", "--ignore-eos", "--json",
                   "--num-cache-blocks", "32", "--block-size", "8"])
    assert rc == 0
    lines = [json.loads(l) for l in capsys.readouterr().out.splitlines() if l.startswith("{")]
    assert len(lines) == 2 and lines[0]["prompt_len"] == 5 and lines[1]["prompt_len"] == 19
    cfg, w = P.read_model_folder(folder)
    toks = [5, 9, 77, 3, 90]
    for t in lines[0]["tokens"]:
        row = P.forward(cfg, w, toks)[-1]
        top = np.sort(row)[-2:]
        if float(top[1] - top[0]) > 1e-3 * float(np.abs(row).max()):
            assert t == int(row.argmax())
        toks.append(t)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_program_replays_a_ruludra_model(dtype, tmp_path):
    """``bin/trace_run`` in a process of its own, four state slots: portions beside single tokens, a request that
    pauses, a fifth request on a slot and pages that another has given back."""
    import subprocess
    import sys
    name = "mixed"
    folder = folder_of(name)
    vocab = Z.ALL[name]["vocab"]
    lengths = {"a": 70, "b": 33, "c": 9, "d": 52, "e": 41}
    requests = {r: random_tokens(vocab, n, 800 + i) for i, (r, n) in enumerate(lengths.items())}
    plan = [{"a": 30, "b": 2}, {"a": 1, "b": 31, "c": 8, "d": 20}, {"a": 1, "c": 1, "d": 1}, {"a": 37, "d": 31},
            {"a": 1, "e": 40}, {"e": 1}]
    done = {r: 0 for r in requests}
    lines, wanted = [], []
    for i, counts in enumerate(plan):
        entries, ended = [], []
        for r, c in counts.items():
            entries.append({"id": r, "tokens": list(requests[r][done[r]:done[r] + c]), "want": list(range(c))})
            wanted.append((i, r, done[r], c))
            done[r] += c
            if done[r] == len(requests[r]):
                ended.append(r)
        lines.append(json.dumps({"step": i, "entries": entries, "end": ended}))
    out_dir = str(tmp_path / "out")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", out_dir, "--max-tokens", "192", "--page-size", "8"],
                          input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(plan))]
    rows = {r: [None] * len(requests[r]) for r in requests}
    for i in range(len(plan)):
        data = np.fromfile(os.path.join(out_dir, f"{i}.f32"), dtype="<f4").reshape(-1, vocab)
        at = 0
        for step, r, first, c in wanted:
            if step == i:
                for j in range(c):
                    rows[r][first + j] = torch.from_numpy(data[at + j].copy())
                at += c
        assert at == data.shape[0]
    for r, toks in requests.items():
        assert_close(torch.stack(rows[r]), plain(folder, toks), dtype, f"trace program, request {r}")
