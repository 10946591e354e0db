"""Vimilix through the engine against the plain implementation (``plain_vimilix.py``): every mechanism alone and all
together, whole prompts against portions and single tokens, unequal batches against each request alone, pages and
slots that are used again, pages that a window has passed and given back, keys far back, at the edges of pages and of
the kernel's tiles of 64 keys, and just inside and outside every window, in prompts and in decoding, the first tokens
of a sequence, long decoding, and greedy generation through ``Engine``, the command line and the trace program.

Models are written with the random-weights mode in bfloat16 (so that both compute types see the same numbers as the
plain implementation) with larger matrices than the architecture's rule draws, so that a mixer or feed-forward that
went wrong moves the logits by far more than the tolerance; where random weights would still hide a fault (one key
among hundreds, a sink, a window's edge) the test makes the inputs or the constants that show it.
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

import plain_vimilix as P
import vimilix_configs as Z
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
            _root = tempfile.mkdtemp(prefix="vimilix-tests-")
            import atexit
            atexit.register(shutil.rmtree, _root, ignore_errors=True)
        _folders[key] = make_random_model(os.path.join(_root, f"{name}-{seed}-{len(_folders)}"), Z.ALL[name], seed,
                                          dtype="bfloat16", matrix_std=0.12)
    return _folders[key]


@functools.lru_cache(maxsize=None)
def _model(folder: str):
    return P.read_model_folder(folder)


@functools.lru_cache(maxsize=None)
def _plain(folder: str, tokens: tuple):
    cfg, w = _model(folder)
    margins = np.full(len(tokens), np.inf)
    return torch.from_numpy(P.forward(cfg, w, list(tokens), margins=margins)), torch.from_numpy(margins)


class Plain(torch.Tensor):
    """The plain logits of a sequence, with ``margins`` [tokens]: the smallest gap by which a router chose for each."""


def plain(folder: str, tokens: tuple) -> torch.Tensor:
    logits, margins = _plain(folder, tokens)
    out = logits.as_subclass(Plain)
    out.margins = margins
    return out


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


def all_pages_free(cache) -> bool:
    return all(g.pages.num_free == g.pages.num_pages for g in cache.groups)


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
# 2e-5 and none beyond 1e-4.  bfloat16 is judged row by row by the root mean square of the difference over the
# vocabulary (its mean taken off) against the root mean square of the plain logits: the median row within 2.5e-2, at
# most one row in ten beyond 5e-2, none beyond 0.15.  The models are drawn with large matrices on purpose, so rounding
# weighs more than in a trained model; a fault (a key too many, a forgotten sink, an expert that was not chosen) moves
# many rows by the size of the logits themselves.  A router chooses by comparing scores, and a score that bfloat16
# rounding of its input moves by a few thousandths can fall on the other side of its neighbour: the token then runs
# another expert in either implementation with equal right.  The plain implementation says by how little every token's
# choices were made; in bfloat16 the rows of tokens that chose by less than ``CLOSE_CALL`` are held to the median and to
# the count of rows beyond 5e-2, not to the bound on the worst row.
F32_ROW, F32_WORST = 2e-5, 1e-4
BF16_MEDIAN, BF16_ROW, BF16_WORST = 2.5e-2, 5e-2, 0.15
CLOSE_CALL, CLOSE_CALL_F32 = 0.03, 1e-5
worst_row = {"float32": 0.0, "bfloat16": 0.0}


def assert_close(got, want, dtype, what=""):
    assert tuple(got.shape) == tuple(want.shape), what
    diff = got.double().cpu() - want
    margins = getattr(want, "margins", None)
    if dtype == "float32":
        per_row = diff.abs().max(dim=-1).values / want.abs().max(dim=-1).values
        if margins is not None:         # a choice made by less than float32 rounding moves a score
            per_row = torch.where(margins < CLOSE_CALL_F32, torch.zeros_like(per_row), per_row)
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
    if margins is not None:
        per_row = torch.where(margins < CLOSE_CALL, torch.zeros_like(per_row), per_row)
    assert float(per_row.max()) <= BF16_WORST, f"{what}: row {int(per_row.argmax())} is off by {float(per_row.max()):.3e} (bfloat16)"


def test_zz_report_worst_rows():
    print(f"worst rows of the Vimilix comparisons: {worst_row}")


# ------------------------------------------------------------------ every mechanism alone

ALONE = ["sink_only", "sink_open", "latent_only", "latent_odd", "latent_huge", "moe_only", "moe_flat", "moe_singles", "shared_open"]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ALONE)
def test_one_mechanism_whole_prompt_and_token_by_token(name, dtype):
    """A model of one layer (or of a layer and its reader): a whole prompt, then the same tokens as a short portion
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


# ------------------------------------------------------------------ the whole design, every schedule

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "shared_kv", "odd_sizes", "latent_huge"])
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
    beside single tokens, requests that pause for a step, pages and slots that the next request takes over as they are.
    Every row equals the plain implementation of its request alone."""
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
    assert not runner.cache.live_requests() and all_pages_free(runner.cache)
    assert runner.cache.slots.num_free == 3


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
def test_pages_that_a_window_has_passed_are_given_back_and_used_again(dtype):
    """A model whose only pages are those of a window of 20 keys: a sequence of 300 tokens through a pool of 160, in
    portions and single tokens, beside a second request that takes the pages the first gives back."""
    name = "sink_only"
    folder = folder_of(name)
    vocab = Z.ALL[name]["vocab"]
    requests = {"a": random_tokens(vocab, 300, 61), "b": random_tokens(vocab, 120, 62)}
    runner = runner_for(folder, dtype, max_tokens=160, max_requests=2)
    steps = [{"a": 41}] + [{"a": 1}] * 30 + [{"a": 17, "b": 20}] + [{"a": 1, "b": 1}] * 60 + [{"a": 26, "b": 39}, {"a": 60}, {"a": 66}, {"b": 1}]
    got = replay(runner, requests, steps)
    for r, toks in requests.items():
        assert_close(got[r], plain(folder, toks), dtype, f"request {r}")
    runner.cache.check()
    assert all_pages_free(runner.cache)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens_of_a_sequence(dtype):
    """Requests of one and of two tokens, and the first rows of a longer one, on the slot and the pages that a longer
    request has just left: nothing of the request before shows."""
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
    """The stream behind every layer, through ``Model.tap``."""
    folder = folder_of("mixed")
    cfg, w = _model(folder)
    toks = list(random_tokens(cfg["vocab"], 40, 8))
    want, margins = [], np.full(len(toks), np.inf)
    P.forward(cfg, w, toks, layers_out=want, margins=margins)
    sure = margins >= (CLOSE_CALL_F32 if dtype == "float32" else CLOSE_CALL)      # tokens whose experts were chosen beyond doubt
    assert sure.sum() >= len(toks) // 2
    runner = runner_for(folder, dtype, use_graphs=False)
    got = []
    runner.model.tap = lambda i, h: got.append(h.detach().double().cpu())
    replay(runner, {"t": tuple(toks)}, [{"t": len(toks)}])
    assert len(got) == len(want) == len(cfg["layers"])
    tol = 2e-5 if dtype == "float32" else 6e-2
    for i, (a, b) in enumerate(zip(got, want)):
        err = float((a - torch.from_numpy(b)).abs()[sure].max() / np.abs(b).max())
        assert err <= tol, f"layer {i}: {err:.3e}"


# ------------------------------------------------------------------ the windows' edges, far keys and the sink, made to show

def _plain_sink_attention(q, k, v, scale, window, sink, H, G):
    T = q.shape[0]
    q, k, v = q.double().numpy(), k.double().numpy(), v.double().numpy()
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        out[:, h] = P.sink_softmax(q[:, h] @ k[:, g].T * scale, float(sink[h]), window) @ v[:, g]
    return torch.from_numpy(out.reshape(T, -1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,dk,dv,page,window,shared", [(6, 2, 16, 32, 8, 75, False), (4, 4, 32, 16, 16, 5, False),
                                                          (3, 1, 24, 24, 4, 130, True), (2, 1, 64, 64, 16, 64, True),
                                                          (5, 5, 16, 16, 8, 1, False), (2, 2, 16, 48, 8, None, False),
                                                          (7, 1, 48, 48, 16, 140, True), (3, 1, 112, 112, 8, None, True),
                                                          (2, 1, 20, 12, 8, 40, False)])
def test_window_edges_far_keys_and_the_sink_in_both_attention_kernels(H, G, dk, dv, page, window, shared, dtype):
    """The attention alone over scattered pages, with one key a query made to stand out: the key just inside the window,
    the key just outside it, a key far back and keys at the edges of the kernel's tiles of 64.  A key that is wrongly
    seen or wrongly missed takes or loses nearly all the weight.  The heads' sinks run from far below the scores (no
    weight) to above the largest score (most of the weight), so a sink that is left out, counted a run too often or
    scaled shows in every row.  ``shared``: keys and values are one pool.  Prompt portions (the matrix-core kernel where
    it takes the sizes, else the vector units) and single tokens with the keys cut into runs must both give the
    written-out softmax."""
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
    sink = torch.linspace(-30.0, 70.0, H) if H > 1 else torch.tensor([5.0])      # the standing-out score is about 80 * scale
    qd, kd = q.to(dtype), k.to(dtype)
    vd = kd if shared else torch.randn(T, G, dv, generator=g).to(dtype)
    want = _plain_sink_attention(qd.float(), kd.float(), vd.float(), scale, window, sink.double().numpy(), H, G)
    n_pages = (T + page - 1) // page
    perm = torch.randperm(n_pages + 5, generator=torch.Generator().manual_seed(1))[:n_pages]
    kpool = torch.full((n_pages + 5, G, page, dk), float("nan"), dtype=dtype)
    vpool = torch.full((n_pages + 5, G, page, dv), float("nan"), dtype=dtype)
    for t in range(T):
        kpool[perm[t // page], :, t % page] = kd[t]
        vpool[perm[t // page], :, t % page] = vd[t]
    kpool = kpool.to(dev)
    vpool = kpool if shared else vpool.to(dev)
    pages = perm.to(torch.int32).view(1, -1).to(dev)
    qrows = qd.reshape(T, H * dk).contiguous().to(dev)
    positions = torch.arange(T, dtype=torch.int32, device=dev)
    sink_dev = sink.to(dev)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    group = H // G

    def check(out, rows, what):
        err = float((out.double().cpu() - want[rows]).abs().max() / want.abs().max())
        assert err <= tol, f"{what}: {err:.3e}"

    for first in (0, 100, 203):
        n = T - first
        for wide in (True, False):
            rows_per = stream.bias_attention_mfma_rows(dk, dv, shared) if wide else stream.bias_attention_rows()
            if not rows_per:
                continue
            heads = min(group, rows_per)
            tile_tokens = max(1, rows_per // heads)
            tiles = torch.tensor(K.build_q_tiles([0], [n], [T], tile_tokens), dtype=torch.int32).view(-1, 4).to(dev)
            out = torch.empty(n, H * dv, dtype=dtype, device=dev)
            fn = stream.bias_attention_mfma if wide else stream.bias_attention
            fn(qrows[first:].contiguous(), kpool, vpool, pages, tiles, positions[first:].contiguous(), None, out, H, scale, 0.0, 0,
               heads, window=window, keep_first=0, sink=sink_dev)
            check(out, slice(first, T), f"portion from {first}, {'matrix cores' if wide else 'vector units'}")
    heads = min(group, stream.bias_attention_rows())
    for pos in (0, 1, win - 2, win - 1, win, win + 1, 63, 64, 65, 128, 200, 299):
        if not 0 <= pos < T:
            continue
        tiles = torch.tensor(K.build_q_tiles([0], [1], [pos + 1], 1), dtype=torch.int32).view(-1, 4).to(dev)
        for runs in (1, 3, 8):
            out = torch.empty(1, H * dv, dtype=dtype, device=dev)
            ws = torch.empty(H * runs * (dv + 2), dtype=torch.float32, device=dev) if runs > 1 else None
            stream.bias_attention(qrows[pos:pos + 1].contiguous(), kpool, vpool, pages, tiles, positions[pos:pos + 1].contiguous(), None,
                                  out, H, scale, 0.0, 0, heads, runs, ws, 4, window, 0, 1.0, sink=sink_dev)
            check(out, slice(pos, pos + 1), f"single token at {pos} in {runs} runs")


@pytest.mark.parametrize("dtype", DTYPES)
def test_sharp_windows_in_a_whole_model(dtype):
    """A model whose score factors are raised until single keys decide, with three windows (19, 23, and 66 on the keys of
    the layer with 19): prompts that end, portions that start and single tokens that fall just before, on and just
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


# ------------------------------------------------------------------ the kernels of the design alone

@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,G,dq,dk,dv,rot,at_q,at_k,normed,page", [(70, 4, 2, 16, 16, 8, 8, 0, 0, 16, 8), (3, 3, 3, 20, 20, 20, 20, 0, 0, 20, 4),
                                                                     (9, 5, 1, 12, 30, 0, 6, 6, 24, 24, 16), (130, 2, 1, 40, 136, 0, 32, 8, 104, 104, 8),
                                                                     (5, 6, 2, 10, 10, 14, 2, 0, 0, 10, 8)])
def test_norm_a_head_rotation_of_neighbours_and_the_store(T, H, G, dq, dk, dv, rot, at_q, at_k, normed, page, out):
    """Queries, keys and values out of one row of projections: a norm a head with one weight for all heads, of the keys
    only their first channels; the rotation of neighbouring pairs from a given channel on; the keys and values into
    scattered page slots.  Sizes of an attention layer (queries and keys alike, rotation of the first channels) and of a
    latent layer (one key head whose first channels are normed and whose last are rotated; query heads of another size
    rotated from their own offset; no values)."""
    from nanoinfer_amd.kernels import stream
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(T + dk)
    before, after = 3, 5                            # columns that belong to nobody, before and behind the projections
    wide = before + H * dq + G * dk + G * dv + after
    proj = torch.randn(T, wide, generator=g)
    wq, wk = 1.0 + 0.3 * torch.randn(dq, generator=g), 1.0 + 0.3 * torch.randn(normed, generator=g)
    freq = torch.rand(rot // 2, generator=g) * 0.5
    positions = torch.randint(0, 5000, (T,), generator=g).to(torch.int32)
    eps = 1e-5
    n_pages = (T + page - 1) // page + 3
    perm = torch.randperm(n_pages * page, generator=g)[:T].to(torch.int32)      # every token a slot of its own, anywhere
    kpool = torch.zeros(n_pages, G, page, dk, dtype=out, device=dev)
    vpool = torch.zeros(n_pages, G, page, dv, dtype=out, device=dev)
    q_out = torch.empty(T, H * dq, dtype=out, device=dev)
    with_q_norm = at_q == 0                        # the latent's queries are not normed
    stream.qk_norm_rope_store(proj.to(dev), positions.to(dev), perm.to(dev), wq.to(dev) if with_q_norm else None, wk.to(dev), eps,
                              freq.to(dev), 1.0, q_out, kpool, vpool, H, col=before, per_head=True, adjacent=True, q_dim=dq,
                              rot_at_q=at_q, rot_at_k=at_k, k_normed=normed)
    x = proj.double().numpy()
    pos = positions.numpy()
    q = x[:, before:before + H * dq].reshape(T, H, dq).copy()
    k = x[:, before + H * dq:before + H * dq + G * dk].reshape(T, G, dk).copy()
    v = x[:, before + H * dq + G * dk:before + H * dq + G * dk + G * dv].reshape(T, G, dv)
    if with_q_norm:
        q = P.rms(q, eps) * wq.double().numpy()
    k[..., :normed] = P.rms(k[..., :normed], eps) * wk.double().numpy()
    f = freq.double().numpy()
    q[..., at_q:at_q + rot] = P.rotate_pairs(q[..., at_q:at_q + rot], pos, f)
    k[..., at_k:at_k + rot] = P.rotate_pairs(k[..., at_k:at_k + rot], pos, f)
    tol = 1e-5 if out == torch.float32 else 1e-2
    # float32 angles of positions in the thousands are rounded before the sine: compare with angles rounded the same way
    f32 = (pos.astype(np.float32)[:, None] * freq.numpy()[None, :]).astype(np.float64)
    q32 = x[:, before:before + H * dq].reshape(T, H, dq).copy()
    if with_q_norm:
        q32 = P.rms(q32, eps) * wq.double().numpy()
    a, b = q32[..., at_q:at_q + rot:2].copy(), q32[..., at_q + 1:at_q + rot:2].copy()
    q32[..., at_q:at_q + rot:2] = a * np.cos(f32)[:, None] - b * np.sin(f32)[:, None]
    q32[..., at_q + 1:at_q + rot:2] = b * np.cos(f32)[:, None] + a * np.sin(f32)[:, None]
    assert float(np.abs(q_out.double().cpu().numpy().reshape(T, H, dq) - q32).max()) <= tol * float(np.abs(q32).max())
    assert float(np.abs(q32 - q).max()) <= 2e-3 * float(np.abs(q).max())          # and the exact angles are close by
    got_k = kpool.double().cpu().numpy().transpose(0, 2, 1, 3).reshape(n_pages * page, G, dk)[perm.long().numpy()]
    assert float(np.abs(got_k - k).max()) <= max(tol, 2e-3) * float(np.abs(k).max())
    if dv:
        got_v = vpool.double().cpu().numpy().transpose(0, 2, 1, 3).reshape(n_pages * page, G, dv)[perm.long().numpy()]
        assert float(np.abs(got_v - v).max()) <= tol * float(np.abs(v).max())
    # queries alone, from rows that hold nothing else (a layer that reads another's keys)
    alone = proj[:, before:before + H * dq].contiguous().to(dev)
    q2 = torch.empty_like(q_out)
    stream.qk_norm_rope_store(alone, positions.to(dev), None, wq.to(dev) if with_q_norm else None, None, eps, freq.to(dev), 1.0, q2,
                              None, None, H, per_head=True, adjacent=True, q_dim=dq, rot_at_q=at_q, queries_only=True)
    assert torch.equal(q2, q_out)


@pytest.mark.parametrize("E,top,groups,keep,scale", [(12, 3, 4, 2, 1.5), (8, 4, 4, 3, 1.0), (5, 1, 1, 1, 1.0), (6, 2, 6, 3, 0.5), (9, 4, 3, 2, 2.5),
                                                     (160, 6, 8, 3, 1.0), (64, 8, 1, 1, 1.0), (300, 5, 10, 4, 0.25)])
def test_the_router_with_sigmoid_scores_a_correction_and_groups_that_count_their_two_best(E, top, groups, keep, scale):
    """Experts chosen by ``sigmoid(z) + correction`` within the groups whose two best such scores sum highest, weighed by
    ``sigmoid(z) * scale``: against the plain router, for logits and corrections large enough to reorder the experts and
    negative enough for choice scores below zero."""
    from nanoinfer_amd import kernels as K
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(E * 7 + top)
    T = 97
    z = torch.randn(T, E, generator=g) * 2.0
    corr = torch.randn(E, generator=g) * 0.6 - 0.4
    mlp = {"router": {"experts": E, "top": top, "scale": scale, "groups": {"count": groups, "keep": keep}}}
    w = {"l0.mlp.router": np.eye(E), "l0.mlp.correction": corr.double().numpy()}
    want_chosen, want_w = P.route(z.double().numpy(), mlp, w, "l0.")
    chosen, mix, dense = K.route_top(z.to(dev), top, mix_all=True, groups=groups, keep=keep, scoring="sigmoid", correction=corr.to(dev),
                                     group_top=2, scale=scale)
    chosen, mix, dense = chosen.cpu().numpy(), mix.cpu().numpy(), dense.cpu().numpy()
    same = [t for t in range(T) if sorted(chosen[t]) == sorted(want_chosen[t])]
    assert len(same) >= T - 1                         # a close call between two float32 scores may fall the other way
    for t in same:
        assert chosen[t].tolist() == want_chosen[t].tolist()          # and in the order of their choice scores
        assert np.allclose(mix[t], want_w[t], rtol=2e-6, atol=1e-7)
        row = np.zeros(E)
        row[want_chosen[t]] = want_w[t]
        assert np.allclose(dense[t], row, rtol=2e-6, atol=1e-7)


def test_the_router_s_other_scorings_are_what_they_were():
    """The softmax among the chosen and the softmax over all experts, with groups that count their best expert."""
    from nanoinfer_amd import kernels as K
    dev = torch.device("cuda")
    z = torch.randn(50, 12, generator=torch.Generator().manual_seed(4)) * 3
    zd = z.double()
    for groups, keep in ((1, 1), (4, 2)):
        best = zd.view(50, groups, -1).max(dim=2).values
        kept = best.topk(keep, dim=1).indices
        open_ = torch.zeros(50, groups, dtype=torch.bool).scatter_(1, kept, True).repeat_interleave(12 // groups, dim=1)
        masked = torch.where(open_, zd, torch.full_like(zd, -math.inf))
        want = masked.topk(3, dim=1)
        for over_all in (False, True):
            chosen, mix, _ = K.route_top(z.to(dev), 3, mix_all=False, over_all=over_all, groups=groups, keep=keep)
            assert torch.equal(chosen.cpu().long(), want.indices)
            ref = torch.softmax(zd, dim=1).gather(1, want.indices) if over_all else torch.softmax(want.values, dim=1)
            assert torch.allclose(mix.cpu().double(), ref, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,ff,limit", [(1, 1, 40, 2.0), (70, 4, 24, 0.7), (9, 3, 37, 1.5)])
def test_capped_hidden_units(T, E, ff, limit, out):
    """``min(g, limit) * sigmoid(1.702 min(g, limit)) * (clamp(u, -limit, limit) + 1)`` over rows of [gate | up] an expert,
    with and without a weight an expert, for values on both sides of the limit."""
    from nanoinfer_amd import kernels as K
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(T + ff)
    up = (torch.randn(T, E * 2 * ff, generator=g) * 2.0).to(out)
    mix = torch.rand(T, E, generator=g)
    mix[:, 0] = 0.0 if E > 1 else 1.0
    x = up.double().view(T, E, 2, ff)
    gate, u = x[:, :, 0].clamp(max=limit), x[:, :, 1].clamp(-limit, limit)
    want = gate * torch.sigmoid(1.702 * gate) * (u + 1.0)
    tol = 1e-6 if out == torch.float32 else 8e-3
    got = K.experts_act(up.to(dev), None, ff, "capped_glu", limit, 1.702)
    assert float((got.double().cpu().view(T, E, ff) - want).abs().max()) <= tol * float(want.abs().max())
    got = K.experts_act(up.to(dev), mix.to(dev), ff, "capped_glu", limit, 1.702)
    weighed = want * mix.double()[:, :, None]
    assert float((got.double().cpu().view(T, E, ff) - weighed).abs().max()) <= tol * float(want.abs().max())


@pytest.mark.parametrize("T,d,n,alpha", [(1, 40, 0, 1.0), (9, 176, 1, 2.0), (70, 33, 2, 0.7), (300, 64, 2, 1.5), (4, 2048, 1, 2.0)])
def test_the_norm_behind_the_sum(T, d, n, alpha):
    """``h <- rmsnorm(alpha h + sum of addends) * w`` in place, and its copy in the compute type."""
    from nanoinfer_amd import kernels as K
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(T + d)
    h = torch.randn(T, d, generator=g)
    add = torch.randn(n, T, d, generator=g) if n else None
    w = 1.0 + 0.3 * torch.randn(d, generator=g)
    total = alpha * h.double() + (add.double().sum(0) if n else 0.0)
    want = total / (total.pow(2).mean(dim=1, keepdim=True) + 1e-5).sqrt() * w.double()
    for addends in ([add] if n != 1 else [add, add[0]]):
        hd = h.to(dev)
        x = torch.empty(T, d, dtype=torch.bfloat16, device=dev)
        K.post_norm(hd, None if addends is None else addends.to(dev), alpha, w.to(dev), 1e-5, x=x)
        assert float((hd.double().cpu() - want).abs().max()) <= 2e-6 * float(want.abs().max())
        assert torch.equal(x, hd.to(torch.bfloat16))


@pytest.mark.parametrize("T,H,dv,before", [(1, 3, 12, 24), (50, 6, 48, 128), (9, 1, 7, 5), (130, 5, 16, 0)])
def test_a_gate_a_head(T, H, dv, before):
    from nanoinfer_amd import kernels as K
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(T + H)
    rows = torch.randn(T, before + H + 3, generator=g)
    gate = torch.sigmoid(rows[:, before:before + H].double())
    o = torch.randn(H, T, dv, generator=g)
    want = (o.double().transpose(0, 1) * gate[:, :, None]).reshape(T, H * dv)
    got = K.gate_heads(o.to(dev), rows.to(dev), before, torch.float32, per_head=True)
    assert float((got.double().cpu() - want).abs().max()) <= 1e-6
    x = o.transpose(0, 1).reshape(T, H * dv).contiguous()
    got = K.gate_rows(x.to(dev), rows.to(dev), before, every=dv)
    assert float((got.double().cpu() - want).abs().max()) <= 1e-6


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
    """The latent layers' rotated key channels ride along when the heads' keys are written out: whole prompt, portions
    on both sides of the threshold in one sequence, a long portion beside single tokens."""
    name = "latent_wide"
    folder = folder_of(name)
    vocab = Z.ALL[name]["vocab"]
    requests = {"a": random_tokens(vocab, 150, 31), "b": random_tokens(vocab, 40, 32)}
    runner = runner_for(folder, dtype, page_size=page_size, use_graphs=False)
    got = replay(runner, requests, [{"a": 150}, {"b": 40}])
    assert written_out, "no step took the written-out way"
    for r, toks in requests.items():
        assert_close(got[r], plain(folder, toks), dtype, f"whole, request {r}")
    del written_out[:]
    got = replay(runner, requests, [{"a": 3, "b": 2}, {"a": 70, "b": 1}, {"a": 1, "b": 1}, {"a": 2, "b": 30}, {"a": 74, "b": 6}])
    assert written_out
    for r, toks in requests.items():
        assert_close(got[r], plain(folder, toks), dtype, f"in portions, request {r}")


# ------------------------------------------------------------------ generation through the framework's entry points

@pytest.mark.parametrize("name", ["mixed", "shared_kv"])
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
    assert all_pages_free(eng.runner.cache)


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


def test_the_command_line_generates_from_a_vimilix_folder(tmp_path, capsys):
    """``bin/nanoinfer``'s program with a Vimilix ``config.json``: the random-weights mode writes the folder, the engine
    generates greedily from two prompts, and the tokens are the plain implementation's."""
    from nanoinfer_amd import cli
    cfg_path, folder = str(tmp_path / "config.json"), str(tmp_path / "model")
    with open(cfg_path, "w") as fh:
        json.dump(Z.SHARED_KV, fh)
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
def test_the_trace_program_replays_a_vimilix_model(dtype, tmp_path):
    """``bin/trace_run`` in a process of its own, four slots: portions beside single tokens, a request that pauses, a
    fifth request on a slot and pages that another has given back."""
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
