"""Small Vimilix configurations for the tests.  Between them every mixer stands alone and beside the other, every
optional block of keys is on and off, and sizes that a model may happen to make equal or 1 (heads and kv heads, key
and value size, rotated and all channels of a head, the windows of a layer and of the layer that reads its keys,
groups and experts, kept groups and all groups, the experts' and the shared expert's limits) differ; several sizes
are no multiples of 4, 8 or 16."""


def rot(dims, base, scaling=None):
    d = {"base": base, "dims": dims}
    if scaling is not None:
        d["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return d


def sink(heads, kv_heads, dim, vdim, scale, rot_, mask=None, kv_from=None):
    d = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot_}
    if mask is not None:
        d["mask"] = {"size": mask}
    if kv_from is not None:
        d["kv_from"] = kv_from
    return {"type": "attention", "mixer": d}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, mask=None, scaling=None):
    d = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": rot(rot_dim, base, scaling)}
    if mask is not None:
        d["mask"] = {"size": mask}
    return {"type": "latent_attention", "mixer": d}


def moe(experts, top, ff, limit, scale=1.0, groups=None, shared=None):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}
    if shared is not None:
        d["shared"] = {"ff": shared[0], "limit": shared[1]}
    return d


def model(width, vocab, layers, alpha=1.5, eps=1e-5):
    return {"architecture": "Vimilix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha,
            "layers": [dict(entry, mlp=mlp) for entry, mlp in layers]}


LONG_WAVES = (4.0, 1.0, 3.0, 64)        # (factor, low, high, original): waves from 21 to 64 positions are blended

# one mechanism at a time
SINK_ONLY = model(64, 97, [(sink(6, 2, 16, 8, 0.3, rot(8, 300.0, LONG_WAVES), mask=20), None)])
SINK_OPEN = model(48, 50, [(sink(3, 3, 20, 20, 0.25, rot(20, 10000.0)), None)], alpha=0.7)       # no window; heads of 20: the vector units
LATENT_ONLY = model(64, 97, [(latent(3, 8, 8, 12, 24, 0.35, base=500.0), None)])                 # rows of 32: the matrix cores
LATENT_ODD = model(48, 50, [(latent(2, 10, 6, 7, 20, 0.3, mask=30, scaling=LONG_WAVES), None)], alpha=2.5)   # rows of 26, a window
MOE_ONLY = model(56, 83, [(latent(1, 8, 4, 8, 12, 0.3), moe(12, 3, 24, 1.25, scale=1.5, groups=(4, 2), shared=(40, 2.0)))], eps=1e-3)
MOE_FLAT = model(40, 61, [(sink(2, 1, 8, 8, 0.4, rot(4, 100.0), mask=9), moe(5, 1, 17, 0.8))])    # no groups, no shared expert, one expert a token
MOE_SINGLES = model(40, 61, [(sink(2, 2, 8, 12, 0.4, rot(8, 100.0)), moe(6, 2, 16, 3.0, scale=0.5, groups=(6, 3), shared=(8, 0.5)))])   # groups of one expert
# layers read the keys and values of another: other query heads, a longer and a shorter window than the layer that writes
SHARED_KV = model(64, 97, [(sink(4, 2, 16, 8, 0.3, rot(8, 300.0, LONG_WAVES), mask=9), None),
                           (latent(2, 8, 4, 8, 12, 0.3), None),
                           (sink(2, 2, 16, 8, 0.25, rot(8, 300.0, LONG_WAVES), mask=50, kv_from=0), moe(4, 2, 16, 1.0, groups=(2, 1))),
                           (sink(6, 2, 16, 8, 0.35, rot(8, 300.0, LONG_WAVES), mask=3, kv_from=0), None)])
# a reader without a window on pages whose writer has one: the pages keep everything
SHARED_OPEN = model(48, 50, [(sink(2, 1, 16, 16, 0.3, rot(16, 1000.0), mask=5), None),
                             (sink(2, 1, 16, 16, 0.3, rot(16, 1000.0), kv_from=0), None)])
# latents wider than a head's keys and values together: long portions write the heads' keys and values out for the step
LATENT_WIDE = model(64, 97, [(latent(3, 8, 8, 8, 40, 0.3, mask=70), None), (latent(2, 4, 4, 12, 28, 0.4), moe(4, 2, 16, 1.0)),
                             (latent(4, 8, 16, 8, 48, 0.25, mask=5), None)])
# a latent of more channels than the attention kernels take as values: every step writes the heads' keys and values out
LATENT_HUGE = model(64, 97, [(latent(2, 8, 16, 8, 272, 0.3), moe(4, 2, 16, 1.0)), (latent(3, 16, 4, 8, 300, 0.25, mask=40), None)])
# sizes that are multiples of nothing much: a width of 50, experts of 37 and 45, a vocabulary of 61
ODD_SIZES = model(50, 61, [(sink(2, 1, 12, 10, 0.3, rot(6, 77.0), mask=11), moe(6, 2, 37, 1.1, groups=(3, 2), shared=(45, 1.7))),
                           (latent(2, 6, 2, 10, 14, 0.3, mask=17), moe(3, 3, 9, 2.0)),
                           (sink(4, 1, 12, 10, 0.2, rot(6, 77.0), kv_from=0), None)], alpha=0.9)
# everything together
MIXED = model(72, 131, [(latent(3, 16, 16, 24, 32, 0.2, base=2000.0), moe(8, 3, 24, 1.5, scale=1.25, groups=(4, 3), shared=(40, 2.0))),
                        (sink(6, 2, 16, 24, 0.3, rot(8, 5000.0, (8.0, 1.0, 4.0, 128)), mask=33), moe(6, 2, 32, 1.0, shared=(16, 1.0))),
                        (latent(5, 8, 8, 16, 40, 0.3, mask=70), None),
                        (sink(4, 2, 16, 24, 0.25, rot(8, 5000.0, (8.0, 1.0, 4.0, 128)), mask=130, kv_from=1),
                         moe(9, 4, 16, 2.0, scale=0.75, groups=(3, 2)))], alpha=1.75)
# softmax that picks one key: whether the key at a window's edge is seen decides the output
SHARP = model(64, 97, [(sink(4, 2, 16, 16, 6.0, rot(8, 100.0), mask=19), None), (latent(2, 16, 8, 16, 24, 5.0, mask=23), None),
                       (sink(2, 2, 16, 16, 6.0, rot(8, 100.0), mask=66, kv_from=0), None)])

ALL = {"sink_only": SINK_ONLY, "sink_open": SINK_OPEN, "latent_only": LATENT_ONLY, "latent_odd": LATENT_ODD, "moe_only": MOE_ONLY,
       "moe_flat": MOE_FLAT, "moe_singles": MOE_SINGLES, "shared_kv": SHARED_KV, "shared_open": SHARED_OPEN, "latent_wide": LATENT_WIDE, "latent_huge": LATENT_HUGE,
       "odd_sizes": ODD_SIZES, "mixed": MIXED, "sharp": SHARP}
