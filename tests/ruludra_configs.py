"""Small Ruludra configurations for the tests.  Between them every mixer stands alone and beside the others, every
optional block of keys is on and off, and sizes that a model may happen to make equal or 1 (heads and kv heads, key
and value size, the ranks of the two latents, the windows of a layer and of the layer that reads its latents, the
gates' caps) differ; several sizes are no multiples of 4, 8 or 16."""


def keyed(heads, kv_heads, dim, scale, mask=None, temp=None):
    d = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if mask is not None:
        d["mask"] = {"size": mask}
    if temp is not None:
        d["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": d}


def latent(heads, dim, vdim, q_rank, kv_rank, scale, mask=None, kv_from=None):
    d = {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}
    if mask is not None:
        d["mask"] = {"size": mask}
    if kv_from is not None:
        d["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": d}


def memory(heads, dim, vdim, cap):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def model(width, vocab, layers, bigram=(53, 31, 7), eps=1e-5, logit_scale=0.5):
    emb = {}
    if bigram is not None:
        emb["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}
    return {"architecture": "Ruludra", "vocab": vocab, "width": width, "embedding": emb, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "layers": [dict(entry, mlp=None if ff is None else {"kind": "dense", "ff": ff}) for entry, ff in layers]}


# one mechanism at a time
KEYED_ONLY = model(64, 97, [(keyed(4, 2, 16, 0.3, mask=20, temp=(0.7, 8)), None)])
KEYED_PLAIN = model(48, 50, [(keyed(3, 3, 20, 0.25, mask=7), None)], bigram=None)            # heads of 20: the vector-unit kernel
KEYED_OPEN = model(40, 61, [(keyed(2, 1, 8, 0.4, temp=(0.3, 5)), None)])                      # no window
LATENT_ONLY = model(64, 97, [(latent(3, 8, 12, 24, 16, 1.5, mask=30), None)])
LATENT_OPEN = model(48, 50, [(latent(2, 10, 6, 9, 20, 1.2), 30)], bigram=None, logit_scale=1.0)   # no window; latent of 20: the vector units
MEMORY_ONLY = model(64, 97, [(memory(3, 12, 20, 6.0), None)])
MEMORY_WIDE = model(40, 61, [(memory(1, 40, 9, 30.0), None)])                                # a key of 40 on 8 lanes, a high cap
MLP_ONLY = model(56, 83, [(memory(1, 8, 8, 4.0), 50)], eps=1e-3)
# a layer reads the latents of another: other heads and sizes, a longer and a shorter window than the layer that writes
LATENT_SHARED = model(64, 97, [(latent(2, 8, 16, 20, 16, 1.5, mask=9), None), (memory(2, 8, 8, 8.0), None),
                               (latent(4, 12, 8, 12, 16, 1.1, mask=50, kv_from=0), 40),
                               (latent(1, 16, 16, 8, 16, 2.0, mask=3, kv_from=0), None)])
# latents wider than a head's keys and values together: long portions write the heads' keys and values out for the step
LATENT_WIDE = model(64, 97, [(latent(3, 8, 8, 24, 32, 1.5, mask=30), None), (memory(2, 8, 8, 8.0), None),
                             (latent(2, 4, 12, 12, 32, 1.1, mask=70, kv_from=0), 40), (latent(4, 8, 8, 16, 48, 0.9), None),
                             (latent(1, 16, 8, 8, 32, 2.0, mask=5, kv_from=0), None)])
# sizes that are multiples of nothing much: a width of 50, feed-forwards of 37 and 45, a vocabulary of 61
ODD_SIZES = model(50, 61, [(keyed(2, 1, 12, 0.3, mask=11, temp=(0.4, 3)), 37), (latent(2, 6, 10, 9, 14, 1.2, mask=17), 45),
                           (memory(1, 12, 9, 5.0), None), (latent(3, 4, 2, 7, 14, 1.4, kv_from=1), None)], bigram=(13, 5, 3))
# everything together
MIXED = model(72, 131, [(keyed(6, 2, 16, 0.3, mask=33, temp=(0.5, 16)), 90), (memory(2, 24, 32, 10.0), 44),
                        (latent(3, 16, 24, 40, 32, 1.3, mask=70), None), (keyed(2, 2, 24, 0.2, mask=130), None),
                        (latent(5, 8, 16, 24, 32, 1.6, mask=21, kv_from=2), 64), (memory(3, 16, 8, 3.5), None)])
# softmax that picks one key: whether the key at a window's edge is seen decides the output
SHARP = model(64, 97, [(keyed(4, 2, 16, 6.0, mask=19, temp=(0.5, 8)), None), (latent(2, 16, 16, 24, 16, 40.0, mask=23), None),
                       (latent(2, 16, 16, 24, 16, 40.0, mask=66, kv_from=1), None)])

ALL = {"keyed_only": KEYED_ONLY, "keyed_plain": KEYED_PLAIN, "keyed_open": KEYED_OPEN, "latent_only": LATENT_ONLY,
       "latent_open": LATENT_OPEN, "memory_only": MEMORY_ONLY, "memory_wide": MEMORY_WIDE, "mlp_only": MLP_ONLY,
       "latent_shared": LATENT_SHARED, "latent_wide": LATENT_WIDE, "odd_sizes": ODD_SIZES, "mixed": MIXED, "sharp": SHARP}
