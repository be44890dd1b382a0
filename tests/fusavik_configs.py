"""Small Fusavik configurations for the tests.  Between them every switch of the design is on and off, and sizes
that a model may happen to make equal or 1 (key and value size, heads and kv heads, rotated channels and head size,
groups kept, the loop's first layer) differ; several sizes are no multiples of anything."""


def rot(dims, base=10000.0, scaling=None):
    d = {"dims": dims, "base": base}
    if scaling is not None:
        d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return d


def left(heads, kv_heads, dim, vdim, scale, mask=None, rot=None):
    d = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if mask is not None:
        d["mask"] = {"size": mask[0], "keep_first": mask[1]}
    if rot is not None:
        d["rot"] = rot
    return d


def right(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def parallel(l, r, left_scale=1.0, right_scale=1.0):
    return {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": left_scale, "right_scale": right_scale}}


def scan(inner, state, dt_rank, conv):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}}


def moe(ff, experts, top, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        d["shared"] = {"ff": shared}
    return d


def model(width, vocab, layers, loop=None, bigram=None, scale=3.0, eps=1e-5):
    emb = {"scale": scale}
    if bigram is not None:
        emb["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}
    d = {"architecture": "Fusavik", "vocab": vocab, "width": width, "embedding": emb, "norm": {"eps": eps},
         "layers": [dict(mixer_entry, mlp=mlp) for mixer_entry, mlp in layers]}
    if loop is not None:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


# one mechanism at a time (the other half of a pair of mixers weighs nothing)
WINDOW_ONLY = model(64, 97, [(parallel(left(4, 2, 16, 24, 0.4, mask=(20, 3), rot=rot(8, 5000.0, (4.0, 64, 8.0, 1.0))),
                                       right(2, 8, 8, (0.5, 0.5)), 1.0, 0.0), None)])
WINDOW_PLAIN = model(48, 50, [(parallel(left(3, 3, 18, 10, 0.3), right(1, 8, 8, (0.5,)), 0.8, 0.0), None)])   # no mask, no rotation
DECAY_ONLY = model(64, 97, [(parallel(left(1, 1, 16, 16, 0.1), right(3, 24, 40, (0.9, 0.35, 0.999)), 0.0, 1.3), None)])
SCAN_ONLY = model(64, 97, [(scan(80, 6, 5, 4), None)])
SCAN_NO_CONV = model(40, 61, [(scan(48, 16, 16, 1), None)])
MOE_ONLY = model(64, 97, [(scan(32, 4, 4, 2), moe(24, 6, 2, groups=(3, 1), shared=40))])
MOE_PLAIN = model(64, 97, [(scan(32, 4, 4, 2), moe(20, 5, 1))])        # no groups, no shared expert, one expert chosen
BIGRAM = model(64, 97, [(scan(32, 4, 4, 2), None)], bigram=(53, 31, 7))

# everything at once: a loop in the middle, both mixers, a layer without a feed-forward
MIXED = model(96, 211, [(scan(72, 8, 6, 3), moe(16, 4, 4, shared=24)),
                        (parallel(left(6, 2, 16, 40, 0.3, mask=(37, 5), rot=rot(16, 300000.0, (8.0, 32, 16.0, 2.0))),
                                  right(3, 16, 32, (0.97, 0.6, 0.8)), 0.7, 1.1), moe(40, 6, 3, groups=(2, 1), shared=56)),
                        (scan(128, 32, 8, 4), None),
                        (parallel(left(5, 5, 24, 8, 0.2, mask=(9, 12), rot=rot(10, 100.0)), right(2, 20, 12, (0.5, 0.99)), 1.2, 0.4),
                         moe(32, 8, 3, groups=(4, 2)))],
              loop=(1, 3, 2), bigram=(61, 113, 5), scale=2.0)
# the loop from the first layer to the last, three passes; a group of more heads than a workgroup's rows; keys of 32
LOOP_ALL = model(80, 130, [(parallel(left(20, 1, 32, 32, 0.18, mask=(64, 1), rot=rot(32, 10000.0)), right(1, 64, 64, (0.9,)), 0.5, 0.5),
                            moe(32, 3, 1, shared=16)),
                           (scan(96, 12, 3, 2), moe(48, 4, 2, groups=(4, 2)))],
                 loop=(0, 2, 3), bigram=(17, 3, 5))

ALL = {"window_only": WINDOW_ONLY, "window_plain": WINDOW_PLAIN, "decay_only": DECAY_ONLY, "scan_only": SCAN_ONLY,
       "scan_no_conv": SCAN_NO_CONV, "moe_only": MOE_ONLY, "moe_plain": MOE_PLAIN, "bigram": BIGRAM, "mixed": MIXED,
       "loop_all": LOOP_ALL}
