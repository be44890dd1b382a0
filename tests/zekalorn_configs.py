"""Small Zekalorn configurations for the tests.  Between them every switch of the design is on and off,
and sizes that a model may happen to make equal (key and value size, heads and kv heads, top and 1) differ."""


def attention(heads, kv_heads, dim, vdim, scale, bias_max=None, q_temp=None, bias_rows=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if bias_max is not None:
        m.update(bias_max=bias_max, bias_rows=bias_rows)
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m}


def delta(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                                               "decay_rank": decay_rank, "gate_rank": gate_rank}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def model(width, vocab, layers, loop=None, side=None, max_positions=512, scale=3.0, eps=1e-5):
    d = {"architecture": "Zekalorn", "vocab": vocab, "width": width, "max_positions": max_positions,
         "embedding": {"scale": scale}, "norm": {"eps": eps},
         "layers": [dict(mixer_entry, mlp=mlp) for mixer_entry, mlp in layers]}
    if loop is not None:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if side is not None:
        d["token_side"] = {"dim": side}
    return d


# one mechanism at a time
ATTENTION_ONLY = model(64, 97, [(attention(4, 2, 16, 24, 0.5, bias_max=40.0, q_temp=(0.5, 8), bias_rows=12), None)])
ATTENTION_PLAIN = model(48, 50, [(attention(3, 3, 18, 10, 0.25), None)])     # sizes that are no whole 16-byte pieces
DELTA_ONLY = model(64, 97, [(delta(4, 2, 16, 24, 3, 8, 12), None)])
DELTA_NO_CONV = model(40, 61, [(delta(2, 1, 20, 8, 1, 5, 7), None)])
DENSE_FF = model(64, 97, [(attention(2, 1, 32, 32, 0.2), dense(88))])
ROUTED_FF = model(64, 97, [(attention(2, 1, 32, 32, 0.2), moe(24, 5, 2))])
SIDE_INPUT = model(64, 97, [(attention(2, 1, 32, 32, 0.2), None)], side=10)

# everything at once: a loop in the middle, both mixers, both feed-forwards, a layer without one, side input
MIXED = model(96, 211, [(delta(3, 1, 32, 16, 4, 6, 9), dense(72)),
                        (attention(6, 2, 16, 40, 0.3, bias_max=100.0, q_temp=(0.4, 16), bias_rows=10), moe(40, 6, 3)),
                        (delta(2, 2, 48, 32, 2, 16, 16), moe(16, 4, 4)),
                        (attention(5, 5, 24, 8, 0.2, bias_max=30.0, bias_rows=8), None)],
              loop=(1, 3, 2), side=12, max_positions=700)
# the loop from the first layer to the last, one expert chosen, a group of more heads than a workgroup's rows
LOOP_ALL = model(80, 130, [(attention(20, 1, 16, 16, 0.25, q_temp=(0.2, 4)), moe(32, 3, 1)),
                           (delta(4, 4, 16, 16, 3, 4, 4), dense(48))],
                 loop=(0, 2, 3), side=None, max_positions=400)

ALL = {"attention_only": ATTENTION_ONLY, "attention_plain": ATTENTION_PLAIN, "delta_only": DELTA_ONLY,
       "delta_no_conv": DELTA_NO_CONV, "dense_ff": DENSE_FF, "routed_ff": ROUTED_FF, "side_input": SIDE_INPUT,
       "mixed": MIXED, "loop_all": LOOP_ALL}
