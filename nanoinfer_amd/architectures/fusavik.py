"""``Fusavik``: its configuration keys, its model as a list of parts, its tensor names.

A decoder of pre-norm layers, ``x += mixer(norm1(x)); x += ff(norm2(x))``.  A mixer is either two mixers side by
side on the same input (softmax attention in a window that keeps the sequence's first tokens in sight, with a norm
over the whole query and key projections and a partial rotation stretched for long contexts; and linear attention
with one decay a head and a gated norm), or a selective scan.  A feed-forward is a set of routed gated experts
chosen within the best groups, weighed by the softmax over all experts, plus one expert every token uses; a layer
may have none.  A run of layers may be repeated with the same weights, every pass on a cache of its own, entered
through a learned vector and (from the second pass on) the embedding's output added again.  The embedding scales
its rows and adds a row of a second table read by a hash of the pair (token before, token); the head is untied.
Tensor names: ``embed``, ``bigram``, ``loop.step``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``final.norm``, ``head``.  The design names no last position.
"""
from __future__ import annotations

import math

from ..config.fusavik_config import FusavikConfig, ParallelMixerConfig, ScanMixerConfig
from ..config.spec import BlockSpec, LayerRun, ModelSpec, PartSpec
from ..registry import Architecture, register_architecture
from ..weights.random_init import InitRule

# positions are counted in int32 and turned into float32 angles: beyond 2^24 a float32 no longer holds every position
POSITIONS = 1 << 24


def _mixer(i: int, cfg: FusavikConfig) -> PartSpec:
    m = cfg.layers[i].mixer
    d, pre = cfg.width, f"l{i}.mix."
    if isinstance(m, ScanMixerConfig):
        names = {k: pre + k for k in ("in", "conv", "x", "dt", "A_log", "D", "o")}
        names.update(conv_b=pre + "conv.b", dt_b=pre + "dt.b")
        return PartSpec("selective_scan", {"hidden_size": d, "inner": m.inner, "state": m.state, "dt_rank": m.dt_rank,
                                           "taps": m.conv}, names)
    assert isinstance(m, ParallelMixerConfig)
    a, b = m.left, m.right
    position = None
    if a.rot is not None:
        scaling, amplitude = None, 1.0
        if a.rot.scaling is not None:
            factor, original, fast, slow = a.rot.scaling
            scaling = {"kind": "yarn", "factor": factor, "original": original, "fast": fast, "slow": slow,
                       "dims": a.rot.dims, "base": a.rot.base}
            amplitude = 0.1 * math.log(factor) + 1.0
        position = PartSpec("rope", {"rotary_dim": a.rot.dims, "theta": a.rot.base, "max_positions": None, "scaling": scaling,
                                     "amplitude": amplitude, "exact": True})
    left = PartSpec("window_attention",
                    {"hidden_size": d, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "key_dim": a.dim, "value_dim": a.vdim,
                     "scale": a.scale, "window": a.window, "keep_first": a.keep_first, "qk_norm": True, "eps": cfg.norm_eps,
                     "position": position, "out_scale": m.left_scale},
                    {"q": pre + "left.q", "k": pre + "left.k", "v": pre + "left.v", "o": pre + "left.o",
                     "q_norm": pre + "left.q.norm", "k_norm": pre + "left.k.norm"})
    right = PartSpec("decay_attention",
                     {"hidden_size": d, "num_heads": b.heads, "key_dim": b.dim, "value_dim": b.vdim, "decay": list(b.decay),
                      "eps": cfg.norm_eps, "out_scale": m.right_scale},
                     {k: pre + "right." + k for k in ("q", "k", "v", "g", "o", "norm")})
    return PartSpec("side_by_side", {"hidden_size": d, "left": left, "right": right})


def _feed_forward(i: int, cfg: FusavikConfig):
    mlp = cfg.layers[i].mlp
    if mlp is None:
        return None
    d, pre = cfg.width, f"l{i}.mlp."
    names = {"router": pre + "router"}
    for e in range(mlp.experts):
        names.update({f"gate{e}": f"{pre}e{e}.gate", f"up{e}": f"{pre}e{e}.up", f"down{e}": f"{pre}e{e}.down"})
    shared = None
    if mlp.shared_ff is not None:
        shared = PartSpec("swiglu", {"hidden_size": d, "intermediate_size": mlp.shared_ff},
                          {"gate": pre + "shared.gate", "up": pre + "shared.up", "down": pre + "shared.down"})
    return PartSpec("routed_experts", {"hidden_size": d, "expert_size": mlp.ff, "experts": mlp.experts, "top": mlp.top,
                                       "activation": "swiglu", "mix": "softmax_all", "groups": mlp.group_count,
                                       "keep": mlp.group_keep, "shared": shared}, names)


def build_spec(cfg: FusavikConfig) -> ModelSpec:
    d, L = cfg.width, len(cfg.layers)
    blocks = []
    for i in range(L):
        parts = {"mixer_norm": PartSpec("rmsnorm", {"size": d, "eps": cfg.norm_eps}, {"weight": f"l{i}.norm1"}),
                 "mixer": _mixer(i, cfg)}
        ff = _feed_forward(i, cfg)
        if ff is not None:
            parts["ffn_norm"] = PartSpec("rmsnorm", {"size": d, "eps": cfg.norm_eps}, {"weight": f"l{i}.norm2"})
            parts["ffn"] = ff
        blocks.append(BlockSpec(kind="prenorm", parts=parts))
    # the order: the layers before the loop, the looped run once for every pass (each pass on caches of its own,
    # entered through its row of the pass vectors), the layers behind it
    pass_input = None
    if cfg.loop is None:
        order = [LayerRun(block=i, cache=i) for i in range(L)]
    else:
        lp = cfg.loop
        runs = [(i, None) for i in range(lp.start)]
        for p in range(lp.times):
            runs += [(i, p if i == lp.start else None) for i in range(lp.start, lp.stop)]
        runs += [(i, None) for i in range(lp.stop, L)]
        order = [LayerRun(block=i, cache=n, enter=p) for n, (i, p) in enumerate(runs)]
        pass_input = PartSpec("vector_rows", {"rows": lp.times, "size": d, "again": True}, {"table": "loop.step"})
    if cfg.bigram is not None:
        embedding = PartSpec("pair_hash_table", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": cfg.embedding_scale,
                                                 "buckets": cfg.bigram.buckets, "mul_prev": cfg.bigram.mul_prev,
                                                 "mul_cur": cfg.bigram.mul_cur}, {"weight": "embed", "pairs": "bigram"})
    else:
        embedding = PartSpec("scaled_table", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": cfg.embedding_scale,
                                              "max_positions": POSITIONS}, {"weight": "embed"})
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=d, max_positions=POSITIONS, embedding=embedding, blocks=blocks, order=order,
        final_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.norm_eps}, {"weight": "final.norm"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d}, {"weight": "head"}),
        pass_input=pass_input,
        ignorable_suffixes=(".norm2",),      # a layer without a feed-forward has no use for its second norm's weight
    )


FUSAVIK = register_architecture(Architecture(
    name="Fusavik",
    config_from_dict=FusavikConfig.from_dict,
    build_spec=build_spec,
    init=InitRule(matrix_std=0.05, vector_mean=1.0, vector_std=0.05,
                  overrides=(("A_log", 0.0, 0.5), ("dt.b", -1.0, 0.5), (".conv", 0.0, 0.4), ("conv.b", 0.0, 0.1), (".D", 1.0, 0.2),
                             ("loop.step", 0.0, 0.3), ("bigram", 0.0, 0.5), ("embed", 0.0, 0.08), (".dt", 0.0, 0.2))),
))
