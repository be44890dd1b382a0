"""``Zekalorn``: its configuration keys, its model as a list of parts, its tensor names.

A decoder whose layers each read ONE norm of the stream with both sublayers, ``x += mixer(n) + ff(n)``,
and then add a side input of the token itself.  Mixers are softmax attention (grouped heads, values of
their own size, a query temperature and a learned bias by distance in place of a rotation) or the gated
delta rule with a decay per key channel; feed-forwards are SwiGLU or routed squared-ReLU experts.  A run
of layers may be repeated with the same weights, every pass on a cache of its own and entered through a
learned vector.  The embedding scales its rows and adds a learned position row; the head is untied.
Tensor names: ``embed``, ``pos``, ``loop.step``, ``side.embed``, ``l<i>.norm1``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``l<i>.side.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.model_config import ConfigError
from ..config.spec import BlockSpec, LayerRun, ModelSpec, PartSpec
from ..config.zekalorn_config import ZekalornConfig, sizes_from_shapes
from ..registry import Architecture, register_architecture
from ..weights.random_init import InitRule


def _mixer(i: int, cfg: ZekalornConfig) -> PartSpec:
    m = cfg.layers[i].mixer
    pre = f"l{i}.mix."
    base = {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim, "value_dim": m.vdim}
    if m.type == "attention":
        names = {k: pre + k for k in ("q", "k", "v", "o")}
        if m.bias_max is not None:
            if m.bias_rows is None:
                raise ConfigError(f"layers[{i}]: the rows of the bias table are known from the tensor {pre}rel alone")
            names["bias"] = pre + "rel"
        return PartSpec("bias_attention", dict(base, scale=m.scale, bias_far=m.bias_max, bias_rows=m.bias_rows,
                                               temp_coef=m.q_temp_coef, temp_every=m.q_temp_every,
                                               max_positions=cfg.max_positions), names)
    if m.decay_rank is None or m.gate_rank is None:
        raise ConfigError(f"layers[{i}]: the ranks of the decay's and the gate's projections are known from the "
                          f"tensors {pre}a1 and {pre}g1 alone")
    names = {k: pre + k for k in ("q", "k", "v", "o", "A_log", "dt_bias", "norm")}
    names.update(q_conv=pre + "q.conv", k_conv=pre + "k.conv", v_conv=pre + "v.conv", beta=pre + "b",
                 decay_in=pre + "a1", decay_out=pre + "a2", gate_in=pre + "g1", gate_out=pre + "g2")
    return PartSpec("channel_delta", dict(base, taps=m.conv, decay_rank=m.decay_rank, gate_rank=m.gate_rank,
                                          eps=cfg.norm_eps), names)


def _feed_forward(i: int, cfg: ZekalornConfig):
    mlp = cfg.layers[i].mlp
    pre = f"l{i}.mlp."
    if mlp is None:
        return None
    if mlp.kind == "dense":
        return PartSpec("swiglu", {"hidden_size": cfg.width, "intermediate_size": mlp.ff},
                        {"gate": pre + "gate", "up": pre + "up", "down": pre + "down"})
    names = {"router": pre + "router"}
    for e in range(mlp.experts):
        names[f"up{e}"] = f"{pre}e{e}.up"
        names[f"down{e}"] = f"{pre}e{e}.down"
    return PartSpec("routed_experts", {"hidden_size": cfg.width, "expert_size": mlp.ff, "experts": mlp.experts,
                                       "top": mlp.top, "activation": "relu2"}, names)


def build_spec(cfg: ZekalornConfig) -> ModelSpec:
    d, L = cfg.width, len(cfg.layers)
    blocks = []
    for i in range(L):
        parts = {"norm": PartSpec("rmsnorm", {"size": d, "eps": cfg.norm_eps}, {"weight": f"l{i}.norm1"}),
                 "mixer": _mixer(i, cfg)}
        ff = _feed_forward(i, cfg)
        if ff is not None:
            parts["ffn"] = ff
        if cfg.side_dim is not None:
            parts["side"] = PartSpec("gated_side_rows", {"hidden_size": d, "size": cfg.side_dim, "first": i * cfg.side_dim,
                                                         "table_cols": L * cfg.side_dim, "vocab_size": cfg.vocab,
                                                         "eps": cfg.norm_eps},
                                     {"table": "side.embed", "gate": f"l{i}.side.gate", "proj": f"l{i}.side.proj",
                                      "norm": f"l{i}.side.norm"})
        blocks.append(BlockSpec(kind="parallel", parts=parts))
    # the order: the layers before the loop, the looped run once for every pass (each pass on caches of its own,
    # entered through its row of the pass vectors), the layers behind it
    order, pass_input = [], None
    if cfg.loop is None:
        order = [LayerRun(block=i, cache=i) for i in range(L)]
    else:
        lp = cfg.loop
        runs = [(i, None) for i in range(lp.start)]
        for p in range(lp.times):
            runs += [(i, p if i == lp.start else None) for i in range(lp.start, lp.stop)]
        runs += [(i, None) for i in range(lp.stop, L)]
        order = [LayerRun(block=i, cache=n, enter=p) for n, (i, p) in enumerate(runs)]
        pass_input = PartSpec("vector_rows", {"rows": lp.times, "size": d}, {"table": "loop.step"})
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=d, max_positions=cfg.max_positions,
        embedding=PartSpec("scaled_table", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": cfg.embedding_scale,
                                            "max_positions": cfg.max_positions},
                           {"weight": "embed", "positions": "pos"}),
        blocks=blocks, order=order,
        final_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.norm_eps}, {"weight": "final.norm"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d}, {"weight": "head"}),
        pass_input=pass_input,
    )


ZEKALORN = register_architecture(Architecture(
    name="Zekalorn",
    config_from_dict=ZekalornConfig.from_dict,
    build_spec=build_spec,
    init=InitRule(matrix_std=0.05, vector_mean=1.0, vector_std=0.05,
                  overrides=(("A_log", -1.0, 0.5), ("dt_bias", 0.0, 0.5), (".conv", 0.0, 0.4), ("pos", 0.0, 0.3),
                             ("loop.step", 0.0, 0.3), ("side.embed", 0.0, 1.0), (".rel", 0.0, 0.5), ("embed", 0.0, 0.08))),
    sizes_from_shapes=sizes_from_shapes,
))
