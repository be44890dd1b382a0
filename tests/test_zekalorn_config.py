"""Zekalorn on the CPU: how ``config.json`` is read, what the model looks like as data, and a few
properties of the plain implementation that do not need the engine."""
import math

import pytest
import torch

import nanoinfer_amd  # noqa: F401
import plain_zekalorn as P
import zekalorn_configs as Z
from nanoinfer_amd.config.model_config import ConfigError
from nanoinfer_amd.config.zekalorn_config import ZekalornConfig, sizes_from_shapes
from nanoinfer_amd.registry import architecture_of
from nanoinfer_amd.weights.loader import expected_tensors, make_random_model, read_model_folder


def test_the_architecture_is_chosen_by_a_string_or_a_list():
    assert architecture_of({"architecture": "Zekalorn"}).name == "Zekalorn"
    assert architecture_of({"architectures": ["Zekalorn"]}).name == "Zekalorn"


@pytest.mark.parametrize("name", sorted(Z.ALL))
def test_configuration_round_trip(name):
    cfg = ZekalornConfig.from_dict(Z.ALL[name])
    again = ZekalornConfig.from_dict(cfg.to_dict())
    assert again == cfg


def test_missing_keys_are_named():
    for path in (("width",), ("embedding", "scale"), ("norm", "eps"), ("layers", 0, "mixer", "heads"), ("loop", "times")):
        d = ZekalornConfig.from_dict(Z.MIXED).to_dict()
        at = d
        for p in path[:-1]:
            at = at[p]
        del at[path[-1]]
        with pytest.raises(ConfigError, match=str(path[-1])):
            ZekalornConfig.from_dict(d)
    bad = ZekalornConfig.from_dict(Z.MIXED).to_dict()
    bad["loop"] = {"start": 2, "stop": 9, "times": 2}
    with pytest.raises(ConfigError, match="loop"):
        ZekalornConfig.from_dict(bad)
    bad = ZekalornConfig.from_dict(Z.MIXED).to_dict()
    bad["layers"][0]["type"] = "mystery"
    with pytest.raises(ConfigError, match="mystery"):
        ZekalornConfig.from_dict(bad)


def test_the_order_of_a_looped_model_and_its_caches():
    arch = architecture_of(Z.MIXED)
    spec = arch.build_spec(arch.config_from_dict(Z.MIXED))
    assert [(r.block, r.enter) for r in spec.order] == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    assert [r.cache for r in spec.order] == list(range(6))          # every pass has caches of its own
    assert spec.pass_input is not None and spec.pass_input.params["rows"] == 2
    spec = arch.build_spec(arch.config_from_dict(Z.LOOP_ALL))
    assert [(r.block, r.enter) for r in spec.order] == [(0, 0), (1, None), (0, 1), (1, None), (0, 2), (1, None)]
    spec = arch.build_spec(arch.config_from_dict(Z.DELTA_ONLY))
    assert spec.pass_input is None and [r.enter for r in spec.order] == [None]
    assert "ffn" not in spec.blocks[0].parts and "side" not in spec.blocks[0].parts


def test_sizes_that_only_shapes_give_are_read_from_the_checkpoint(tmp_path):
    folder = make_random_model(str(tmp_path / "m"), Z.MIXED, 1, dtype="bfloat16")
    import json
    import os
    with open(os.path.join(folder, "config.json")) as fh:
        raw = json.load(fh)
    for layer in raw["layers"]:                      # a configuration as another exporter writes it: no such keys
        for key in ("decay_rank", "gate_rank", "bias_rows"):
            layer["mixer"].pop(key, None)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(raw, fh)
    arch, cfg, spec = read_model_folder(folder)
    assert cfg.layers[0].mixer.decay_rank == 6 and cfg.layers[0].mixer.gate_rank == 9
    assert cfg.layers[1].mixer.bias_rows == 10 and cfg.layers[3].mixer.bias_rows == 8
    want = expected_tensors(spec)
    assert want["l2.mix.a2"] == (2 * 48, 16) and want["l1.mix.rel"] == (10, 6) and want["loop.step"] == (2, 96)
    assert want["side.embed"] == (211, 4 * 12) and "l3.mlp.router" not in want
    bare = ZekalornConfig.from_dict(raw)
    with pytest.raises(ConfigError, match="a1"):
        arch.build_spec(bare)
    assert sizes_from_shapes(bare, {}) == bare


def test_a_cache_group_keeps_keys_and_values_of_their_own_sizes():
    from nanoinfer_amd.cache.manager import KVCacheManager
    from nanoinfer_amd.parts.base import CacheNeed, KVNeed, StateNeed
    needs = {0: CacheNeed(kv=KVNeed(2, 16, None, 40)), 1: CacheNeed(state=StateNeed((7,))), 2: CacheNeed(kv=KVNeed(2, 16, None, 40))}
    m = KVCacheManager(needs, page_size=4, num_pages=6, max_requests=2, dtype=torch.float32, device=torch.device("cpu"))
    assert len(m.groups) == 1 and m.groups[0].kpools[0].shape == (6, 2, 4, 16) and m.groups[0].vpools[2].shape == (6, 2, 4, 40)
    assert m.pool_bytes() == 2 * 6 * 2 * 4 * (16 + 40) * 4
    assert KVCacheManager.pages_for_bytes(needs, 4, m.pool_bytes(), torch.float32) == 6
    assert m.state[1].shape == (2, 7)
    assert m.reserve("a", 9) and m.reserve("b", 3) and not m.reserve("c", 1)
    m.state[1][m.state_slot("a")] = 5.0
    m.release("a")
    assert m.reserve("c", 1) and float(m.state[1][m.state_slot("c")].abs().max()) == 0.0      # a slot starts empty


# ------------------------------------------------------------------ the plain implementation itself

def test_the_plain_convolution_is_a_causal_correlation():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(9, 5, generator=g, dtype=torch.float64)
    taps = torch.randn(5, 3, generator=g, dtype=torch.float64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.t()[None], (2, 0)), taps[:, None, :], groups=5)[0].t()
    assert torch.allclose(P.short_conv(x, taps), want)


def test_the_plain_delta_rule_recalls_what_it_stored():
    """With no decay and beta 1, a key that was written once returns its value: o = S^T k = v."""
    dk, dv = 6, 4
    k = torch.zeros(dk, dtype=torch.float64)
    k[2] = 1.0
    v = torch.arange(1.0, dv + 1, dtype=torch.float64)
    S = torch.zeros(dk, dv, dtype=torch.float64)
    u = 1.0 * (v - S.t() @ k)
    S = S + torch.outer(k, u)
    assert torch.allclose(S.t() @ k, v)
    u = 1.0 * (2 * v - S.t() @ k)                    # written again: replaced, not added
    S = S + torch.outer(k, u)
    assert torch.allclose(S.t() @ k, 2 * v)


def test_plain_buckets_and_temperature():
    assert [P.distance_bucket(n, 8, 64.0) for n in (0, 3, 4, 7, 8, 15, 16, 63, 64, 1000)] == [0, 3, 4, 4, 5, 5, 6, 7, 7, 7]
    assert P.query_temperature(0, 0.5, 4) == 1.0 and P.query_temperature(3, 0.5, 4) == 1.0 + 0.5 * math.log(2)


def test_plain_routing_with_all_experts_chosen_is_a_full_softmax():
    g = torch.Generator().manual_seed(1)
    d, ff, E = 6, 5, 3
    w = {"router": torch.randn(E, d, generator=g)}
    for e in range(E):
        w[f"e{e}.up"] = torch.randn(ff, d, generator=g)
        w[f"e{e}.down"] = torch.randn(d, ff, generator=g)
    n = torch.randn(2, d, generator=g)
    mix = torch.softmax(P.linear(n, w["router"]), dim=-1)
    want = sum(mix[:, e:e + 1] * P.linear(torch.relu(P.linear(n, w[f"e{e}.up"])) ** 2, w[f"e{e}.down"]) for e in range(E))
    assert torch.allclose(P.routed_ff(n, w, E, E), want)


@pytest.mark.parametrize("shape", ["1b", "3b", "8b"])
def test_the_bench_shapes_are_valid_configurations(shape):
    """``bench.py --workload hybrid --shape ...`` writes a Zekalorn model with the layer sizes of that Llama shape."""
    import bench
    like = bench.SHAPES[shape][2]
    d = bench.hybrid_config(8, 1000, 4096, like)
    cfg = ZekalornConfig.from_dict(d)
    spec = architecture_of(d).build_spec(cfg)
    assert len(spec.order) == 8
    mixers = [layer["type"] for layer in d["layers"]]
    assert mixers.count("attention") == 2 and mixers.count("channel_delta") == 6
    attn = next(layer["mixer"] for layer in d["layers"] if layer["type"] == "attention")
    assert attn["heads"] == like["num_attention_heads"] and attn["dim"] == like["head_dim"]
