"""Fusavik's configuration reader and model description, on the CPU: every key is read, what is absent switches
its mechanism off, what does not fit is refused by name, and the spec asks for the tensors the design names."""
import copy

import numpy as np
import pytest

import fusavik_configs as Z
import plain_fusavik as P
import nanoinfer_amd  # noqa: F401
from nanoinfer_amd.config.model_config import ConfigError
from nanoinfer_amd.registry import architecture_of
from nanoinfer_amd.weights.loader import expected_tensors


def spec_of(cfg_json):
    arch = architecture_of(cfg_json)
    cfg = arch.config_from_dict(cfg_json)
    return arch, cfg, arch.build_spec(cfg)


@pytest.mark.parametrize("name", sorted(Z.ALL))
def test_configuration_round_trip_and_tensor_names(name):
    arch, cfg, spec = spec_of(Z.ALL[name])
    assert arch.name == "Fusavik" and cfg.to_dict() == Z.ALL[name]
    want = expected_tensors(spec)
    d = cfg.width
    assert want["embed"] == (cfg.vocab, d) and want["head"] == (cfg.vocab, d) and want["final.norm"] == (d,)
    for i, layer in enumerate(Z.ALL[name]["layers"]):
        m = layer["mixer"]
        if layer["type"] == "parallel":
            a, b = m["left"], m["right"]
            assert want[f"l{i}.mix.left.q"] == (a["heads"] * a["dim"], d) and want[f"l{i}.mix.left.q.norm"] == (a["heads"] * a["dim"],)
            assert want[f"l{i}.mix.left.k.norm"] == (a["kv_heads"] * a["dim"],) and want[f"l{i}.mix.left.v"] == (a["kv_heads"] * a["vdim"], d)
            assert want[f"l{i}.mix.left.o"] == (d, a["heads"] * a["vdim"])
            assert want[f"l{i}.mix.right.k"] == (b["heads"] * b["dim"], d) and want[f"l{i}.mix.right.g"] == (b["heads"] * b["vdim"], d)
            assert want[f"l{i}.mix.right.norm"] == (b["heads"] * b["vdim"],)
        else:
            assert want[f"l{i}.mix.in"] == (2 * m["inner"], d) and want[f"l{i}.mix.x"] == (m["dt_rank"] + 2 * m["state"], m["inner"])
            assert want[f"l{i}.mix.conv"] == (m["inner"], m["conv"]) and want[f"l{i}.mix.conv.b"] == (m["inner"],)
            assert want[f"l{i}.mix.dt"] == (m["inner"], m["dt_rank"]) and want[f"l{i}.mix.A_log"] == (m["inner"], m["state"])
        mlp = layer["mlp"]
        assert (f"l{i}.norm2" in want) == (mlp is not None)
        if mlp is not None:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            assert want[f"l{i}.mlp.router"] == (E, d) and want[f"l{i}.mlp.e{E - 1}.gate"] == (ff, d) and want[f"l{i}.mlp.e0.down"] == (d, ff)
            assert (f"l{i}.mlp.shared.up" in want) == ("shared" in mlp)
    assert ("bigram" in want) == ("bigram" in Z.ALL[name]["embedding"])
    assert ("loop.step" in want) == ("loop" in Z.ALL[name])


def test_the_order_of_runs_follows_the_loop():
    _, cfg, spec = spec_of(Z.MIXED)
    assert [(r.block, r.enter) for r in spec.order] == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    assert [r.cache for r in spec.order] == list(range(6)) and P.layer_runs(Z.MIXED) == [(r.block, r.enter) for r in spec.order]
    _, _, spec = spec_of(Z.LOOP_ALL)
    assert [(r.block, r.enter) for r in spec.order] == [(0, 0), (1, None), (0, 1), (1, None), (0, 2), (1, None)]
    _, _, spec = spec_of(Z.SCAN_ONLY)
    assert spec.pass_input is None and [(r.block, r.enter) for r in spec.order] == [(0, None)]


@pytest.mark.parametrize("edit,word", [
    (lambda c: c["layers"][1].__setitem__("type", "conv"), "layer type"),
    (lambda c: c["layers"][1]["mixer"]["left"].__setitem__("kv_heads", 4), "do not divide"),
    (lambda c: c["layers"][1]["mixer"]["right"].__setitem__("decay", [0.5]), "decay"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].__setitem__("dims", 18), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].__setitem__("dims", 7), "even"),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 4), "top"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].__setitem__("count", 4), "groups"),
    (lambda c: c["loop"].__setitem__("stop", 9), "loop"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"].pop("dt_rank"), "dt_rank"),
    (lambda c: c["layers"][1]["mixer"]["left"]["mask"].pop("size"), "mask.size"),
])
def test_what_does_not_fit_is_refused_by_name(edit, word):
    cfg = copy.deepcopy(Z.MIXED)
    edit(cfg)
    with pytest.raises(ConfigError) as e:
        architecture_of(cfg).config_from_dict(cfg)
    assert word in str(e.value)


def test_the_plain_pieces_on_cases_worked_out_by_hand():
    # a window of 3 that keeps the first 2: position 6 sees 0, 1 (kept) and 4, 5, 6
    assert [j for j in range(8) if P.visible(6, j, 3, 2)] == [0, 1, 4, 5, 6]
    assert [j for j in range(8) if P.visible(1, j, 3, 2)] == [0, 1]
    assert P.bigram_rows([5, 7, 7], 11, 3, 2) == [11, (5 * 3 + 7 * 2) % 11, (7 * 3 + 7 * 2) % 11]
    # nine experts in three groups of which one is kept: the best expert's group wins, the two best of it are taken
    z = np.array([0.1, 3.0, 0.2, 2.9, 2.8, 2.7, 2.6, 2.5, 2.4])
    order, weight, margin = P.route(z, {"experts": 9, "top": 2, "groups": {"count": 3, "keep": 1}})
    s = np.exp(z) / np.exp(z).sum()
    assert list(order) == [1, 2] and np.allclose(weight, s[[1, 2]]) and abs(margin - 0.1) < 1e-12
    # without a scaling rule the frequencies are the plain powers; with one, slow pairs are divided by the factor
    f, amp = P.rotary_frequencies({"dims": 4, "base": 100.0})
    assert np.allclose(f, [1.0, 0.1]) and amp == 1.0
    f, amp = P.rotary_frequencies({"dims": 8, "base": 10000.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}})
    assert np.isclose(f[0], 1.0) and np.isclose(f[3], 10000.0 ** -0.75 / 4.0) and np.isclose(amp, 0.1 * np.log(4.0) + 1.0)
    # one channel, one state number, constant inputs: the recurrence by hand
    w = {"m.in": np.array([[1.0], [0.0]]), "m.conv": np.array([[1.0]]), "m.conv.b": np.zeros(1), "m.x": np.array([[1.0], [1.0], [1.0]]),
         "m.dt": np.array([[0.0]]), "m.dt.b": np.array([np.log(np.e - 1.0)]), "m.A_log": np.zeros((1, 1)), "m.D": np.zeros(1),
         "m.o": np.array([[1.0]])}
    # z = 0 -> silu(z) = 0: the output is zero whatever the state; so look at a gate of 1 through z's weight
    w["m.in"] = np.array([[1.0], [1.0]])
    h = np.ones((2, 1))
    u = P.silu(1.0)
    s1 = u * u                       # dt = 1, A = -1: S1 = dt u B = u * u; S2 = e^-1 S1 + u u
    want = np.array([s1 * u, (np.exp(-1.0) * s1 + s1) * u]) * P.silu(1.0)
    got = P.selective_scan(h, {"inner": 1, "state": 1, "dt_rank": 1, "conv": 1}, w, "m.")
    assert np.allclose(got[:, 0], want)
