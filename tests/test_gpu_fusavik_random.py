"""Fusavik configurations drawn at random (head counts and groups, key and value sizes, rotated channels, windows and
kept tokens on either side of each other and of the kernel's tiles, decay heads, scans, experts and groups, loops, with
and without each optional block of keys), each replayed in three ways in both compute types against the plain
implementation: the whole prompt, portions of changing size, and a prompt followed by single tokens."""
import os
import random
import shutil
import tempfile

import numpy as np
import pytest
import torch

import fusavik_configs as Z
import plain_fusavik as P
from gpu_common import random_tokens
from test_gpu_fusavik import assert_close, cuts, replay, runner_for, _margins

pytestmark = pytest.mark.gpu


def draw(seed: int) -> dict:
    r = random.Random(seed)
    width = r.choice([32, 40, 48, 64, 72, 96, 128])

    def pair():
        kv = r.choice([1, 2, 3, 4])
        heads = kv * r.choice([1, 2, 3, 5])
        dim = r.choice([8, 16, 24, 32, 40, 64])
        vdim = r.choice([8, 12, 16, 32, 48, 64])
        rot = None
        if r.random() < 0.8:
            dims = r.choice([d for d in (2, 4, 8, 16, 32, 64) if d <= dim] + [dim])
            scaling = (r.choice([2.0, 4.0, 16.0]), r.choice([16, 64, 512]), r.choice([4.0, 32.0]), r.choice([0.5, 1.0])) if r.random() < 0.6 else None
            rot = Z.rot(dims, r.choice([100.0, 10000.0, 500000.0]), scaling)
        mask = (r.choice([1, 2, 7, 16, 33, 64, 65, 100]), r.choice([0, 1, 3, 8, 70])) if r.random() < 0.85 else None
        rh = r.choice([1, 2, 3, 4])
        return Z.parallel(Z.left(heads, kv, dim, vdim, r.choice([0.1, 0.25, 0.5]), mask=mask, rot=rot),
                          Z.right(rh, r.choice([8, 12, 16, 32, 64]), r.choice([8, 20, 32, 64]), [r.choice([0.3, 0.8, 0.95, 0.999]) for _ in range(rh)]),
                          r.choice([0.5, 1.0, 1.5]), r.choice([0.5, 1.0]))

    def scan():
        return Z.scan(r.choice([24, 48, 64, 100, 128]), r.choice([1, 4, 6, 16, 24]), r.choice([1, 3, 8, 16]), r.choice([1, 2, 3, 4]))

    def mlp():
        if r.random() < 0.2:
            return None
        count = r.choice([1, 2, 3, 4])
        per = r.choice([1, 2, 3])
        keep = r.randint(1, count)
        top = r.randint(1, per * keep)
        groups = (count, keep) if (count > 1 or r.random() < 0.5) else None
        return Z.moe(r.choice([8, 12, 16, 40]), count * per, top, groups=groups, shared=r.choice([None, 8, 24, 48]))

    n = r.randint(1, 4)
    layers = [((pair() if r.random() < 0.6 else scan()), mlp()) for _ in range(n)]
    loop = None
    if r.random() < 0.6:
        start = r.randint(0, n - 1)
        loop = (start, r.randint(start + 1, n), r.choice([1, 2, 3]))
    bigram = (r.choice([7, 64, 101]), r.choice([1, 31, 1000003]), r.choice([1, 7, 65537])) if r.random() < 0.7 else None
    return Z.model(width, r.choice([33, 64, 100, 257]), layers, loop=loop, bigram=bigram, scale=r.choice([1.0, 4.0]), eps=r.choice([1e-6, 1e-5]))


_root = []
_kept = []


def folder_for(cfg, seed):
    import nanoinfer_amd  # noqa: F401
    from nanoinfer_amd.weights.loader import make_random_model
    if not _root:
        _root.append(tempfile.mkdtemp(prefix="fusavik-random-"))
        import atexit
        atexit.register(shutil.rmtree, _root[0], ignore_errors=True)
    return make_random_model(os.path.join(_root[0], f"m{seed}"), cfg, seed, dtype="bfloat16", matrix_std=0.1)


@pytest.mark.parametrize("seed", list(range(1, 13)))
def test_a_configuration_drawn_at_random(seed):
    cfg = draw(seed)
    folder = folder_for(cfg, seed)
    config, w = P.read_model_folder(folder)
    toks = random_tokens(cfg["vocab"], 140 if seed % 3 == 0 else 80, seed)
    margins = []
    want = torch.from_numpy(P.forward(list(toks), config, w, margins=margins))
    _kept.append(want)       # alive for good: the margins are looked up by the result's identity
    if margins:
        _margins[id(want)] = torch.from_numpy(np.stack(margins).min(axis=0))
    rng = random.Random(seed)
    for dtype in ("float32", "bfloat16"):
        runner = runner_for(folder, dtype, page_size=rng.choice([1, 4, 8, 16, 32]))
        got = replay(runner, {"w": toks}, [{"w": len(toks)}])["w"]
        assert_close(got, want, dtype, f"seed {seed}: whole")
        sizes = [rng.choice([1, 2, 3, 5, 16, 31, 64]) for _ in range(5)]
        got = replay(runner, {"p": toks}, [{"p": c} for c in cuts(len(toks), sizes)])["p"]
        assert_close(got, want, dtype, f"seed {seed}: portions of {sizes}")
        first = rng.randint(1, len(toks) - 20)
        got = replay(runner, {"d": toks}, [{"d": first}] + [{"d": 1}] * (len(toks) - first))["d"]
        assert_close(got, want, dtype, f"seed {seed}: {first} tokens, then one by one")
        assert not runner.cache.live_requests()
