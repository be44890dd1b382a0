"""A plain, slow implementation of the Fusavik design in float64 numpy: one function per mechanism,
written from the equations, sharing no code with the engine.  It runs one whole sequence at a time and
keeps nothing between calls; the tests compare the engine's logits, layer outputs and kernels with it.

Notation: ``d`` width, ``T`` tokens of the sequence, weights as stored ([out, in], applied as ``W x``).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import numpy as np

F = np.float64


def rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def silu(z):
    return z / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


# ------------------------------------------------------------------ embedding

def bigram_rows(tokens: List[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Row of the bigram table for every token: a hash of (previous, current); the first token takes the last row."""
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets)
    return rows


def embed(tokens: List[int], cfg: dict, w: Dict[str, np.ndarray]) -> np.ndarray:
    e = cfg["embedding"]
    x = w["embed"][tokens] * e["scale"]
    if e.get("bigram") is not None:
        b = e["bigram"]
        x = x + w["bigram"][bigram_rows(tokens, b["buckets"], b["mul_prev"], b["mul_cur"])]
    return x


# ------------------------------------------------------------------ rotation

def rotary_frequencies(rot: dict):
    """(frequency of every pair, factor on cos and sin) for a ``rot`` entry of a mixer's configuration."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    sc = rot.get("scaling")
    if sc is None:
        return f, 1.0

    def dim_of(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(sc["fast"])), 0)
    hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(half, dtype=F) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    f = f / sc["factor"] * ramp + f * (1.0 - ramp)
    return f, 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x: np.ndarray, positions: np.ndarray, rot: dict) -> np.ndarray:
    """x [T, heads, dim]: the first ``dims`` channels of every head rotated, channel i with channel i + dims/2."""
    f, amp = rotary_frequencies(rot)
    dims = rot["dims"]
    half = dims // 2
    a = positions[:, None].astype(F) * f[None, :]
    c, s = (np.cos(a) * amp)[:, None, :], (np.sin(a) * amp)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ------------------------------------------------------------------ the two halves of the 'parallel' mixer

def visible(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def window_attention(h: np.ndarray, m: dict, w: Dict[str, np.ndarray], pre: str, eps: float) -> np.ndarray:
    """Softmax attention with grouped heads, a norm over the whole query and key projections, a rotation of
    part of every head, a sliding window and first tokens that stay visible."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(h @ w[pre + "q"].T, eps) * w[pre + "q.norm"]
    k = rms(h @ w[pre + "k"].T, eps) * w[pre + "k.norm"]
    v = (h @ w[pre + "v"].T).reshape(T, G, dv)
    pos = np.arange(T)
    q, k = q.reshape(T, H, dk), k.reshape(T, G, dk)
    if m.get("rot") is not None:
        q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    size, keep = (m["mask"]["size"], m["mask"].get("keep_first", 0)) if m.get("mask") is not None else (T + 1, 0)
    out = np.zeros((T, H, dv), dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            js = [j for j in range(i + 1) if visible(i, j, size, keep)]
            s = (k[js, g] @ q[i, hd]) * m["scale"]
            p = np.exp(s - s.max())
            out[i, hd] = (p / p.sum()) @ v[js, g]
    return out.reshape(T, H * dv) @ w[pre + "o"].T


def decay_attention(h: np.ndarray, m: dict, w: Dict[str, np.ndarray], pre: str, eps: float) -> np.ndarray:
    """Linear attention with one decay a head: S <- decay S + k v^T, o = S^T q; q, k, v after silu; the heads'
    read-outs normed together, gated by sigmoid(W_g h), projected."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[pre + "q"].T).reshape(T, H, dk)
    k = silu(h @ w[pre + "k"].T).reshape(T, H, dk)
    v = silu(h @ w[pre + "v"].T).reshape(T, H, dv)
    o = np.zeros((T, H, dv), dtype=F)
    for hd in range(H):
        S = np.zeros((dk, dv), dtype=F)
        for t in range(T):
            S = m["decay"][hd] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    y = rms(o.reshape(T, H * dv), eps) * w[pre + "norm"] * sigmoid(h @ w[pre + "g"].T)
    return y @ w[pre + "o"].T


def parallel_mixer(h, m, w, pre, eps):
    return (m["left_scale"] * window_attention(h, m["left"], w, pre + "left.", eps)
            + m["right_scale"] * decay_attention(h, m["right"], w, pre + "right.", eps))


# ------------------------------------------------------------------ selective scan

def selective_scan(h: np.ndarray, m: dict, w: Dict[str, np.ndarray], pre: str) -> np.ndarray:
    T = h.shape[0]
    inner, N, R, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
    xz = h @ w[pre + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    padded = np.concatenate([np.zeros((taps - 1, inner), dtype=F), x], axis=0)
    conv = w[pre + "conv"]                          # [inner, taps]; the last column is the current token's
    x = sum(padded[j: j + T] * conv[:, j] for j in range(taps)) + w[pre + "conv.b"]
    x = silu(x)
    p = x @ w[pre + "x"].T
    dt = softplus(p[:, :R] @ w[pre + "dt"].T + w[pre + "dt.b"])
    Bm, Cm = p[:, R: R + N], p[:, R + N: R + 2 * N]
    A = -np.exp(w[pre + "A_log"])
    S = np.zeros((inner, N), dtype=F)
    y = np.zeros((T, inner), dtype=F)
    for t in range(T):
        S = np.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * Bm[t][None, :]
        y[t] = S @ Cm[t] + w[pre + "D"] * x[t]
    return (y * silu(z)) @ w[pre + "o"].T


# ------------------------------------------------------------------ feed-forward

def gated_ff(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def route(z: np.ndarray, router: dict):
    """For one token's router logits: (chosen experts, their weights, how close the closest call was: the smallest
    difference of logits between something chosen and something left out, a group or an expert)."""
    E, top = router["experts"], router["top"]
    s = np.exp(z - z.max())
    s = s / s.sum()
    allowed = np.ones(E, dtype=bool)
    groups = router.get("groups")
    margin = np.inf
    if groups is not None:
        n = groups["count"]
        per = E // n
        score = s.reshape(n, per).max(axis=1)
        ranked = np.argsort(-score, kind="stable")
        best = ranked[: groups["keep"]]
        if groups["keep"] < n:
            top_logit = z.reshape(n, per).max(axis=1)
            margin = top_logit[ranked[groups["keep"] - 1]] - top_logit[ranked[groups["keep"]]]
        allowed[:] = False
        for g in best:
            allowed[g * per: (g + 1) * per] = True
    ranked = np.argsort(-np.where(allowed, s, -1.0), kind="stable")
    order = ranked[:top]
    if top < int(allowed.sum()):
        margin = min(margin, z[ranked[top - 1]] - z[ranked[top]])
    return order, s[order], margin


def moe(h: np.ndarray, mlp: dict, w: Dict[str, np.ndarray], pre: str, margins: Optional[list] = None) -> np.ndarray:
    out = np.zeros_like(h)
    z = h @ w[pre + "router"].T
    closest = np.full(h.shape[0], np.inf)
    for t in range(h.shape[0]):
        chosen, weight, closest[t] = route(z[t], mlp["router"])
        for e, a in zip(chosen, weight):
            out[t] += a * gated_ff(h[t: t + 1], w, f"{pre}e{e}.")[0]
    if margins is not None:
        margins.append(closest)
    if mlp.get("shared") is not None:
        out += gated_ff(h, w, pre + "shared.")
    return out


# ------------------------------------------------------------------ the model

def layer(x, i: int, cfg: dict, w, margins: Optional[list] = None):
    L = cfg["layers"][i]
    eps = cfg["norm"]["eps"]
    pre = f"l{i}."
    n = rms(x, eps) * w[pre + "norm1"]
    if L["type"] == "parallel":
        x = x + parallel_mixer(n, L["mixer"], w, pre + "mix.", eps)
    elif L["type"] == "mamba1":
        x = x + selective_scan(n, L["mixer"], w, pre + "mix.")
    else:
        raise ValueError(L["type"])
    if L.get("mlp") is not None:
        x = x + moe(rms(x, eps) * w[pre + "norm2"], L["mlp"], w, pre + "mlp.", margins)
    return x


def layer_runs(cfg: dict):
    """(layer, number of the pass it opens or None) in the order they run."""
    L = len(cfg["layers"])
    lp = cfg.get("loop")
    if lp is None:
        return [(i, None) for i in range(L)]
    runs = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"]):
        runs += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, None) for i in range(lp["stop"], L)]


def forward(tokens: List[int], cfg: dict, weights: Dict[str, np.ndarray], taps: Optional[list] = None,
            margins: Optional[list] = None) -> np.ndarray:
    """Logits [T, vocab] of one whole sequence; ``taps`` (a list) receives the stream after every layer run,
    ``margins`` (a list) per routed layer run the closest call of its router for every token."""
    w = {k: np.asarray(v, dtype=F) for k, v in weights.items()}
    e = embed(tokens, cfg, w)
    x = e.copy()
    for i, enters in layer_runs(cfg):
        if enters is not None:
            if enters > 0:
                x = x + e
            x = x + w["loop.step"][enters]
        x = layer(x, i, cfg, w, margins)
        if taps is not None:
            taps.append(x.copy())
    x = rms(x, cfg["norm"]["eps"]) * w["final.norm"]
    return x @ w["head"].T


# ------------------------------------------------------------------ a model folder, read without the engine

def read_model_folder(folder: str):
    """(config.json as a dict, tensor name -> float64 array) of a folder with ``model.safetensors``: eight bytes of
    header length, the JSON header (name -> dtype, shape, data_offsets), the data."""
    import json
    import os
    import struct
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    with open(os.path.join(folder, "model.safetensors"), "rb") as fh:
        blob = fh.read()
    n = struct.unpack("<Q", blob[:8])[0]
    header = json.loads(blob[8: 8 + n])
    data = blob[8 + n:]
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        a, b = info["data_offsets"]
        raw = data[a:b]
        if info["dtype"] == "BF16":
            arr = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32)
        elif info["dtype"] == "F32":
            arr = np.frombuffer(raw, dtype="<f4")
        elif info["dtype"] == "I32":
            arr = np.frombuffer(raw, dtype="<i4")
        else:
            raise ValueError(f"{name}: dtype {info['dtype']}")
        out[name] = arr.astype(F).reshape(info["shape"])
    return cfg, out
