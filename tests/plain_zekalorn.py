"""A plain, slow Zekalorn forward: whole sequences, no cache, float64, one function per mechanism.

The oracle of the Zekalorn tests.  It shares no code with ``nanoinfer_amd``: it reads a model folder
with ``json`` and the ``safetensors`` package, and works token by token where the design is
recurrent.  Notation: ``d`` the width of the residual stream, ``T`` the tokens of the sequence,
positions 0..T-1, matrices stored [out, in] and applied as ``x @ W.T``.

The design, in short.  ``x_t = E[tok_t] * s_e + P[t]``.  The layers run in the listed order; the
layers ``start..stop-1`` of the ``loop`` run ``times`` times with the same weights (every pass from
an empty memory), and vector ``L[p]`` is added to ``x`` ahead of pass ``p``.  A layer is
``n = rms(x) * w1``, ``x += mixer(n) + ff(n)``, and then the token's own side input:
``y = Wp (gelu_tanh(Wg x) * Es[tok, i*ds:(i+1)*ds])``, ``x += rms(y) * ws``.  Mixers: softmax
attention with grouped heads, a query temperature that grows with the position and a learned bias by
(bucketed) distance; or the gated delta rule with one decay per key channel.  Feed-forwards: SwiGLU,
or a router that picks the ``top`` largest of its logits and mixes squared-ReLU experts with the
softmax of the chosen logits.  At the end ``logits = H (rms(x) * wf)``.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64


# --------------------------------------------------------------------------- small functions

def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps)`` over the last axis."""
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * w.to(F64)


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    return x.to(F64) @ w.to(F64).t()


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# --------------------------------------------------------------------------- embedding

def embed(table: torch.Tensor, positions: torch.Tensor, scale: float, ids: Sequence[int]) -> torch.Tensor:
    """``x_t = E[id_t] * scale + P[t]``."""
    idx = torch.tensor(list(ids), dtype=torch.long)
    return table.to(F64)[idx] * scale + positions.to(F64)[: len(ids)]


# --------------------------------------------------------------------------- attention

def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the bias table for a key ``n`` tokens back: the distance itself below ``rows // 2``,
    beyond that logarithmic steps that reach the last row at distance ``far``."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def query_temperature(p: int, coef: float, every: int) -> float:
    """``1 + coef * ln(floor((p + 1) / every) + 1)`` for a query at position ``p``."""
    return 1.0 + coef * math.log((p + 1) // every + 1)


def attention(n: torch.Tensor, w: Dict[str, torch.Tensor], m: dict) -> torch.Tensor:
    """Causal softmax attention of the normed rows ``n`` [T, d], head by head and query by query."""
    T = n.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(n, w["q"]).view(T, H, dk)
    k = linear(n, w["k"]).view(T, G, dk)
    v = linear(n, w["v"]).view(T, G, dv)
    rel = w["rel"].to(F64) if "rel" in w else None
    temp = m.get("q_temp")
    out = torch.zeros(T, H, dv, dtype=F64)
    if rel is not None:     # the bias of every distance that occurs, [T, H]
        by_distance = rel[torch.tensor([distance_bucket(n_back, rel.shape[0], m["bias_max"]) for n_back in range(T)])]
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            qi = q[i, h] * (query_temperature(i, temp["coef"], temp["every"]) if temp else 1.0)
            s = (k[: i + 1, g] @ qi) * m["scale"]
            if rel is not None:
                s = s + by_distance[: i + 1, h].flip(0)          # key j is i - j back
            p = torch.softmax(s, dim=0)
            out[i, h] = p @ v[: i + 1, g]
    return linear(out.reshape(T, H * dv), w["o"])


# --------------------------------------------------------------------------- gated delta rule

def short_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """Causal convolution over time, one filter a channel: ``y_t[c] = sum_j taps[c, j] * x_{t-(n-1-j)}[c]``
    (the last column is the current token's; zeros before the start)."""
    T, C = x.shape
    n = taps.shape[1]
    taps = taps.to(F64)
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(n):
            src = t - (n - 1 - j)
            if src >= 0:
                y[t] += taps[:, j] * x[src]
    return y


def unit(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + 1e-6)


def channel_delta(n: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """The gated delta rule with a decay per key channel over the normed rows ``n`` [T, d], token by token."""
    T = n.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(linear(n, w["q"]), w["q.conv"])).view(T, G, dk)
    k = silu(short_conv(linear(n, w["k"]), w["k.conv"])).view(T, G, dk)
    v = silu(short_conv(linear(n, w["v"]), w["v.conv"])).view(T, H, dv)
    q = unit(q) * dk ** -0.5
    k = unit(k)
    beta = torch.sigmoid(linear(n, w["b"]))                                             # [T, H]
    rate = torch.exp(w["A_log"].to(F64)).view(1, H, 1)
    decay = torch.exp(-rate * softplus(linear(linear(n, w["a1"]), w["a2"]) + w["dt_bias"].to(F64)).view(T, H, dk))
    gate = torch.sigmoid(linear(linear(n, w["g1"]), w["g2"])).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for h in range(H):
        g = h // (H // G)
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = decay[t, h].view(dk, 1) * S
            u = beta[t, h] * (v[t, h] - S.t() @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, h] = S.t() @ q[t, g]
    out = rms(out, eps) * w["norm"].to(F64) * gate
    return linear(out.reshape(T, H * dv), w["o"])


# --------------------------------------------------------------------------- feed-forwards

def dense_ff(n: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return linear(silu(linear(n, w["gate"])) * linear(n, w["up"]), w["down"])


def routed_ff(n: torch.Tensor, w: Dict[str, torch.Tensor], experts: int, top: int, margins: Optional[List] = None) -> torch.Tensor:
    """Every token goes to the ``top`` experts with the largest router logits, weighted by the
    softmax over those logits alone; an expert is ``Wd relu(Wu n)^2``.  ``margins`` collects, per row, by how
    much the last chosen logit beats the first one left out (how close a call the choice was)."""
    T = n.shape[0]
    z = linear(n, w["router"])
    if margins is not None and top < experts:
        ranked = torch.sort(z, dim=-1, descending=True).values
        margins.append(ranked[:, top - 1] - ranked[:, top])
    out = torch.zeros(T, w["e0.down"].shape[0], dtype=F64)
    for t in range(T):
        chosen = torch.topk(z[t], top).indices
        mix = torch.softmax(z[t][chosen], dim=0)
        for c, e in enumerate(chosen.tolist()):
            hid = torch.relu(linear(n[t], w[f"e{e}.up"])) ** 2
            out[t] += mix[c] * linear(hid, w[f"e{e}.down"])
    return out


def side_input(x: torch.Tensor, w: Dict[str, torch.Tensor], rows: torch.Tensor, eps: float) -> torch.Tensor:
    """What the token's own side vector (``rows`` [T, ds]) adds to the stream ``x``."""
    y = linear(gelu_tanh(linear(x, w["gate"])) * rows.to(F64), w["proj"])
    return rmsnorm(y, w["norm"], eps)


# --------------------------------------------------------------------------- the model

def sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def layer(i: int, x: torch.Tensor, ids: Sequence[int], config: dict, tensors: Dict[str, torch.Tensor],
          margins: Optional[List] = None) -> torch.Tensor:
    spec = config["layers"][i]
    eps = config["norm"]["eps"]
    n = rmsnorm(x, tensors[f"l{i}.norm1"], eps)
    mix_w = sub(tensors, f"l{i}.mix.")
    if spec["type"] == "attention":
        y = attention(n, mix_w, spec["mixer"])
    elif spec["type"] == "channel_delta":
        y = channel_delta(n, mix_w, spec["mixer"], eps)
    else:
        raise ValueError(f"mixer {spec['type']!r}")
    mlp = spec.get("mlp")
    if mlp is not None:
        ff_w = sub(tensors, f"l{i}.mlp.")
        if mlp["kind"] == "dense":
            y = y + dense_ff(n, ff_w)
        elif mlp["kind"] == "moe":
            y = y + routed_ff(n, ff_w, mlp["router"]["experts"], mlp["router"]["top"], margins)
        else:
            raise ValueError(f"feed-forward {mlp['kind']!r}")
    x = x + y
    side = config.get("token_side")
    if side is not None:
        ds = side["dim"]
        rows = tensors["side.embed"][torch.tensor(list(ids), dtype=torch.long)][:, i * ds:(i + 1) * ds]
        x = x + side_input(x, sub(tensors, f"l{i}.side."), rows, eps)
    return x


def layer_runs(config: dict):
    """(layer, number of the pass or None) in the order they run; the pass number stands at the first
    layer of every pass of the loop."""
    L = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None) for i in range(L)]
    runs = [(i, None) for i in range(loop["start"])]
    for p in range(loop["times"]):
        runs += [(i, p if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], L)]


def forward(config: dict, tensors: Dict[str, torch.Tensor], ids: Sequence[int], streams: Optional[List] = None,
            margins: Optional[List] = None) -> torch.Tensor:
    """Logits [T, vocab] of the whole sequence; ``streams`` collects the residual stream after every layer run,
    ``margins`` the routers' margins [T] of every routed layer run."""
    x = embed(tensors["embed"], tensors["pos"], config["embedding"]["scale"], ids)
    for i, p in layer_runs(config):
        if p is not None:
            x = x + tensors["loop.step"].to(F64)[p]
        x = layer(i, x, ids, config, tensors, margins)
        if streams is not None:
            streams.append(x.clone())
    return linear(rmsnorm(x, tensors["final.norm"], config["norm"]["eps"]), tensors["head"])


def read_model_folder(folder: str):
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return config, tensors


def round_to_bfloat16(tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: (v.to(torch.bfloat16).to(torch.float32) if v.is_floating_point() and v.dim() > 1 else v) for k, v in tensors.items()}
