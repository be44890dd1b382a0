"""Typed configuration of the Zekalorn family, read from the keys of its ``config.json``.

Every size comes from the file (or, for a tensor's shape, follows from sizes in it); so does every
constant that one model of the design may choose differently from another.  A key the file must give
and does not is an error that names it; a block of keys that is absent altogether (``loop``,
``token_side``, an attention's ``q_temp`` or ``bias_max``, a layer's ``mlp``) switches that mechanism off.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError

MIXER_KINDS = ("attention", "channel_delta")
MLP_KINDS = ("dense", "moe")


def _opt_int(d: Dict[str, Any], key: str) -> Optional[int]:
    return None if d.get(key) is None else int(d[key])


def _need(d: Dict[str, Any], key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json lacks {where}.{key}" if where else f"config.json lacks {key!r}")
    return d[key]


@dataclass(frozen=True)
class MlpConfig:
    kind: str                     # "dense": gated, ff wide; "moe": ``experts`` small ones of which a token uses ``top``
    ff: int
    experts: int = 0
    top: int = 0

    @staticmethod
    def from_dict(d: Optional[Dict[str, Any]], where: str) -> Optional["MlpConfig"]:
        if d is None:
            return None
        kind = str(_need(d, "kind", where))
        if kind == "dense":
            out = MlpConfig(kind, int(_need(d, "ff", where)))
        elif kind == "moe":
            router = _need(d, "router", where)
            out = MlpConfig(kind, int(_need(_need(d, "expert", where), "ff", where + ".expert")),
                            int(_need(router, "experts", where + ".router")), int(_need(router, "top", where + ".router")))
            if not 1 <= out.top <= out.experts:
                raise ConfigError(f"{where}.router: top {out.top} of {out.experts} experts")
        else:
            raise ConfigError(f"{where}.kind {kind!r} is not one of {MLP_KINDS}")
        if out.ff <= 0:
            raise ConfigError(f"{where}: ff must be positive")
        return out

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class MixerConfig:
    type: str
    heads: int
    kv_heads: int
    dim: int                      # size of a query and of a key
    vdim: int                     # size of a value
    conv: int = 0                 # channel_delta: taps of the short convolutions
    scale: float = 0.0            # attention: factor of q . k
    bias_max: Optional[float] = None          # attention: distance at which the bias table's last row is reached
    q_temp_coef: Optional[float] = None       # attention: query temperature 1 + coef * ln(floor((p + 1) / every) + 1)
    q_temp_every: int = 0
    # sizes that only the shapes of a checkpoint's tensors give (ranks of the two-step projections of the
    # decay and of the output gate; rows of the bias table): read from the shapes when a folder is opened
    # (:func:`sizes_from_shapes`), from these keys in a configuration that the random-weights mode wrote
    decay_rank: Optional[int] = None
    gate_rank: Optional[int] = None
    bias_rows: Optional[int] = None

    @staticmethod
    def from_dict(kind: str, d: Dict[str, Any], where: str) -> "MixerConfig":
        if kind not in MIXER_KINDS:
            raise ConfigError(f"{where}: mixer type {kind!r} is not one of {MIXER_KINDS}")
        base = dict(type=kind, heads=int(_need(d, "heads", where)), kv_heads=int(_need(d, "kv_heads", where)),
                    dim=int(_need(d, "dim", where)), vdim=int(_need(d, "vdim", where)))
        if kind == "channel_delta":
            out = MixerConfig(conv=int(_need(d, "conv", where)), decay_rank=_opt_int(d, "decay_rank"),
                              gate_rank=_opt_int(d, "gate_rank"), **base)
            if out.conv < 1:
                raise ConfigError(f"{where}.conv must be at least 1")
        else:
            temp = d.get("q_temp")
            out = MixerConfig(scale=float(_need(d, "scale", where)),
                              bias_max=None if d.get("bias_max") is None else float(d["bias_max"]),
                              q_temp_coef=None if temp is None else float(_need(temp, "coef", where + ".q_temp")),
                              q_temp_every=0 if temp is None else int(_need(temp, "every", where + ".q_temp")),
                              bias_rows=_opt_int(d, "bias_rows"), **base)
            if temp is not None and out.q_temp_every < 1:
                raise ConfigError(f"{where}.q_temp.every must be at least 1")
        for name in ("heads", "kv_heads", "dim", "vdim"):
            if getattr(out, name) <= 0:
                raise ConfigError(f"{where}.{name} must be positive")
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: {out.heads} heads do not divide into {out.kv_heads} kv heads")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim}
        for key in ("decay_rank", "gate_rank", "bias_rows"):
            if getattr(self, key) is not None:
                d[key] = getattr(self, key)
        if self.type == "channel_delta":
            d["conv"] = self.conv
        else:
            d["scale"] = self.scale
            if self.bias_max is not None:
                d["bias_max"] = self.bias_max
            if self.q_temp_coef is not None:
                d["q_temp"] = {"coef": self.q_temp_coef, "every": self.q_temp_every}
        return d


@dataclass(frozen=True)
class LayerConfig:
    mixer: MixerConfig
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class ZekalornConfig:
    architecture: str
    vocab: int
    width: int
    max_positions: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[LayerConfig, ...]
    loop: Optional[LoopConfig]
    side_dim: Optional[int]       # size of a layer's share of a token's side row (None: no side input)
    torch_dtype: str = "bfloat16"

    @staticmethod
    def from_dict(d: Dict[str, Any]) -> "ZekalornConfig":
        name = d.get("architecture") or (d.get("architectures") or [None])[0]
        if not name:
            raise ConfigError("config.json lacks 'architecture'")
        layers = []
        for i, entry in enumerate(_need(d, "layers", "")):
            where = f"layers[{i}]"
            layers.append(LayerConfig(MixerConfig.from_dict(str(_need(entry, "type", where)), _need(entry, "mixer", where), where + ".mixer"),
                                      MlpConfig.from_dict(entry.get("mlp"), where + ".mlp")))
        if not layers:
            raise ConfigError("config.json lists no layers")
        loop = d.get("loop")
        if loop is not None:
            loop = LoopConfig(int(_need(loop, "start", "loop")), int(_need(loop, "stop", "loop")), int(_need(loop, "times", "loop")))
            if not (0 <= loop.start < loop.stop <= len(layers) and loop.times >= 1):
                raise ConfigError(f"loop {loop} does not fit {len(layers)} layers")
        side = d.get("token_side")
        cfg = ZekalornConfig(
            architecture=str(name), vocab=int(_need(d, "vocab", "")), width=int(_need(d, "width", "")),
            max_positions=int(_need(d, "max_positions", "")),
            embedding_scale=float(_need(_need(d, "embedding", ""), "scale", "embedding")),
            norm_eps=float(_need(_need(d, "norm", ""), "eps", "norm")),
            layers=tuple(layers), loop=loop, side_dim=None if side is None else int(_need(side, "dim", "token_side")), torch_dtype=str(d.get("torch_dtype", "bfloat16")))
        for name_, v in (("vocab", cfg.vocab), ("width", cfg.width), ("max_positions", cfg.max_positions)):
            if v <= 0:
                raise ConfigError(f"{name_} must be positive, got {v}")
        if not cfg.norm_eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {cfg.norm_eps}")
        if cfg.side_dim is not None and cfg.side_dim <= 0:
            raise ConfigError("token_side.dim must be positive")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture,
            "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
            "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
            "layers": [{"type": l.mixer.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                       for l in self.layers],
        }
        if self.loop is not None:
            d["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        if self.side_dim is not None:
            d["token_side"] = {"dim": self.side_dim}
        return d


def sizes_from_shapes(cfg: ZekalornConfig, shapes: Dict[str, Tuple[int, ...]]) -> ZekalornConfig:
    """``cfg`` with the sizes that ``config.json`` leaves to the tensors filled in from ``shapes`` (tensor name ->
    shape of a checkpoint).  A tensor that is not there leaves its size open; the loader then names it as missing."""
    import dataclasses
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        new = {}
        if m.type == "channel_delta":
            for key, tensor in (("decay_rank", f"l{i}.mix.a1"), ("gate_rank", f"l{i}.mix.g1")):
                if getattr(m, key) is None and tensor in shapes and len(shapes[tensor]) == 2:
                    new[key] = int(shapes[tensor][0])
        elif m.bias_max is not None and m.bias_rows is None:
            tensor = f"l{i}.mix.rel"
            if tensor in shapes and len(shapes[tensor]) == 2:
                new["bias_rows"] = int(shapes[tensor][0])
        layers.append(dataclasses.replace(layer, mixer=dataclasses.replace(m, **new)) if new else layer)
    return dataclasses.replace(cfg, layers=tuple(layers))
