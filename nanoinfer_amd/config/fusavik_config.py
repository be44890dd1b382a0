"""Typed configuration of the Fusavik family, read from the keys of its ``config.json``.

Every size and every constant that one model of the design may choose differently from another comes
from the file.  A key the file must give and does not is an error that names it; a block of keys that is
absent altogether (``loop``, ``embedding.bigram``, a layer's ``mlp``, an attention's ``rot``, its
``rot.scaling`` or its ``mask``, a router's ``groups``, an ``mlp.shared``) switches that mechanism off.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError

LAYER_TYPES = ("parallel", "mamba1")


def _need(d: Any, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json lacks {where}.{key}" if where else f"config.json lacks {key!r}")
    return d[key]


def _positive(value, what: str):
    if not value > 0:
        raise ConfigError(f"{what} must be positive, got {value}")
    return value


@dataclass(frozen=True)
class RotationConfig:
    """Rotation of the first ``dims`` channels of a head, channel i with channel i + dims/2; ``scaling`` (factor,
    original, fast, slow) stretches the slow pairs and raises cos and sin by ``0.1 ln(factor) + 1``."""

    dims: int
    base: float
    scaling: Optional[Tuple[float, float, float, float]] = None      # (factor, original, fast, slow)

    @staticmethod
    def from_dict(d: Optional[Dict[str, Any]], where: str) -> Optional["RotationConfig"]:
        if d is None:
            return None
        sc = d.get("scaling")
        if sc is not None:
            sc = tuple(float(_need(sc, k, where + ".scaling")) for k in ("factor", "original", "fast", "slow"))
        out = RotationConfig(int(_need(d, "dims", where)), float(_need(d, "base", where)), sc)
        if out.dims <= 0 or out.dims % 2:
            raise ConfigError(f"{where}.dims must be positive and even, got {out.dims}")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            factor, original, fast, slow = self.scaling
            d["scaling"] = {"factor": factor, "original": int(original) if float(original).is_integer() else original,
                            "fast": fast, "slow": slow}
        return d


@dataclass(frozen=True)
class WindowAttentionConfig:
    """The softmax half of a ``parallel`` mixer."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]         # a query sees the last ``window`` keys (its own among them); None: all
    keep_first: int               # ... and always the first ``keep_first`` keys of the sequence
    rot: Optional[RotationConfig]

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> "WindowAttentionConfig":
        mask = d.get("mask")
        out = WindowAttentionConfig(
            heads=int(_need(d, "heads", where)), kv_heads=int(_need(d, "kv_heads", where)), dim=int(_need(d, "dim", where)),
            vdim=int(_need(d, "vdim", where)), scale=float(_need(d, "scale", where)),
            window=None if mask is None else int(_need(mask, "size", where + ".mask")),
            keep_first=0 if mask is None else int(mask.get("keep_first", 0)),
            rot=RotationConfig.from_dict(d.get("rot"), where + ".rot"))
        for name in ("heads", "kv_heads", "dim", "vdim"):
            _positive(getattr(out, name), f"{where}.{name}")
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: {out.heads} heads do not divide into {out.kv_heads} kv heads")
        if out.window is not None and out.window < 1:
            raise ConfigError(f"{where}.mask.size must be at least 1")
        if out.keep_first < 0:
            raise ConfigError(f"{where}.mask.keep_first must not be negative")
        if out.rot is not None and out.rot.dims > out.dim:
            raise ConfigError(f"{where}.rot.dims {out.rot.dims} exceeds the head's {out.dim} channels")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale}
        if self.window is not None:
            d["mask"] = {"size": self.window, "keep_first": self.keep_first}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class DecayAttentionConfig:
    """The linear half of a ``parallel`` mixer: one decay a head."""

    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> "DecayAttentionConfig":
        out = DecayAttentionConfig(int(_need(d, "heads", where)), int(_need(d, "dim", where)), int(_need(d, "vdim", where)),
                                   tuple(float(x) for x in _need(d, "decay", where)))
        for name in ("heads", "dim", "vdim"):
            _positive(getattr(out, name), f"{where}.{name}")
        if len(out.decay) != out.heads:
            raise ConfigError(f"{where}.decay has {len(out.decay)} entries for {out.heads} heads")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: WindowAttentionConfig
    right: DecayAttentionConfig
    left_scale: float
    right_scale: float

    def to_dict(self) -> Dict[str, Any]:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class ScanMixerConfig:
    """The selective scan: ``inner`` channels with ``state`` numbers each, steps through a projection of ``dt_rank``."""

    inner: int
    state: int
    dt_rank: int
    conv: int

    def to_dict(self) -> Dict[str, Any]:
        return {"inner": self.inner, "state": self.state, "dt_rank": self.dt_rank, "conv": self.conv}


@dataclass(frozen=True)
class MoeConfig:
    ff: int
    experts: int
    top: int
    group_count: int = 1          # the experts form this many equal groups of neighbours ...
    group_keep: int = 1           # ... of which the best this many may be chosen from
    shared_ff: Optional[int] = None

    @staticmethod
    def from_dict(d: Optional[Dict[str, Any]], where: str) -> Optional["MoeConfig"]:
        if d is None:
            return None
        kind = str(d.get("kind", "moe"))
        if kind != "moe":
            raise ConfigError(f"{where}.kind {kind!r} is not 'moe'")
        router = _need(d, "router", where)
        groups = router.get("groups")
        shared = d.get("shared")
        out = MoeConfig(ff=int(_need(_need(d, "expert", where), "ff", where + ".expert")),
                        experts=int(_need(router, "experts", where + ".router")), top=int(_need(router, "top", where + ".router")),
                        group_count=1 if groups is None else int(_need(groups, "count", where + ".router.groups")),
                        group_keep=1 if groups is None else int(_need(groups, "keep", where + ".router.groups")),
                        shared_ff=None if shared is None else int(_need(shared, "ff", where + ".shared")))
        _positive(out.ff, f"{where}.expert.ff")
        if out.shared_ff is not None:
            _positive(out.shared_ff, f"{where}.shared.ff")
        if out.group_count < 1 or out.experts % out.group_count or not 1 <= out.group_keep <= out.group_count:
            raise ConfigError(f"{where}.router.groups: {out.group_keep} of {out.group_count} groups of {out.experts} experts")
        if not 1 <= out.top <= out.experts // out.group_count * out.group_keep:
            raise ConfigError(f"{where}.router: top {out.top} of {out.experts} experts in {out.group_keep} of "
                              f"{out.group_count} groups")
        return out

    def to_dict(self) -> Dict[str, Any]:
        router: Dict[str, Any] = {"experts": self.experts, "top": self.top}
        if (self.group_count, self.group_keep) != (1, 1):
            router["groups"] = {"count": self.group_count, "keep": self.group_keep}
        d: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff}, "router": router}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclass(frozen=True)
class FusavikLayer:
    type: str
    mixer: Any                    # ParallelMixerConfig or ScanMixerConfig
    mlp: Optional[MoeConfig]


@dataclass(frozen=True)
class BigramConfig:
    """A second embedding, of the pair (previous token, token): row ``(prev * mul_prev + cur * mul_cur) mod buckets``;
    a sequence's first token takes row ``buckets``."""

    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


def _mixer(kind: str, d: Dict[str, Any], where: str):
    if kind == "parallel":
        return ParallelMixerConfig(WindowAttentionConfig.from_dict(_need(d, "left", where), where + ".left"),
                                   DecayAttentionConfig.from_dict(_need(d, "right", where), where + ".right"),
                                   float(_need(d, "left_scale", where)), float(_need(d, "right_scale", where)))
    if kind == "mamba1":
        out = ScanMixerConfig(int(_need(d, "inner", where)), int(_need(d, "state", where)), int(_need(d, "dt_rank", where)),
                              int(_need(d, "conv", where)))
        for name in ("inner", "state", "dt_rank", "conv"):
            _positive(getattr(out, name), f"{where}.{name}")
        return out
    raise ConfigError(f"{where}: layer type {kind!r} is not one of {LAYER_TYPES}")


@dataclass(frozen=True)
class FusavikConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    bigram: Optional[BigramConfig]
    norm_eps: float
    layers: Tuple[FusavikLayer, ...]
    loop: Optional[LoopConfig]
    torch_dtype: str = "bfloat16"

    @staticmethod
    def from_dict(d: Dict[str, Any]) -> "FusavikConfig":
        name = d.get("architecture") or (d.get("architectures") or [None])[0]
        if not name:
            raise ConfigError("config.json lacks 'architecture'")
        layers = []
        for i, entry in enumerate(_need(d, "layers", "")):
            where = f"layers[{i}]"
            kind = str(_need(entry, "type", where))
            layers.append(FusavikLayer(kind, _mixer(kind, _need(entry, "mixer", where), where + ".mixer"),
                                       MoeConfig.from_dict(entry.get("mlp"), where + ".mlp")))
        if not layers:
            raise ConfigError("config.json lists no layers")
        loop = d.get("loop")
        if loop is not None:
            loop = LoopConfig(int(_need(loop, "start", "loop")), int(_need(loop, "stop", "loop")), int(_need(loop, "times", "loop")))
            if not (0 <= loop.start < loop.stop <= len(layers) and loop.times >= 1):
                raise ConfigError(f"loop {loop} does not fit {len(layers)} layers")
        emb = _need(d, "embedding", "")
        bigram = emb.get("bigram")
        if bigram is not None:
            bigram = BigramConfig(int(_need(bigram, "buckets", "embedding.bigram")), int(_need(bigram, "mul_prev", "embedding.bigram")),
                                  int(_need(bigram, "mul_cur", "embedding.bigram")))
            _positive(bigram.buckets, "embedding.bigram.buckets")
        cfg = FusavikConfig(architecture=str(name), vocab=int(_need(d, "vocab", "")), width=int(_need(d, "width", "")),
                            embedding_scale=float(_need(emb, "scale", "embedding")), bigram=bigram,
                            norm_eps=float(_need(_need(d, "norm", ""), "eps", "norm")), layers=tuple(layers), loop=loop,
                            torch_dtype=str(d.get("torch_dtype", "bfloat16")))
        _positive(cfg.vocab, "vocab")
        _positive(cfg.width, "width")
        _positive(cfg.norm_eps, "norm.eps")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        emb: Dict[str, Any] = {"scale": self.embedding_scale}
        if self.bigram is not None:
            emb["bigram"] = {"buckets": self.bigram.buckets, "mul_prev": self.bigram.mul_prev, "mul_cur": self.bigram.mul_cur}
        d: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width, "embedding": emb,
            "norm": {"eps": self.norm_eps},
            "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                       for l in self.layers],
        }
        if self.loop is not None:
            d["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return d
