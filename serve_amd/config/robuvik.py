"""Typed configuration of the Robuvik decoder, read from config.json's own keys.

config.json gives `vocab`, `width`, `norm.eps`, `embedding.bigram` ({"buckets", "mul_prev", "mul_cur"}: a second
embedding row chosen by a hash of the previous and the current token), `layers` (a list whose entries name the layer's
mixer by `type`: "attention" = grouped-query attention with biases, a sliding window and a sink, or "latent_attention"
= attention over one latent per token with an output gate; the mixer's sizes and constants in `mixer`; the feed-forward
in `mlp`: null, {"kind": "dense", "ff"} or {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"},
"shared": {"ff"}}) and optionally `loop` ({"start", "stop", "times"}: layers start .. stop-1 run `times` times in a row
with the same weights).  Layers differ from each other; nothing about them stands in code.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple, Union

from .kotipel import LoopConfig, _need
from .llama import ConfigError


@dataclass(frozen=True)
class YarnScaling:
    factor: float
    original: float
    fast: float
    slow: float

    @staticmethod
    def from_dict(s: Dict[str, Any], where: str) -> "YarnScaling":
        _need(s, ("factor", "original", "fast", "slow"), where)
        c = YarnScaling(float(s["factor"]), float(s["original"]), float(s["fast"]), float(s["slow"]))
        if min(c.factor, c.original, c.fast, c.slow) <= 0:
            raise ConfigError(f"{where}: factor, original, fast and slow must be positive")
        return c

    def to_dict(self) -> Dict[str, Any]:
        o = self.original
        return {"factor": self.factor, "fast": self.fast, "original": int(o) if o == int(o) else o, "slow": self.slow}


@dataclass(frozen=True)
class RotConfig:
    base: float
    dims: int
    scaling: Optional[YarnScaling] = None

    @staticmethod
    def from_dict(r: Dict[str, Any], where: str) -> "RotConfig":
        _need(r, ("base", "dims"), where)
        s = r.get("scaling")
        c = RotConfig(float(r["base"]), int(r["dims"]), YarnScaling.from_dict(s, where + ".scaling") if s else None)
        if c.dims <= 0 or c.dims % 2 or not c.base > 1:
            raise ConfigError(f"{where}: dims must be positive and even, base above 1")
        return c

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotConfig] = None
    window: Optional[int] = None

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "WindowAttentionConfig":
        _need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
        rot = RotConfig.from_dict(m["rot"], where + ".rot") if m.get("rot") else None
        mask = m.get("mask")
        window = None
        if mask:
            _need(mask, ("size",), where + ".mask")
            window = int(mask["size"])
        c = WindowAttentionConfig(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                                  rot, window)
        if min(c.heads, c.kv_heads, c.dim, c.vdim) <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"{where}: sizes must be positive and heads a multiple of kv_heads")
        if rot is not None and rot.dims > c.dim:
            raise ConfigError(f"{where}.rot.dims={rot.dims} does not fit heads of {c.dim}")
        if window is not None and window <= 0:
            raise ConfigError(f"{where}.mask.size must be positive")
        return c

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        d.update(scale=self.scale, vdim=self.vdim)
        return d


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: RotConfig

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "LatentAttentionConfig":
        _need(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale", "rot"), where)
        rot = RotConfig.from_dict(m["rot"], where + ".rot")
        c = LatentAttentionConfig(int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]),
                                  int(m["q_rank"]), float(m["scale"]), rot)
        if min(c.heads, c.dim, c.rot_dim, c.vdim, c.kv_rank, c.q_rank) <= 0:
            raise ConfigError(f"{where}: sizes must be positive")
        if rot.dims != c.rot_dim:
            raise ConfigError(f"{where}: the rotation takes the whole rotated part: rot.dims={rot.dims}, rot_dim={c.rot_dim}")
        return c

    def to_dict(self) -> Dict[str, Any]:
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank,
                "rot": self.rot.to_dict(), "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class DenseConfig:
    ff: int

    def to_dict(self) -> Dict[str, Any]:
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class ExpertsConfig:
    experts: int
    top: int
    ff: int
    shared_ff: Optional[int] = None

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"expert": {"ff": self.ff}, "kind": "moe", "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclass(frozen=True)
class RobuvikLayerConfig:
    mixer: Union[WindowAttentionConfig, LatentAttentionConfig]
    mlp: Union[None, DenseConfig, ExpertsConfig]

    @property
    def type(self) -> str:
        return "attention" if isinstance(self.mixer, WindowAttentionConfig) else "latent_attention"

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class BigramConfig:
    buckets: int
    mul_prev: int
    mul_cur: int

    def to_dict(self) -> Dict[str, Any]:
        return {"buckets": self.buckets, "mul_cur": self.mul_cur, "mul_prev": self.mul_prev}


def _mlp_from_dict(mlp: Optional[Dict[str, Any]], where: str):
    if mlp is None:
        return None
    kind = mlp.get("kind") if isinstance(mlp, dict) else None
    if kind == "dense":
        _need(mlp, ("ff",), where)
        c = DenseConfig(int(mlp["ff"]))
        if c.ff <= 0:
            raise ConfigError(f"{where}.ff must be positive")
        return c
    if kind == "moe":
        _need(mlp, ("expert", "router"), where)
        _need(mlp["expert"], ("ff",), where + ".expert")
        _need(mlp["router"], ("experts", "top"), where + ".router")
        shared = mlp.get("shared")
        if shared:
            _need(shared, ("ff",), where + ".shared")
        c = ExpertsConfig(int(mlp["router"]["experts"]), int(mlp["router"]["top"]), int(mlp["expert"]["ff"]),
                          int(shared["ff"]) if shared else None)
        if c.ff <= 0 or not 0 < c.top <= c.experts or (c.shared_ff is not None and c.shared_ff <= 0):
            raise ConfigError(f"{where}: widths must be positive and top within the number of experts")
        return c
    raise ConfigError(f"{where}.kind={kind!r} is not supported (known: 'dense', 'moe')")


@dataclass(frozen=True)
class RobuvikConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[RobuvikLayerConfig, ...]
    bigram: Optional[BigramConfig] = None
    loop: Optional[LoopConfig] = None

    architecture = "Robuvik"

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    def passes(self) -> List[Tuple[int, Optional[int]]]:
        """(layer, pass or None) in the order they run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(n)]
        a, b, times = self.loop.start, self.loop.stop, self.loop.times
        return ([(i, None) for i in range(a)] + [(i, t) for t in range(times) for i in range(a, b)]
                + [(i, None) for i in range(b, n)])

    @staticmethod
    def from_hf_dict(d: Dict[str, Any]) -> "RobuvikConfig":
        _need(d, ("vocab", "width", "norm", "layers"), "config.json")
        _need(d["norm"], ("eps",), "config.json norm")
        layers: List[RobuvikLayerConfig] = []
        for i, layer in enumerate(d["layers"]):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            if layer["type"] == "attention":
                mixer = WindowAttentionConfig.from_dict(layer["mixer"], where + ".mixer")
            elif layer["type"] == "latent_attention":
                mixer = LatentAttentionConfig.from_dict(layer["mixer"], where + ".mixer")
            else:
                raise ConfigError(f"{where}.type={layer['type']!r} is not supported (known: 'attention', "
                                  "'latent_attention')")
            layers.append(RobuvikLayerConfig(mixer, _mlp_from_dict(layer.get("mlp"), where + ".mlp")))
        bigram = (d.get("embedding") or {}).get("bigram")
        if bigram:
            _need(bigram, ("buckets", "mul_prev", "mul_cur"), "config.json embedding.bigram")
            bigram = BigramConfig(int(bigram["buckets"]), int(bigram["mul_prev"]), int(bigram["mul_cur"]))
        else:
            bigram = None
        loop = d.get("loop")
        if loop:
            _need(loop, ("start", "stop", "times"), "config.json loop")
            loop = LoopConfig(int(loop["start"]), int(loop["stop"]), int(loop["times"]))
        else:
            loop = None
        cfg = RobuvikConfig(int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), tuple(layers), bigram, loop)
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.eps <= 0 or not self.layers:
            raise ConfigError("vocab, width and norm.eps must be positive, and there must be layers")
        if self.bigram is not None and (self.bigram.buckets <= 0 or self.bigram.mul_prev < 0 or self.bigram.mul_cur < 0):
            raise ConfigError("embedding.bigram: buckets must be positive, the multipliers not negative")
        if self.loop is not None:
            l = self.loop
            if not 0 <= l.start < l.stop <= len(self.layers) or l.times <= 0:
                raise ConfigError(f"loop: 0 <= start < stop <= {len(self.layers)} and times > 0 are needed, "
                                  f"got {l.start}, {l.stop}, {l.times}")

    def to_hf_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": self.architecture}
        if self.bigram is not None:
            d["embedding"] = {"bigram": self.bigram.to_dict()}
        d["layers"] = [l.to_dict() for l in self.layers]
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        d["norm"] = {"eps": self.eps}
        d.update(vocab=self.vocab, width=self.width)
        return d
