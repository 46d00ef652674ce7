"""Typed configuration of the Kotipel decoder, read from config.json's own keys.

config.json gives `vocab`, `width`, `norm.eps`, `layers` (a list whose entries name the layer's mixer
by `type`: "parallel" = a gated softmax attention (`mixer.left`) beside a gated linear attention
(`mixer.right`), or "mamba2" = a selective state-space mixer; the mixer's sizes and constants in
`mixer`; the feed-forward in `mlp`: null or {"kind": "dense", "ff", "limit"}), optionally `loop`
({"start", "stop", "times"}: layers start .. stop-1 run `times` times in a row with the same weights)
and optionally `token_side` ({"dim"}: every layer ends with an input made from a second embedding row
of the token).  Layers differ from each other; nothing about them stands in code.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple, Union

from .llama import ConfigError


def _need(d: Dict[str, Any], keys, where: str) -> None:
    if not isinstance(d, dict):
        raise ConfigError(f"{where} must be an object")
    missing = [k for k in keys if k not in d]
    if missing:
        raise ConfigError(f"{where} lacks the keys {missing}")


@dataclass(frozen=True)
class RotScaling:
    factor: float
    low: float
    high: float
    original: float

    def to_dict(self) -> Dict[str, Any]:
        o = self.original
        return {"factor": self.factor, "high": self.high, "low": self.low, "original": int(o) if o == int(o) else o}


@dataclass(frozen=True)
class GatedAttentionConfig:
    """The left half of a parallel layer."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    rot_scaling: Optional[RotScaling]

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "GatedAttentionConfig":
        _need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
        rot = m.get("rot")
        dims, base, scaling = 0, 10000.0, None
        if rot:
            _need(rot, ("base", "dims"), where + ".rot")
            dims, base = int(rot["dims"]), float(rot["base"])
            s = rot.get("scaling")
            if s:
                _need(s, ("factor", "low", "high", "original"), where + ".rot.scaling")
                scaling = RotScaling(float(s["factor"]), float(s["low"]), float(s["high"]), float(s["original"]))
                if scaling.factor <= 0 or scaling.original <= 0 or scaling.high == scaling.low:
                    raise ConfigError(f"{where}.rot.scaling: factor and original must be positive, high and low differ")
        c = GatedAttentionConfig(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                                 dims, base, scaling)
        if min(c.heads, c.kv_heads, c.dim, c.vdim) <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"{where}: sizes must be positive and heads a multiple of kv_heads")
        if c.rot_dims < 0 or c.rot_dims % 2 or c.rot_dims > c.dim or c.rot_base <= 0:
            raise ConfigError(f"{where}.rot: dims must be even and within dim, base positive")
        return c

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads}
        if self.rot_dims:
            rot: Dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling is not None:
                rot["scaling"] = self.rot_scaling.to_dict()
            d["rot"] = rot
        d.update(scale=self.scale, vdim=self.vdim)
        return d


@dataclass(frozen=True)
class LinearAttentionConfig:
    """The right half of a parallel layer."""
    heads: int
    dim: int
    vdim: int
    tau: float
    # the width between the decay's two matrices: the checkpoint's tensors give it; a configuration for random weights
    # names it (key `decay_rank`, written only then)
    decay_rank: Optional[int] = None

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "LinearAttentionConfig":
        _need(m, ("heads", "dim", "vdim", "tau"), where)
        rank = m.get("decay_rank")
        c = LinearAttentionConfig(int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"]),
                                  None if rank is None else int(rank))
        if min(c.heads, c.dim, c.vdim) <= 0 or not c.tau > 0 or (c.decay_rank is not None and c.decay_rank <= 0):
            raise ConfigError(f"{where}: sizes and tau must be positive")
        return c

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {}
        if self.decay_rank is not None:
            d["decay_rank"] = self.decay_rank
        d.update(dim=self.dim, heads=self.heads, tau=self.tau, vdim=self.vdim)
        return d


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: GatedAttentionConfig
    right: LinearAttentionConfig

    def to_dict(self) -> Dict[str, Any]:
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class StateSpaceMixerConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "StateSpaceMixerConfig":
        _need(m, ("heads", "vdim", "state", "groups", "conv", "norm_groups"), where)
        c = StateSpaceMixerConfig(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]),
                                  int(m["norm_groups"]))
        if min(c.heads, c.vdim, c.state, c.groups, c.conv, c.norm_groups) <= 0:
            raise ConfigError(f"{where}: sizes must be positive")
        if c.heads % c.groups or (c.heads * c.vdim) % c.norm_groups:
            raise ConfigError(f"{where}: heads must be a multiple of groups, heads * vdim of norm_groups")
        return c

    def to_dict(self) -> Dict[str, Any]:
        return {"conv": self.conv, "groups": self.groups, "heads": self.heads, "norm_groups": self.norm_groups,
                "state": self.state, "vdim": self.vdim}


@dataclass(frozen=True)
class ClampedDenseConfig:
    ff: int
    limit: float

    def to_dict(self) -> Dict[str, Any]:
        return {"ff": self.ff, "kind": "dense", "limit": self.limit}


@dataclass(frozen=True)
class KotipelLayerConfig:
    mixer: Union[ParallelMixerConfig, StateSpaceMixerConfig]
    mlp: Optional[ClampedDenseConfig]

    @property
    def type(self) -> str:
        return "parallel" if isinstance(self.mixer, ParallelMixerConfig) else "mamba2"

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int

    def to_dict(self) -> Dict[str, Any]:
        return {"start": self.start, "stop": self.stop, "times": self.times}


@dataclass(frozen=True)
class KotipelConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[KotipelLayerConfig, ...]
    loop: Optional[LoopConfig] = None
    side_dim: Optional[int] = None

    architecture = "Kotipel"

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
    def from_hf_dict(d: Dict[str, Any]) -> "KotipelConfig":
        _need(d, ("vocab", "width", "norm", "layers"), "config.json")
        _need(d["norm"], ("eps",), "config.json norm")
        layers: List[KotipelLayerConfig] = []
        for i, layer in enumerate(d["layers"]):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            if layer["type"] == "parallel":
                _need(layer["mixer"], ("left", "right"), where + ".mixer")
                mixer = ParallelMixerConfig(GatedAttentionConfig.from_dict(layer["mixer"]["left"], where + ".mixer.left"),
                                            LinearAttentionConfig.from_dict(layer["mixer"]["right"], where + ".mixer.right"))
            elif layer["type"] == "mamba2":
                mixer = StateSpaceMixerConfig.from_dict(layer["mixer"], where + ".mixer")
            else:
                raise ConfigError(f"{where}.type={layer['type']!r} is not supported (known: 'parallel', 'mamba2')")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}.mlp.kind={mlp.get('kind')!r} is not supported (known: 'dense')")
                _need(mlp, ("ff", "limit"), where + ".mlp")
                mlp = ClampedDenseConfig(int(mlp["ff"]), float(mlp["limit"]))
                if mlp.ff <= 0 or not mlp.limit > 0:
                    raise ConfigError(f"{where}.mlp: ff and limit must be positive")
            layers.append(KotipelLayerConfig(mixer, mlp))
        loop = d.get("loop")
        if loop:
            _need(loop, ("start", "stop", "times"), "config.json loop")
            loop = LoopConfig(int(loop["start"]), int(loop["stop"]), int(loop["times"]))
        else:
            loop = None
        side = d.get("token_side")
        side_dim = None
        if side:
            _need(side, ("dim",), "config.json token_side")
            side_dim = int(side["dim"])
        cfg = KotipelConfig(int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), tuple(layers), loop, side_dim)
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.eps <= 0 or not self.layers:
            raise ConfigError("vocab, width and norm.eps must be positive, and there must be layers")
        if self.loop is not None:
            l = self.loop
            if not 0 <= l.start < l.stop <= len(self.layers) or l.times <= 0:
                raise ConfigError(f"loop: 0 <= start < stop <= {len(self.layers)} and times > 0 are needed, "
                                  f"got {l.start}, {l.stop}, {l.times}")
        if self.side_dim is not None and self.side_dim <= 0:
            raise ConfigError("token_side.dim must be positive")

    def to_hf_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers]}
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        d["norm"] = {"eps": self.eps}
        if self.side_dim is not None:
            d["token_side"] = {"dim": self.side_dim}
        d.update(vocab=self.vocab, width=self.width)
        return d
