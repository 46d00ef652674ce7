"""Two mixers side by side that read the same input; their outputs are each divided by their root mean square
over the model width, multiplied by a weight of their own and averaged:

    out = (N(left(h)) w_left + N(right(h)) w_right) / 2           N(y) = y / sqrt(mean(y^2) + eps)

The two mixers are parts like any others (any registered mixer kinds); their tensors are named `left.*` and
`right.*`, the two weights `left.out` and `right.out`.  At most one of the two may keep per-token cache; their
per-request states lie one behind the other in the layer's state row.

`ParallelResidual` (an arrangement) is the other kind of side by side: a mixer and a feed-forward behind ONE norm,

    h = N(x) w;   x <- x + mixer(h) + ff(h)
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..config.spec import PartSpec
from ..registry import get_part, register_part
from .base import LayerCache, ParamRequest, Part, Runtime, StateRequest, StepCost, TokenCacheRequest

SIDES = ("left", "right")


class ParallelMixers(Part):
    def __init__(self, hidden_size: int, eps: float, left: PartSpec, right: PartSpec):
        self.hidden_size, self.eps = int(hidden_size), float(eps)
        self.sides: Dict[str, Part] = {}
        for name, spec in zip(SIDES, (left, right)):
            if not isinstance(spec, PartSpec):
                spec = PartSpec(spec["kind"], spec["params"])
            self.sides[name] = get_part("mixer", spec.kind)(**spec.params)
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in self.sides.values())
        if sum(p.cache_request() is not None for p in self.sides.values()) > 1:
            raise ValueError("only one of two parallel mixers may keep per-token cache")
        for p in self.sides.values():
            sr = p.state_request()
            if sr is not None and (len(sr.shape) != 1 or sr.dtype != torch.float32):
                raise ValueError("parallel mixers share a state row: each state must be one fp32 row")

    def param_requests(self) -> List[ParamRequest]:
        out = []
        for name, p in self.sides.items():
            for pr in p.param_requests():
                if pr.alias_of is not None:
                    raise ValueError("a mixer inside parallel mixers cannot share another part's tensor")
                out.append(ParamRequest(f"{name}.{pr.name}", pr.shape, pr.init, pr.optional))
            out.append(ParamRequest(f"{name}.out", (self.hidden_size,), init="ones_normal"))
        return out

    def cache_request(self) -> Optional[TokenCacheRequest]:
        for p in self.sides.values():
            if p.cache_request() is not None:
                return p.cache_request()
        return None

    def _state_ranges(self):
        at, out = 0, {}
        for name, p in self.sides.items():
            sr = p.state_request()
            if sr is not None:
                out[name] = (at, at + int(sr.shape[0]))
                at += int(sr.shape[0])
        return out, at

    def state_request(self) -> Optional[StateRequest]:
        _, total = self._state_ranges()
        return StateRequest((total,), torch.float32) if total else None

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        cost = StepCost(2 * self.hidden_size, 0.0)
        for p in self.sides.values():
            c = p.step_cost(tokens, context_before)
            cost.weight_elements += c.weight_elements
            cost.flops += c.flops
        return cost

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.out_w = {}
        for name, p in self.sides.items():
            prefix = name + "."
            own = {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix) and k != prefix + "out"}
            p.load(own, rt)
            self.out_w[name] = tensors[prefix + "out"].float().contiguous()
        self.ranges, _ = self._state_ranges()

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        outs = []
        for name, p in self.sides.items():
            sub = LayerCache(group=cache.group, pages=cache.pages, page_size=cache.page_size)
            if name in self.ranges:
                lo, hi = self.ranges[name]
                sub.state = cache.state[:, lo:hi]
            outs.append(p.forward(h, ctx, sub, writes_cache))
        out = torch.empty((h.shape[0], self.hidden_size), dtype=torch.float32, device=h.device)
        return ops.dual_norm_mix(outs[0], outs[1], self.out_w["left"], self.out_w["right"], 0.5, 0.5, self.eps, out)


class ParallelResidual:
    """x <- x + mixer(h) + ffn(h), h = norm(x): one norm a layer, and both sublayers read its output.

    As in the other arrangements the additions are folded into later kernels: the mixer's output joins the stream in
    one pass of its own (`stream_add`), the feed-forward's is returned as what is still to be added and rides in the
    next layer's norm.  A layer may have no feed-forward."""

    PART_ROLES = {"mixer": "mixer", "ffn": "feed_forward", "norm": "norm"}
    OPTIONAL_PARTS = ("ffn",)

    def __init__(self, mixer, norm, ffn=None):
        self.mixer, self.norm, self.ffn = mixer, norm, ffn

    def cache_owner(self) -> Part:
        return self.mixer

    def parts(self) -> Dict[str, Part]:
        out = {"mixer": self.mixer, "norm": self.norm}
        if self.ffn is not None:
            out["ffn"] = self.ffn
        return out

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], ctx, cache: LayerCache,
                writes_cache: bool = True) -> Optional[torch.Tensor]:
        h = self.norm.forward(x, pending)
        a = self.mixer.forward(h, ctx, cache, writes_cache)
        if self.ffn is None:
            return a
        b = self.ffn.forward(h, ctx)
        ops.stream_add(x, a)
        return b


register_part("mixer", "parallel", ParallelMixers)
register_part("arrangement", "parallel_residual", ParallelResidual)
