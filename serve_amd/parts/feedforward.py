"""Feed-forwards beside SwiGLU: two products with a plain activation between them, and routed
experts with an optional shared expert.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from ..registry import register_part
from .base import ParamRequest, Part, Runtime, StepCost
from .linear import linear
from .standard import SwiGLU, _prepare_products


class DenseFeedForward(Part):
    """down(act(up x)), no biases; act = one of `ops.ACTIVATIONS` ('gelu_tanh', 'silu', 'relu_squared')."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "gelu_tanh"):
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {sorted(ops.ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size, self.activation = int(hidden_size), int(intermediate_size), activation

    def param_requests(self) -> List[ParamRequest]:
        d, i = self.hidden_size, self.intermediate_size
        return [ParamRequest("up", (i, d), init="normal:0.07"), ParamRequest("down", (d, i), init="normal:0.07")]

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.w_up, self.w_down = tensors["up"], tensors["down"]
        _prepare_products(rt, self.w_up)

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        a = ops.activation(linear(h, self.w_up), self.activation)
        return linear(a, self.w_down, partial_ok=True)


class RoutedExperts(Part):
    """Every token takes the `top` of `experts` small gated feed-forwards (down(silu(gate x) * up x))
    with the largest router logits, weighted by the softmax over the chosen logits alone; the router's
    product gives fp32.  `shared_size`: one more expert of that width runs for every token and is added,
    times sigmoid(w_sg . x) if `shared_gate`.  The tokens are grouped by expert on the device; nothing is
    read back, so steps with this part can be replayed from graphs.

    `activation` / `limit`: another gate of `ops.GATES` in the experts (`shared_limit`: the shared expert's
    limit, if it differs).  `router_softmax="all"`: the weights are the chosen experts' shares of the softmax
    over all experts, divided by their sum (+ 1e-20); `"sigmoid"`: the weights are the sigmoids of the chosen
    logits as they are; `router_scale` multiplies the weights.  `weight_inputs`: a weight multiplies its expert's
    input and not its output (the experts' outputs are then added as they are)."""

    graph_safe = True

    def __init__(self, hidden_size: int, experts: int, top: int, expert_size: int,
                 shared_size: Optional[int] = None, shared_gate: bool = True, activation: str = "silu",
                 limit: float = 0.0, shared_limit: Optional[float] = None, router_softmax: str = "chosen",
                 router_scale: float = 1.0, weight_inputs: bool = False):
        if not 0 < top <= experts:
            raise ValueError("top must be within the number of experts")
        if router_softmax not in ops.ROUTER_MODES:
            raise ValueError(f"router_softmax must be one of {sorted(ops.ROUTER_MODES)}")
        if activation not in ops.GATES:
            raise ValueError(f"unknown gate {activation!r}; known: {sorted(ops.GATES)}")
        self.hidden_size, self.experts, self.top, self.expert_size = int(hidden_size), int(experts), int(top), int(expert_size)
        self.shared_size = None if not shared_size else int(shared_size)
        self.shared_gate = bool(shared_gate) and self.shared_size is not None
        self.activation, self.limit = activation, float(limit)
        self.over_all, self.router_scale = router_softmax, float(router_scale)      # (the router's mode, by name)
        self.weight_inputs = bool(weight_inputs)
        self.shared = None
        if self.shared_size:
            self.shared = SwiGLU(self.hidden_size, self.shared_size, activation,
                                 self.limit if shared_limit is None else float(shared_limit))

    def param_requests(self) -> List[ParamRequest]:
        d, F = self.hidden_size, self.expert_size
        out = [ParamRequest("router", (self.experts, d), init="normal:0.25")]
        for e in range(self.experts):
            out += [ParamRequest(f"e{e}.gate", (F, d), init="normal:0.08"), ParamRequest(f"e{e}.up", (F, d), init="normal:0.08"),
                    ParamRequest(f"e{e}.down", (d, F), init="normal:0.08")]
        if self.shared_size:
            S = self.shared_size
            out += [ParamRequest("shared.gate", (S, d), init="normal:0.08"), ParamRequest("shared.up", (S, d), init="normal:0.08"),
                    ParamRequest("shared.down", (d, S), init="normal:0.08")]
            if self.shared_gate:
                out.append(ParamRequest("shared.sg", (1, d), init="normal:0.1"))
        return out

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        """The router and the shared expert for every token; of the experts, `top` a token: their flops,
        and as weights no more experts than the step's tokens can choose."""
        d, F = self.hidden_size, self.expert_size
        used = min(self.experts, tokens * self.top)
        elements = self.experts * d + used * 3 * F * d
        flops = 2.0 * tokens * self.experts * d + 2.0 * tokens * self.top * 3 * F * d
        if self.shared_size:
            elements += 3 * self.shared_size * d + (d if self.shared_gate else 0)
            flops += 2.0 * tokens * (3 * self.shared_size * d + (d if self.shared_gate else 0))
        return StepCost(elements, flops)

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        E = self.experts
        router = tensors["router"]
        rows = [router] + ([tensors["shared.sg"].to(router.dtype)] if self.shared_gate else [])
        self.w_router = torch.cat(rows, dim=0).contiguous()              # the shared expert's gate rides along
        dt = rt.dtype
        # (gates and ups in one tensor [2, E, F, d]: the kernel for many rows finds an expert's ups E F rows behind its gates)
        gate_up = torch.stack([torch.stack([tensors[f"e{e}.{m}"].to(dt) for e in range(E)]) for m in ("gate", "up")]).contiguous()
        self.w_gate, self.w_up = gate_up[0], gate_up[1]
        self.w_down = torch.stack([tensors[f"e{e}.down"].to(dt) for e in range(E)]).contiguous()
        if self.shared is not None:
            self.shared.load({"gate_proj.weight": tensors["shared.gate"], "up_proj.weight": tensors["shared.up"],
                              "down_proj.weight": tensors["shared.down"]}, rt)
        _prepare_products(rt, self.w_router)

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        T, d = h.shape
        dev = h.device
        logits = linear(h, self.w_router, out_dtype=torch.float32)
        ids = torch.empty((T, self.top), dtype=torch.int32, device=dev)
        weights = torch.empty((T, self.top), dtype=torch.float32, device=dev)
        yk = torch.empty((T * self.top, d), dtype=torch.float32, device=dev)
        if T <= ops.MOE_ROUTE_INSIDE:
            ops.moe_experts(h, ids, self.w_gate, self.w_up, self.w_down, yk, logits, weights, self.over_all,
                            self.router_scale, self.activation, self.limit, self.weight_inputs)    # routes, too
        else:
            ops.moe_route(logits, self.experts, self.top, ids, weights, self.over_all, self.router_scale)
            ops.moe_experts(h, ids, self.w_gate, self.w_up, self.w_down, yk, weights=weights, gate=self.activation,
                            limit=self.limit, weight_inputs=self.weight_inputs)
        shared = self.shared.forward(h, ctx) if self.shared is not None else None
        y = torch.empty((T, d), dtype=torch.float32, device=dev)
        return ops.moe_combine(yk, None if self.weight_inputs else weights, shared,
                               logits if self.shared_gate else None, self.experts, y)


register_part("feed_forward", "dense", DenseFeedForward)
register_part("feed_forward", "routed_experts", RoutedExperts)
