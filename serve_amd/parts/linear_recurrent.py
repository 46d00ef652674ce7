"""Mixers whose memory is one fp32 matrix per head and request that decays and takes an outer product a token:

    S_t = diag(a_t) S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t

`GatedLinearAttention`: q = W_q h * dim^-1/2, k = W_k h (heads x dim), v = W_v h (heads x vdim); a decay per key
channel a = sigmoid(W_a2 (W_a1 h) + b)^(1/tau); the read-out of every head over its root mean square, times a weight
shared by the heads, times silu(W_g h), then W_o.

`StateSpaceMixer` (the selective state-space mixer in its state-space-duality form): W_in h = [z | x | B | C | dt] with
inner = heads * vdim, B and C of groups * state; x, B, C pass a causal convolution per channel (`conv` taps, bias) and
silu; dt = softplus(dt + dt_bias); per head S [state, vdim] with a = exp(-exp(A_log) dt), k = B, v = dt x, q = C
(head h reads group h // (heads / groups)); y = S^T C + D x, times silu(z), over the root mean square of each of
`norm_groups` equal parts, times a weight, then W_o.

Per-request state (fp32, zero at admission): the matrices S in the recurrence kernel's own layout, and for the
state-space mixer the convolution's last conv - 1 inputs behind them.  Decays, their logarithms, softplus,
exponentials, step sizes and the recurrence are fp32 in both engines; the decay's and the step size's logits come
from products with fp32 results.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from ..registry import register_part
from .base import LayerCache, ParamRequest, Part, Runtime, StateRequest, StepCost
from .linear import linear
from .standard import _prepare_products


def _same_dtype(tensors) -> torch.dtype:
    return tensors[0].dtype if all(t.dtype == tensors[0].dtype for t in tensors) else torch.float32


class GatedLinearAttention(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, heads: int, dim: int, vdim: int, tau: float, eps: float,
                 decay_rank: Optional[int] = None):
        """`decay_rank`: the width between the decay's two matrices; None: whatever the checkpoint's tensors have."""
        if not (0 < dim <= ops.SCAN_MAX_DIM and vdim > 0 and heads > 0 and tau > 0) or (decay_rank is not None and decay_rank <= 0):
            raise ValueError(f"key sizes up to {ops.SCAN_MAX_DIM} are taken; got heads {heads}, dim {dim}, vdim {vdim}, "
                             f"decay_rank {decay_rank}, tau {tau}")
        self.hidden_size, self.heads, self.dim, self.vdim = int(hidden_size), int(heads), int(dim), int(vdim)
        self.tau, self.eps = float(tau), float(eps)
        self.decay_rank = -1 if decay_rank is None else int(decay_rank)

    def param_requests(self) -> List[ParamRequest]:
        d, H, D, Dv, r = self.hidden_size, self.heads, self.dim, self.vdim, self.decay_rank
        return [ParamRequest("q", (H * D, d), init="normal:0.08"), ParamRequest("k", (H * D, d), init="normal:0.08"),
                ParamRequest("v", (H * Dv, d), init="normal:0.08"), ParamRequest("g", (H * Dv, d), init="normal:0.08"),
                ParamRequest("o", (d, H * Dv), init="normal:0.08"), ParamRequest("norm", (Dv,), init="ones_normal:0.15"),
                ParamRequest("a1", (r, d), init="normal:0.08"), ParamRequest("a2", (H * D, r), init="normal:0.5"),
                ParamRequest("a2.b", (H * D,), init="uniform:2:6")]

    def state_request(self) -> StateRequest:
        return StateRequest((ops.decay_scan_state_floats(self.heads, self.dim, self.vdim),), torch.float32)

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        """The projections, and per token and head the decay with the outer product and the read-out: 4 dim vdim flops."""
        cost = super().step_cost(tokens, context_before)
        cost.flops += 4.0 * tokens * self.heads * self.dim * self.vdim
        return cost

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        big = [tensors[n] for n in ("q", "k", "v", "g")]
        dt = _same_dtype(big)
        self.w_in = torch.cat([t.to(dt) for t in big], dim=0).contiguous()        # one product: q | k | v | gate
        self.w_a1, self.w_a2 = tensors["a1"], tensors["a2"]
        if self.w_a1.shape[0] != self.w_a2.shape[1]:
            raise ValueError(f"the decay's matrices do not fit: {list(self.w_a1.shape)} and {list(self.w_a2.shape)}")
        self.a_bias = tensors["a2.b"].float().contiguous()
        self.norm_w = tensors["norm"].float().contiguous()
        self.wo = tensors["o"]
        _prepare_products(rt, self.w_in)

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        if cache.state is None:
            raise ValueError("the linear attention needs its per-request state")
        H, D, Dv = self.heads, self.dim, self.vdim
        T = h.shape[0]
        z = linear(h, self.w_in)
        logits = linear(linear(h, self.w_a1), self.w_a2, out_dtype=torch.float32)      # what enters the recurrence is fp32
        decay = ops.gla_decay(logits, self.a_bias, self.tau, logits)                   # in place
        o = torch.empty((T, H * Dv), dtype=torch.float32, device=h.device)
        ops.decay_scan(z[:, : H * D], z[:, H * D: 2 * H * D], z[:, 2 * H * D: 2 * H * D + H * Dv], decay.view(T, H, D),
                       cache.state, 0, ctx, o, H, H, D, Dv, q_scale=D ** -0.5)
        y = self.rt.empty((T, H * Dv))
        ops.gated_group_norm(o, z, 2 * H * D + H * Dv, self.norm_w, Dv, False, self.eps, y)
        return linear(y, self.wo, partial_ok=True)


class StateSpaceMixer(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, heads: int, vdim: int, state: int, groups: int, conv: int, norm_groups: int,
                 eps: float):
        if heads % groups or (heads * vdim) % norm_groups:
            raise ValueError("heads must be a multiple of groups, heads * vdim of norm_groups")
        if not (0 < state <= ops.SCAN_MAX_DIM and vdim > 0 and 1 <= conv <= ops.SCAN_MAX_TAPS):
            raise ValueError(f"states up to {ops.SCAN_MAX_DIM} and up to {ops.SCAN_MAX_TAPS} taps are taken; got state "
                             f"{state}, vdim {vdim}, conv {conv}")
        self.hidden_size, self.heads, self.vdim, self.state = int(hidden_size), int(heads), int(vdim), int(state)
        self.groups, self.taps, self.norm_groups, self.eps = int(groups), int(conv), int(norm_groups), float(eps)
        self.inner = self.heads * self.vdim
        self.channels = self.inner + 2 * self.groups * self.state          # what the convolution sees
        self.scan_floats = ops.decay_scan_state_floats(self.heads, self.state, self.vdim)

    def param_requests(self) -> List[ParamRequest]:
        d, H, C, taps = self.hidden_size, self.heads, self.channels, self.taps
        return [ParamRequest("in", (2 * self.inner + 2 * self.groups * self.state + H, d), init="normal:0.08"),
                ParamRequest("conv", (C, taps), init="normal:0.5"), ParamRequest("conv.b", (C,), init="normal:0.1"),
                ParamRequest("dt_bias", (H,), init="uniform:-3:0"), ParamRequest("A_log", (H,), init="uniform:-2:1"),
                ParamRequest("D", (H,), init="ones_normal:0.3"), ParamRequest("norm", (self.inner,), init="ones_normal:0.15"),
                ParamRequest("o", (d, self.inner), init="normal:0.08")]

    def state_request(self) -> StateRequest:
        return StateRequest((self.scan_floats + (self.taps - 1) * self.channels,), torch.float32)

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        cost = super().step_cost(tokens, context_before)
        cost.flops += 4.0 * tokens * self.heads * self.state * self.vdim
        return cost

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        w = tensors["in"]
        n = self.inner + self.channels
        self.w_zx = w[:n].contiguous()               # z | x | B | C in the activation dtype
        self.w_dt = w[n:].contiguous()               # the step sizes' logits: their product gives fp32
        self.conv_w = tensors["conv"].float().contiguous()
        self.conv_b = tensors["conv.b"].float().contiguous()
        self.A_log = tensors["A_log"].float().contiguous()
        self.dt_bias = tensors["dt_bias"].float().contiguous()
        self.D = tensors["D"].float().contiguous()
        self.norm_w = tensors["norm"].float().contiguous()
        self.wo = tensors["o"]
        _prepare_products(rt, self.w_zx)

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        if cache.state is None:
            raise ValueError("the state-space mixer needs its per-request state")
        H, P, N, G, C, inner = self.heads, self.vdim, self.state, self.groups, self.channels, self.inner
        T = h.shape[0]
        zx = linear(h, self.w_zx)
        dt_raw = linear(h, self.w_dt, out_dtype=torch.float32)
        f32 = dict(dtype=torch.float32, device=h.device)
        xbc, v, decay = torch.empty((T, C), **f32), torch.empty((T, inner), **f32), torch.empty((T, H), **f32)
        ops.ssm_prepare(zx, inner, self.conv_w, self.conv_b, cache.state, self.scan_floats, dt_raw, self.A_log,
                        self.dt_bias, ctx, xbc, v, decay, H, P, self.taps)
        if self.taps > 1:
            ops.conv_state_update(zx, inner, C, cache.state, self.scan_floats, ctx, self.taps)
        o = torch.empty((T, inner), **f32)
        ops.decay_scan(xbc[:, inner + G * N:], xbc[:, inner: inner + G * N], v, decay, cache.state, 0, ctx, o, H, G, N, P)
        y = self.rt.empty((T, inner))
        ops.gated_group_norm(o, zx, 0, self.norm_w, inner // self.norm_groups, True, self.eps, y,
                             skip_x=xbc, skip_d=self.D, head_dim=P)
        return linear(y, self.wo, partial_ok=True)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "state_space", StateSpaceMixer)
