"""Grouped-query softmax attention with the options of plain (un-normed) queries and keys:

    q = W_q h (+ b_q),  k = W_k h (+ b_k),  v = W_v h (+ b_v)
    q, k <- the first rot dims of every head turned by the position (the position part says which pairs, which
            frequencies, and by what magnitude sine and cosine are multiplied)
    w_ij = exp(s_ij) / (sum_j exp(s_ij) + exp(sink)),  s_ij = scale q_i . k_j   over 0 <= i - j (< window)
    out  = W_o [o_1 .. o_H],  o_h = sum_j w_ij v_j of key/value head h // (heads / kv_heads)

`bias`: the three projections have biases (tensors `q.b`, `k.b`, `v.b`).  `sink`: a constant logit that takes part in
the softmax's denominator and has no value (0.0: "one added to the denominator"); None: the ordinary softmax.
Keys have `dim` dims and values `vdim`: the cache and the attention kernels work on one padded head size (the places
behind are zeros), so the framework's paged attention kernels run unchanged.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops, trace
from ..config.spec import PartSpec
from ..registry import get_part, register_part
from .base import LayerCache, ParamRequest, Part, Runtime, StepCost, TokenCacheRequest, kv_cache_request
from .linear import linear
from .normed_attention import padded_head_size
from .standard import _prepare_products


class RotaryAttention(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, scale: float,
                 position: Optional[PartSpec] = None, bias: bool = False, sink: Optional[float] = None,
                 window: Optional[int] = None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if window is not None and int(window) <= 0:
            raise ValueError("a window holds at least the token itself")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.scale = int(dim), int(vdim), float(scale)
        self.bias, self.sink = bool(bias), None if sink is None else float(sink)
        self.window = None if window is None else int(window)
        self.head_size = padded_head_size(self.dim, self.vdim)
        if self.head_size > ops.SIMPLE_ATTENTION_MAX_HEAD_DIM:
            raise ValueError(f"head sizes up to {ops.SIMPLE_ATTENTION_MAX_HEAD_DIM} are taken, got {self.head_size}")
        self.position = None
        if position is not None:
            if not isinstance(position, PartSpec):
                position = PartSpec(position["kind"], position["params"])
            self.position = get_part("position", position.kind)(**position.params)
            self.graph_safe = bool(getattr(self.position, "graph_safe", False))

    def param_requests(self) -> List[ParamRequest]:
        d, H, G, D, Dv = self.hidden_size, self.num_heads, self.num_kv_heads, self.dim, self.vdim
        out = [ParamRequest("q", (H * D, d), init="normal:0.08"), ParamRequest("k", (G * D, d), init="normal:0.08"),
               ParamRequest("v", (G * Dv, d), init="normal:0.08")]
        if self.bias:
            out += [ParamRequest("q.b", (H * D,), init="normal:0.3"), ParamRequest("k.b", (G * D,), init="normal:0.3"),
                    ParamRequest("v.b", (G * Dv,), init="normal:0.3")]
        return out + [ParamRequest("o", (d, H * Dv), init="normal:0.08")]

    def cache_request(self) -> TokenCacheRequest:
        return kv_cache_request(self.num_kv_heads, self.head_size, self.window)

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        """The projections, and scores (dim) and weighted values (vdim) over the keys each token sees."""
        cost = super().step_cost(tokens, context_before)
        if self.window:
            keys = sum(min(context_before + j + 1, self.window) for j in range(tokens))
        else:
            keys = tokens * context_before + tokens * (tokens + 1) // 2
        cost.flops += 2.0 * self.num_heads * (self.dim + self.vdim) * keys
        return cost

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        H, Dv, Dp = self.num_heads, self.vdim, self.head_size
        parts = [tensors["q"], tensors["k"], tensors["v"]]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        self.w_in = torch.cat([p.to(dt) for p in parts], dim=0).contiguous()     # one product: q | k | v
        self.b_in = None
        if self.bias:
            self.b_in = torch.cat([tensors[n].float() for n in ("q.b", "k.b", "v.b")]).contiguous()
        wo = tensors["o"]
        if Dp != Dv:
            # the attention's output rows hold Dp places a head, of which the last Dp - Dv are zeros
            padded = torch.zeros((self.hidden_size, H, Dp), dtype=wo.dtype, device=wo.device)
            padded[:, :, :Dv] = wo.view(self.hidden_size, H, Dv)
            wo = padded.view(self.hidden_size, H * Dp)
        self.wo = wo.contiguous()
        self.inv_freq, self.rot_dim, self.adjacent, self.magnitude = None, 0, False, 1.0
        if self.position is not None:
            self.position.load({}, rt)
            rot = self.position.rotary()
            if rot is None:
                raise ValueError("this attention takes a rotation (a position part with `rotary()`), or no position part")
            self.inv_freq, self.rot_dim = rot.inv_freq.contiguous(), int(rot.rot_dim)
            self.adjacent, self.magnitude = bool(rot.adjacent_pairs), float(rot.magnitude)
            if self.rot_dim > self.dim:
                raise ValueError(f"a rotation of {self.rot_dim} dims does not fit heads of {self.dim}")
        self.sinks = None
        if self.sink is not None:
            self.sinks = torch.full((H,), self.sink, dtype=torch.float32, device=rt.device)
        _prepare_products(rt, self.w_in)

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        H, G, D, Dv, Dp = self.num_heads, self.num_kv_heads, self.dim, self.vdim, self.head_size
        T = h.shape[0]
        grp = ctx.groups[cache.group]
        if cache.k_pages.shape[-1] != Dp:
            raise ValueError(f"the cache keeps heads of {cache.k_pages.shape[-1]}, this layer works on {Dp}")
        with trace.span("write_to_cache"):
            q = self.rt.empty((T, H * Dp))
            if (writes_cache and D == Dv == Dp and self.rot_dim == D
                    and ops.qkv_rope_available(h, self.w_in, cache.k_pages, D, self.rot_dim, self.adjacent)):
                # few rows, whole heads rotated, keys and values of one size: product, biases, rotation and cache
                # write are one kernel (the biases join the fp32 sums)
                ops.qkv_rope_bf16(h, self.w_in, q, ctx.positions, self.inv_freq, grp.slots, cache.k_pages,
                                  cache.v_pages, H, G, D, cache.page_size, self.b_in, self.magnitude)
                z = None
            else:
                z = linear(h, self.w_in)
        if z is not None:
            ops.bias_rope_kv_write(z, q, ctx.positions, grp.slots if writes_cache else None, cache.k_pages,
                                   cache.v_pages, self.b_in, self.inv_freq, self.rot_dim, self.adjacent, self.magnitude,
                                   H, G, D, Dv)
        attn = self.rt.empty((T, H * Dp))
        with trace.span("attention"):
            ops.paged_attention(q, H * Dp, attn, cache.k_pages, cache.v_pages, grp.block_table, ctx, H, self.scale,
                                self.window, sinks=self.sinks)
        return linear(attn, self.wo, partial_ok=True)      # the consumer adds the parts


register_part("mixer", "rotary_attention", RotaryAttention)
