"""Grouped-query softmax attention whose queries and keys are normed over the whole projection, then rotated,
and whose heads pass an output gate:

    q = N(W_q h) * w_qn,   k = N(W_k h) * w_kn        N over all heads' values of a token at once, before the split
    q, k <- rotation by position of the first rot dims of every head (the position part says which)
    o_h = softmax(q_h . k_g * scale over the keys j <= i) v_g * sigmoid(W_g h)_h       g = h // (heads / kv_heads)
    out = W_o [o_1 .. o_H]

Keys have `dim` dims and values `vdim`: the cache and the attention kernels work on one padded head size (the
places behind are zeros), so the framework's paged attention kernels run unchanged.  `out_gate=False` leaves the
gate out (no `g` tensor then).
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


class GatedRotaryAttention(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, scale: float,
                 eps: float, position: Optional[PartSpec] = None, out_gate: bool = True, window: Optional[int] = None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.scale, self.eps = int(dim), int(vdim), float(scale), float(eps)
        self.out_gate, self.window = bool(out_gate), window
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
               ParamRequest("v", (G * Dv, d), init="normal:0.08"),
               ParamRequest("q.norm", (H * D,), init="ones_normal:0.2"),
               ParamRequest("k.norm", (G * D,), init="ones_normal:0.2")]
        if self.out_gate:
            out.append(ParamRequest("g", (H, d), init="normal:0.08"))
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
        parts = [tensors["q"], tensors["k"], tensors["v"]] + ([tensors["g"]] if self.out_gate else [])
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        self.w_in = torch.cat([p.to(dt) for p in parts], dim=0).contiguous()     # one product: q | k | v | gate logits
        self.gate_col = H * self.dim + self.num_kv_heads * (self.dim + Dv)
        wo = tensors["o"]
        if Dp != Dv:
            # the attention's output rows hold Dp places a head, of which the last Dp - Dv are zeros
            padded = torch.zeros((self.hidden_size, H, Dp), dtype=wo.dtype, device=wo.device)
            padded[:, :, :Dv] = wo.view(self.hidden_size, H, Dv)
            wo = padded.view(self.hidden_size, H * Dp)
        self.wo = wo.contiguous()
        self.q_norm = tensors["q.norm"].float().contiguous()
        self.k_norm = tensors["k.norm"].float().contiguous()
        self.inv_freq, self.rot_dim = None, 0
        if self.position is not None:
            self.position.load({}, rt)
            rot = self.position.rotary()
            if rot is None or rot.adjacent_pairs or rot.magnitude != 1.0:
                raise ValueError("this attention takes a plain rotation of the pairs (i, i + rot/2), or no position part")
            self.inv_freq, self.rot_dim = rot.inv_freq.contiguous(), int(rot.rot_dim)
            if self.rot_dim > self.dim:
                raise ValueError(f"a rotation of {self.rot_dim} dims does not fit heads of {self.dim}")
        _prepare_products(rt, self.w_in)

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        H, G, D, Dv, Dp = self.num_heads, self.num_kv_heads, self.dim, self.vdim, self.head_size
        T = h.shape[0]
        grp = ctx.groups[cache.group]
        if cache.k_pages.shape[-1] != Dp:
            raise ValueError(f"the cache keeps heads of {cache.k_pages.shape[-1]}, this layer works on {Dp}")
        with trace.span("write_to_cache"):
            z = linear(h, self.w_in)
            q = self.rt.empty((T, H * Dp))
            ops.row_norm_rope_kv_write(z, q, ctx.positions, grp.slots if writes_cache else None, cache.k_pages,
                                       cache.v_pages, self.q_norm, self.k_norm, self.eps, self.inv_freq, self.rot_dim,
                                       H, G, D, Dv)
        attn = self.rt.empty((T, H * Dp))
        with trace.span("attention"):
            ops.paged_attention(q, H * Dp, attn, cache.k_pages, cache.v_pages, grp.block_table, ctx, H, self.scale,
                                self.window)
        if self.out_gate:
            ops.head_gate(attn, z, self.gate_col, H)
        return linear(attn, self.wo, partial_ok=True)      # the consumer adds the parts


register_part("mixer", "gated_rotary_attention", GatedRotaryAttention)
