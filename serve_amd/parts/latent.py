"""Latent attention: a token keeps one normed latent vector c [kv_rank] and one rotated key part
[rot_dim] that all heads share; head h's key is [W_uk_h c | rotated part], its value W_uv_h c.

Scores are taken in the latent space, q_h . (W_uk_h c) = (W_uk_h^T q_h) . c: the cached row
[c | rotated part] is the key of one key/value head that every query head reads, c is its value,
and head h's output is W_uv_h applied to the weighted sum of latents.  So the framework's paged
attention kernels (prompt portions and single tokens, both dtypes, windows, cut key ranges) run
over the latent cache as over any other, and only c and the rotated part are kept per token.

A layer may read another layer's cache instead of writing its own (`own_kv=False`, and the run
order gives it that layer's cache): it then has no down-projection, but its own queries, W_uk, W_uv,
window and scale.

Options: `q_rank`: the queries go through a latent of their own, q = W_uq (N(W_dq h) w_dq) (tensors `dq`, `dq.norm`,
`uq` in place of `q`); `out_gate`: the concatenated heads are multiplied element by element with sigmoid(W_g h) before
W_o.  The rotation of the shared key part may pair (i, i + rot_dim / 2) or (2i, 2i + 1): queries and keys are only ever
multiplied with each other, so the second kind is the first after the rows of the projections that make the rotated
parts have been put into the order (even places, odd places), which is done when the part loads.  A rotation with a
magnitude (sine and cosine times a constant) is carried out by the kernels.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops, trace
from ..config.spec import PartSpec
from ..registry import get_part, register_part
from .base import CacheTensor, LayerCache, ParamRequest, Part, Runtime, StepCost, TokenCacheRequest
from .linear import linear
from .standard import _prepare_products

LATENT_MAX_ROW = ops.SIMPLE_ATTENTION_MAX_HEAD_DIM        # the widest cache row the attention kernels take


class LatentAttention(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float,
                 eps: float, position: PartSpec, window: Optional[int] = None, retain: Optional[int] = None,
                 own_kv: bool = True, q_rank: Optional[int] = None, out_gate: bool = False):
        """`window`: a query at position i sees keys j with 0 <= i - j < window (None: all).  `retain`:
        how many keys the cache keeps (None: all): at least the window, and more if another layer
        with a longer window reads this layer's cache."""
        self.hidden_size, self.heads, self.dim, self.rot_dim = int(hidden_size), int(heads), int(dim), int(rot_dim)
        self.vdim, self.kv_rank, self.scale, self.eps = int(vdim), int(kv_rank), float(scale), float(eps)
        self.window, self.retain, self.own_kv = window, retain, bool(own_kv)
        self.q_rank, self.out_gate = None if not q_rank else int(q_rank), bool(out_gate)
        if self.rot_dim % 2:
            raise ValueError("rot_dim must be even")
        if window is not None and retain is not None and retain < window:
            raise ValueError("the cache must keep at least the window")
        self.row = -(-(self.kv_rank + self.rot_dim) // 16) * 16        # a cache row, padded with zeros
        if self.row > LATENT_MAX_ROW:
            raise ValueError(f"kv_rank + rot_dim = {self.kv_rank + self.rot_dim} is above the attention kernels' "
                             f"limit of {LATENT_MAX_ROW}")
        if not isinstance(position, PartSpec):
            position = PartSpec(position["kind"], position["params"])
        self.position = get_part("position", position.kind)(**position.params)

    def param_requests(self) -> List[ParamRequest]:
        d, H, R = self.hidden_size, self.heads, self.kv_rank
        if self.q_rank:
            out = [ParamRequest("dq", (self.q_rank, d), init="normal:0.08"),
                   ParamRequest("dq.norm", (self.q_rank,), init="ones_normal:0.15"),
                   ParamRequest("uq", (H * (self.dim + self.rot_dim), self.q_rank), init="normal:0.12")]
        else:
            out = [ParamRequest("q", (H * (self.dim + self.rot_dim), d), init="normal:0.08")]
        if self.out_gate:
            out.append(ParamRequest("g", (H * self.vdim, d), init="normal:0.08"))
        if self.own_kv:
            out += [ParamRequest("dkv", (R + self.rot_dim, d), init="normal:0.07"),
                    ParamRequest("dkv.norm", (R,), init="ones_normal:0.15")]
        return out + [ParamRequest("uk", (H * self.dim, R), init="normal:0.17"),
                      ParamRequest("uv", (H * self.vdim, R), init="normal:0.12"),
                      ParamRequest("o", (d, H * self.vdim), init="normal:0.07")]

    def cache_request(self) -> Optional[TokenCacheRequest]:
        if not self.own_kv:
            return None
        return TokenCacheRequest((CacheTensor("k", (1, self.row), 1), CacheTensor("v", (1, self.row), 2)), self.retain)

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        cost = super().step_cost(tokens, context_before)
        # uk and uv are applied per head: their default account (tokens x the whole matrix) is right;
        # scores and weighted latents over the keys each token sees
        if self.window:
            keys = sum(min(context_before + j + 1, self.window) for j in range(tokens))
        else:
            keys = tokens * context_before + tokens * (tokens + 1) // 2
        cost.flops += 2.0 * self.heads * (2 * self.kv_rank + self.rot_dim) * keys
        return cost

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        H, R = self.heads, self.kv_rank
        self.position.load({}, rt)
        rot = self.position.rotary()
        if rot is None or rot.rot_dim != self.rot_dim:
            raise ValueError("latent attention rotates the whole shared key part")
        self.inv_freq, self.magnitude = rot.inv_freq, float(rot.magnitude)
        # pairs (2i, 2i + 1) become pairs (i, i + rot_dim / 2) by the order of the rows that make the rotated parts
        order = None
        if rot.adjacent_pairs and self.rot_dim:
            order = torch.cat([torch.arange(0, self.rot_dim, 2), torch.arange(1, self.rot_dim, 2)]).to(rt.device)
        self.wq = tensors["uq"] if self.q_rank else tensors["q"]
        if order is not None:
            per = self.dim + self.rot_dim
            w = self.wq.view(H, per, self.wq.shape[1])
            self.wq = torch.cat([w[:, : self.dim], w[:, self.dim:][:, order]], dim=1).reshape(H * per, -1).contiguous()
        if self.q_rank:
            self.w_dq = tensors["dq"]
            self.q_norm = tensors["dq.norm"].float().contiguous()
        self.w_g = tensors["g"] if self.out_gate else None
        dt = self.wq.dtype
        # [H, dim, R]: the queries' way into the latent space; [H, R, vdim]: the latents' way out
        self.w_uk = tensors["uk"].to(dt).view(H, self.dim, R).contiguous()
        self.w_uv = tensors["uv"].to(dt).view(H, self.vdim, R).transpose(1, 2).contiguous()
        self.wo = tensors["o"]
        if self.own_kv:
            self.w_dkv = tensors["dkv"]
            if order is not None:
                self.w_dkv = torch.cat([self.w_dkv[:R], self.w_dkv[R:][order]], dim=0).contiguous()
            self.latent_norm = tensors["dkv.norm"].float().contiguous()
        _prepare_products(rt, self.wq)

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        H, R, D = self.heads, self.kv_rank, self.row
        T = h.shape[0]
        grp = ctx.groups[cache.group]
        k_pages, v_pages = cache.pages["k"], cache.pages["v"]
        if k_pages.shape[-1] != D:
            raise ValueError(f"the cache keeps rows of {k_pages.shape[-1]}, this layer reads rows of {D}")
        with trace.span("write_to_cache"):
            if writes_cache:
                if not self.own_kv:
                    raise ValueError("a latent attention without a down-projection cannot write a cache")
                z = linear(h, self.w_dkv)
                ops.latent_kv_write(z, self.latent_norm, ctx.positions, self.inv_freq, grp.slots, k_pages, v_pages,
                                    self.eps, R, self.rot_dim, self.magnitude)
            if self.q_rank:
                # the queries' own latent: the product's fp32 sums are normed as a norm norms the stream
                zq = linear(h, self.w_dq, out_dtype=torch.float32)
                cq = ops.add_rmsnorm(zq, None, self.q_norm, self.eps, self.rt.empty((T, self.q_rank)))
                q = linear(cq, self.wq)
            else:
                q = linear(h, self.wq)
            qf = self.rt.empty((T, H * D))
            # the queries into the latent space, their rotated parts behind them, zeros up to the row's end
            ops.head_linear(q, q.shape[1], self.dim + self.rot_dim, self.w_uk, qf, H * D, D, T, ctx.positions,
                            self.inv_freq, self.rot_dim, D - R, self.magnitude)
        attn = self.rt.empty((T, H * D))
        with trace.span("attention"):
            ops.paged_attention(qf, H * D, attn, k_pages, v_pages, grp.block_table, ctx, H, self.scale, self.window)
        o = self.rt.empty((T, H * self.vdim))
        ops.head_linear(attn, H * D, D, self.w_uv, o, H * self.vdim, self.vdim, T)
        if self.out_gate:
            ops.sigmoid_mul(o, linear(h, self.w_g))
        return linear(o, self.wo, partial_ok=True)


register_part("mixer", "latent_attention", LatentAttention)
