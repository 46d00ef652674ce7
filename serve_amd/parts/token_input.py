"""Inputs to the residual stream beside the token embedding.

`GatedSideEmbedding` (role `token_input`, the last part of a layer): with e the layer's slice of a second embedding
row of the token, and x the stream after the layer's sublayers,

    g = gelu_tanh(W_gate x) * e;    y = W_proj g;    x <- x + y / sqrt(mean(y^2) + eps) * w

The second table is the embedding part's (`embedding.side`); a layer reads the columns [offset, offset + dim).

`PassVectors` (role `stream_input`, a part of the model): a table [rows, width] of which the run order adds one row to
the stream before an entry runs (and, where the entry says so, the embedding's output once more).

`PairEmbedding` (role `embedding`): the token's row plus a row of a second table chosen by a hash of the pair
(previous token, token); the previous token of a request is per-request state.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from ..registry import register_part
from .base import NORMED_STREAM, LayerCache, ParamRequest, Part, Runtime, StateRequest, StepCost
from .linear import linear


class GatedSideEmbedding(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, vocab_size: int, table_width: int, offset: int, dim: int, eps: float):
        if not 0 <= offset and offset + dim <= table_width:
            raise ValueError(f"columns [{offset}, {offset + dim}) do not lie in a table of width {table_width}")
        self.hidden_size, self.vocab_size, self.table_width = int(hidden_size), int(vocab_size), int(table_width)
        self.offset, self.dim, self.eps = int(offset), int(dim), float(eps)

    def param_requests(self) -> List[ParamRequest]:
        d, n = self.hidden_size, self.dim
        return [ParamRequest("gate", (n, d), init="normal:0.08"), ParamRequest("proj", (d, n), init="normal:0.08"),
                ParamRequest("norm", (d,), init="ones_normal"),
                ParamRequest("table", (self.vocab_size, self.table_width), alias_of="embedding.side", alias_only=True)]

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        """The two small products; of the table only the tokens' rows are read."""
        n = 2 * self.dim * self.hidden_size
        return StepCost(n + self.hidden_size, 2.0 * tokens * n)

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.w_gate, self.w_proj, self.table = tensors["gate"], tensors["proj"], tensors["table"]
        self.norm_w = tensors["norm"].float().contiguous()
        self.ones = torch.ones((self.hidden_size,), dtype=torch.float32, device=rt.device)

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], ctx) -> Optional[torch.Tensor]:
        """Fold `pending` (the layer's last output) into the stream, then add this part's own.  Returns what is
        still to be added: nothing."""
        xc = self.rt.empty(tuple(x.shape))
        ops.stream_add(x, pending, None, xc)
        z = linear(xc, self.w_gate)
        g = ops.gelu_mul_rows(z, self.table, self.offset, ctx.token_ids, self.rt.empty(tuple(z.shape)), ctx.src_row,
                              ctx.prev_tokens)
        y = linear(g, self.w_proj, partial_ok=True)
        following = getattr(ctx, "next_input_norm", None)
        if getattr(following, "weight_f32", None) is not None and following.size == self.hidden_size:
            # the norm that the next layer begins with, in the same kernel
            h = ops.output_norm_add(x, y, self.norm_w, self.ones, self.eps, self.rt.empty(tuple(x.shape)),
                                    following.weight_f32, following.eps)
            ctx.shared[NORMED_STREAM] = (h, following)
        else:
            ops.output_norm_add(x, y, self.norm_w, self.ones, self.eps, None)
        return None


class PassVectors(Part):
    graph_safe = True

    def __init__(self, rows: int, hidden_size: int):
        self.rows, self.hidden_size = int(rows), int(hidden_size)

    def param_requests(self) -> List[ParamRequest]:
        return [ParamRequest("weight", (self.rows, self.hidden_size), init="normal:0.3")]

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        return StepCost(0, 0.0)

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.table = tensors["weight"].float().contiguous()          # the stream is fp32

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], row: int,
                extra: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """x += pending + table[row] (+ extra, fp32 [T, width]); nothing is left to be added."""
        if not 0 <= row < self.rows:
            raise ValueError(f"pass vector {row} of {self.rows}")
        ops.stream_add(x, pending, self.table[row], None, extra)
        return None


class PairEmbedding(Part):
    """x = E[token] + B[(previous token * mul_prev + token * mul_cur) mod buckets]; a sequence's first token takes
    B's last row (B has buckets + 1 rows).  The previous token of a request's next portion is kept in a per-request
    state row (`state_request`), read and replaced by the embedding's kernels on the device, so that portions cut
    anywhere, and tokens that never reached the host, see the right row."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, buckets: int, mul_prev: int, mul_cur: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        if self.buckets <= 0 or self.mul_prev < 0 or self.mul_cur < 0:
            raise ValueError("buckets must be positive, the multipliers not negative")
        if max(self.mul_prev, self.mul_cur) * self.vocab_size >= 2 ** 62:
            raise ValueError("the pair's hash must fit 64 bits")

    def param_requests(self) -> List[ParamRequest]:
        return [ParamRequest("weight", (self.vocab_size, self.hidden_size)),
                ParamRequest("pairs", (self.buckets + 1, self.hidden_size))]

    def state_request(self) -> StateRequest:
        return StateRequest((1,), torch.int32)           # the request's latest token

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        return StepCost(0, 0.0)                          # (gathered rows, as for the plain embedding)

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = tensors["weight"]
        self.pairs = tensors["pairs"].to(self.weight.dtype).contiguous()

    def forward(self, ctx, cache: LayerCache, keep: bool = False):
        """fp32 [T, width]; with `keep` also a second copy of it, for whoever adds it to the stream again."""
        T = ctx.token_ids.numel()
        x = self.rt.empty((T, self.hidden_size), torch.float32)
        copy = self.rt.empty((T, self.hidden_size), torch.float32) if keep else None
        ops.pair_embed(self.weight, self.pairs, ctx, cache.state, x, self.mul_prev, self.mul_cur, copy)
        return (x, copy) if keep else x


register_part("embedding", "pair_embedding", PairEmbedding)

register_part("token_input", "gated_side_embedding", GatedSideEmbedding)
register_part("stream_input", "pass_vectors", PassVectors)
