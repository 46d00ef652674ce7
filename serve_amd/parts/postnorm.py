"""Layers whose norm sits on the sublayer's output:

    x <- x + s1 * N1(mixer(x));   x <- x + s2 * N2(ffn(x))     N(y) = y / sqrt(mean(y^2) + eps) * (offset + w)

The sublayers read the residual stream itself (its copy in the activation dtype), the norm
weights may be stored around zero (`offset` 1), and every sublayer's normed output is scaled
element by element (`scale`, a "layer scale") before it joins the stream.  A layer may have no
feed-forward.

And layers with a norm on both sides of every sublayer (`SandwichResidual`):

    x <- x + c * Nb1(mixer(Na1(x)));   x <- x + c * Nb2(ffn(Na2(x)))

with one constant c for the model in place of the layer scale.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..registry import register_part
from .base import NORMED_STREAM, LayerCache, ParamRequest, Part, Runtime


class ScaledOutputNorm(Part):
    """x += scale * (y / sqrt(mean(y^2) + eps) * (offset + weight)) on the fp32 stream, in one kernel
    that also hands back the new stream in the activation dtype for the sublayer that reads it next."""

    graph_safe = True

    def __init__(self, size: int, eps: float, offset: float = 0.0, constant_scale: Optional[float] = None):
        """`constant_scale`: one number in place of the stored layer scale (no `scale` tensor then)."""
        self.size, self.eps, self.offset = int(size), float(eps), float(offset)
        self.constant_scale = None if constant_scale is None else float(constant_scale)

    def param_requests(self) -> List[ParamRequest]:
        out = [ParamRequest("weight", (self.size,), init="normal:0.2" if self.offset else "ones_normal")]
        if self.constant_scale is None:
            out.append(ParamRequest("scale", (self.size,), init="ones_normal:0.2"))
        return out

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = (tensors["weight"].float() + self.offset).contiguous()       # fp32, whatever the storage
        if self.constant_scale is None:
            self.scale = tensors["scale"].float().contiguous()
        else:
            self.scale = torch.full((self.size,), self.constant_scale, dtype=torch.float32, device=rt.device)

    def add(self, x: torch.Tensor, y: torch.Tensor) -> None:
        """Only x += scale * N(y): no copy of the stream is made."""
        ops.output_norm_add(x, y, self.weight, self.scale, self.eps, None)

    def add_then_norm(self, x: torch.Tensor, y: torch.Tensor, following) -> torch.Tensor:
        """x += scale * N(y), and in the same kernel what the norm `following` (an `RMSNorm`) makes of the new
        x: the activations that the next sublayer reads."""
        h = self.rt.empty(tuple(x.shape))
        return ops.output_norm_add(x, y, self.weight, self.scale, self.eps, h, following.weight_f32, following.eps)

    def forward(self, x: torch.Tensor, y: Optional[torch.Tensor], rows=None) -> torch.Tensor:
        """Add the normed, scaled `y` into x (in place) and return what the next sublayer reads: x
        itself in the float32 engine, else its copy in the activation dtype."""
        if rows is not None:
            raise ValueError("a norm on a sublayer's output takes whole steps, not rows")
        h = None if self.rt.exact else self.rt.empty(tuple(x.shape))
        ops.output_norm_add(x, y, self.weight, self.scale, self.eps, h)
        return x if h is None else h


def stream_copy(x: torch.Tensor, rt: Runtime) -> torch.Tensor:
    """The fp32 stream as the sublayers read it."""
    if rt.exact:
        return x
    return ops.output_norm_add(x, None, None, None, 0.0, rt.empty(tuple(x.shape)))


class PostNormResidual:
    """x += s1 N1(mixer(x)); x += s2 N2(ffn(x)), the second half only if the layer has a feed-forward.

    It leaves no pending output: the stream is complete when the layer returns.  The copy of the
    stream in the activation dtype that its last norm made travels to the next layer of this kind
    on the step's context, so that only the first such layer of a model makes one itself."""

    PART_ROLES = {"mixer": "mixer", "ffn": "feed_forward", "mixer_norm": "norm", "ffn_norm": "norm"}
    OPTIONAL_PARTS = ("ffn", "ffn_norm")

    def __init__(self, mixer, mixer_norm, ffn=None, ffn_norm=None):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm

    def cache_owner(self) -> Part:
        return self.mixer

    def parts(self) -> Dict[str, Part]:
        out = {"mixer": self.mixer, "mixer_norm": self.mixer_norm}
        if self.ffn is not None:
            out.update(ffn=self.ffn, ffn_norm=self.ffn_norm)
        return out

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], ctx, cache: LayerCache,
                writes_cache: bool = True) -> None:
        rt = self.mixer_norm.rt
        kept = getattr(ctx, "stream_copy", None)
        ctx.stream_copy = None
        if pending is not None:
            # a layer of another arrangement left its last output unadded
            x.add_(pending.sum(0) if pending.dim() == 3 else pending)
            kept = None
        h = kept if kept is not None else stream_copy(x, rt)
        h = self.mixer_norm.forward(x, self.mixer.forward(h, ctx, cache, writes_cache))
        if self.ffn is not None:
            h = self.ffn_norm.forward(x, self.ffn.forward(h, ctx))
        ctx.stream_copy = h
        return None




class SandwichResidual:
    """x += c Nb1(mixer(Na1(x))); x += c Nb2(ffn(Na2(x))), the second half only if the layer has a feed-forward.

    `mixer_norm` and `ffn_norm` are norms of the stream (kind `rmsnorm`), `mixer_out_norm` and `ffn_out_norm`
    norms of a sublayer's output that add into the stream (kind `scaled_output_rmsnorm`, which carries c).
    It leaves no pending output: the stream is complete when the layer returns.  Each norm behind a sublayer and the
    norm in front of the next one are one kernel, across layers too: where the model says which norm the next layer
    begins with (`ctx.next_input_norm`), the activations it makes travel on the step's context."""

    PART_ROLES = {"mixer": "mixer", "ffn": "feed_forward", "mixer_norm": "norm", "mixer_out_norm": "norm",
                  "ffn_norm": "norm", "ffn_out_norm": "norm"}
    OPTIONAL_PARTS = ("ffn", "ffn_norm", "ffn_out_norm")

    def __init__(self, mixer, mixer_norm, mixer_out_norm, ffn=None, ffn_norm=None, ffn_out_norm=None):
        if not ((ffn is None) == (ffn_norm is None) == (ffn_out_norm is None)):
            raise ValueError("a feed-forward and its two norms come together")
        self.mixer, self.mixer_norm, self.mixer_out_norm = mixer, mixer_norm, mixer_out_norm
        self.ffn, self.ffn_norm, self.ffn_out_norm = ffn, ffn_norm, ffn_out_norm

    def cache_owner(self) -> Part:
        return self.mixer

    def parts(self) -> Dict[str, Part]:
        out = {"mixer": self.mixer, "mixer_norm": self.mixer_norm, "mixer_out_norm": self.mixer_out_norm}
        if self.ffn is not None:
            out.update(ffn=self.ffn, ffn_norm=self.ffn_norm, ffn_out_norm=self.ffn_out_norm)
        return out

    def input_norm(self) -> Part:
        """The norm this layer begins with: the layer before may apply it at the end of its own last kernel."""
        return self.mixer_norm

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], ctx, cache: LayerCache,
                writes_cache: bool = True) -> None:
        ctx.stream_copy = None                      # (this layer changes the stream and keeps no such copy)
        ready = ctx.shared.pop(NORMED_STREAM, None)
        if ready is not None and ready[1] is self.mixer_norm and pending is None:
            h = ready[0]                            # the layer before has made it, with this layer's norm
        else:
            h = self.mixer_norm.forward(x, pending)     # (adds what a layer of another arrangement left unadded)
        y, last = self.mixer.forward(h, ctx, cache, writes_cache), self.mixer_out_norm
        if self.ffn is not None:
            h = last.add_then_norm(x, y, self.ffn_norm)
            y, last = self.ffn.forward(h, ctx), self.ffn_out_norm
        following = getattr(ctx, "next_input_norm", None)
        if getattr(following, "weight_f32", None) is not None and following.size == last.size:
            ctx.shared[NORMED_STREAM] = (last.add_then_norm(x, y, following), following)
        else:
            last.add(x, y)
        return None


register_part("norm", "scaled_output_rmsnorm", ScaledOutputNorm)
register_part("arrangement", "postnorm_residual", PostNormResidual)
register_part("arrangement", "sandwich_residual", SandwichResidual)
