"""Plain, slow, cache-free implementation of the Kotipel decoder.

One function per mechanism, written from the design's equations, whole sequences on the CPU, in
the dtype it is given (float64 as the oracle).  It shares no code with the `serve_amd` package:
the tests compare the engine with it.

Notation.  h [T, d] is a sublayer's input, W["<name>"] a checkpoint tensor stored [out, in],
N_w(y) = y / sqrt(mean(y^2) + eps) * w.  A layer is

    x <- x + mixer(N_1(x));   x <- x + ff(N_2(x))  (if it has a feed-forward);
    x <- x + N_s(P (gelu_tanh(G x) * e))           (if the model has per-layer token inputs; e is the layer's
                                                    slice of a second embedding row of the token)

Layers `start .. stop-1` run `times` times in a row with the same weights; before pass t the row t of a table
is added to the stream.  The mixer is either two mixers side by side whose normed outputs are averaged (a
softmax attention with an output gate and a gated linear attention), or a selective state-space mixer.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

Tensor = torch.Tensor


# --------------------------------------------------------------------------------------
# elementwise pieces
# --------------------------------------------------------------------------------------
def rms(y: Tensor, eps: float) -> Tensor:
    return y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps)


def rms_norm(y: Tensor, w: Tensor, eps: float) -> Tensor:
    return rms(y, eps) * w


def gelu_tanh(z: Tensor) -> Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: Tensor) -> Tensor:
    return z * torch.sigmoid(z)


def softplus(z: Tensor) -> Tensor:
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


# --------------------------------------------------------------------------------------
# rotation
# --------------------------------------------------------------------------------------
def rotary_frequencies(dims: int, base: float, scaling: Optional[dict]) -> List[float]:
    """f_i = base^(-2i/dims), i < dims/2; with `scaling` {factor, low, high, original} a frequency whose
    wavelength l = 2 pi / f is shorter than original/high stays, one longer than original/low is divided by
    factor, and between the two it is blended linearly in original/l."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling is not None:
            factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            l = 2.0 * math.pi / f
            if l < orig / high:
                pass
            elif l > orig / low:
                f = f / factor
            else:
                s = (orig / l - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x: Tensor, positions: Tensor, freqs: Sequence[float]) -> Tensor:
    """x [T, H, D]: dimension i is paired with i + dims/2 over the first dims = 2 len(freqs) dimensions of every
    head; the pair (u, v) at position p becomes (u cos a - v sin a, v cos a + u sin a), a = p f_i."""
    half = len(freqs)
    if half == 0:
        return x
    f = torch.tensor(list(freqs), dtype=x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :]            # [T, half]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half: 2 * half]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half: 2 * half] = v * c + u * s
    return out


# --------------------------------------------------------------------------------------
# the left mixer: softmax attention, q/k normed over the whole projection, output gate per head
# --------------------------------------------------------------------------------------
def gated_attention(h: Tensor, W: Dict[str, Tensor], m: dict, eps: float, positions: Tensor) -> Tensor:
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ W["q"].t(), W["q.norm"], eps).view(T, H, D)
    k = rms_norm(h @ W["k"].t(), W["k.norm"], eps).view(T, G, D)
    v = (h @ W["v"].t()).view(T, G, Dv)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q, k = rotate(q, positions, f), rotate(k, positions, f)
    gate = torch.sigmoid(h @ W["g"].t())                        # [T, H]
    seen = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for i in range(H):
        g = i // (H // G)
        s = (q[:, i] @ k[:, g].t()) * float(m["scale"])
        s = s.masked_fill(~seen, float("-inf"))
        out[:, i] = (torch.softmax(s, dim=-1) @ v[:, g]) * gate[:, i: i + 1]
    return out.reshape(T, H * Dv) @ W["o"].t()


# --------------------------------------------------------------------------------------
# recurrences:  S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t        (one head)
# --------------------------------------------------------------------------------------
def decayed_recurrence(q: Tensor, k: Tensor, v: Tensor, a: Tensor) -> Tensor:
    """q, k [T, dk]; v [T, dv]; a [T, dk] (a decay per key channel) or [T] (one per head)."""
    T, dk = q.shape
    S = torch.zeros(dk, v.shape[1], dtype=q.dtype)
    out = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for t in range(T):
        at = a[t][:, None] if a.dim() == 2 else a[t]
        S = at * S + torch.outer(k[t], v[t])
        out[t] = S.t() @ q[t]
    return out


def gated_linear_attention(h: Tensor, W: Dict[str, Tensor], m: dict, eps: float) -> Tensor:
    """The right mixer: per key channel alpha = sigmoid(z)^(1/tau), z = W_a2 (W_a1 h) + b."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W["q"].t()).view(T, H, D) * D ** -0.5
    k = (h @ W["k"].t()).view(T, H, D)
    v = (h @ W["v"].t()).view(T, H, Dv)
    z = (h @ W["a1"].t()) @ W["a2"].t() + W["a2.b"]
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / float(m["tau"])).view(T, H, D)
    o = torch.stack([decayed_recurrence(q[:, i], k[:, i], v[:, i], alpha[:, i]) for i in range(H)], dim=1)
    o = rms_norm(o, W["norm"], eps).reshape(T, H * Dv)
    return (o * silu(h @ W["g"].t())) @ W["o"].t()


def parallel_mixer(h: Tensor, W: Dict[str, Tensor], m: dict, eps: float, positions: Tensor) -> Tensor:
    left = gated_attention(h, _sub(W, "left."), m["left"], eps, positions)
    right = gated_linear_attention(h, _sub(W, "right."), m["right"], eps)
    return 0.5 * (rms_norm(left, W["left.out"], eps) + rms_norm(right, W["right.out"], eps))


# --------------------------------------------------------------------------------------
# the selective state-space mixer
# --------------------------------------------------------------------------------------
def causal_conv(x: Tensor, w: Tensor, b: Tensor) -> Tensor:
    """x [T, C], w [C, taps] (the last column is the current token's), b [C]; zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    out = b[None, :].repeat(T, 1).to(x.dtype)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                out[t] = out[t] + w[:, j] * x[s]
    return out


def grouped_rms_norm(y: Tensor, w: Tensor, groups: int, eps: float) -> Tensor:
    T, n = y.shape
    return (rms(y.view(T, groups, n // groups), eps)).reshape(T, n) * w


def state_space_mixer(h: Tensor, W: Dict[str, Tensor], m: dict, eps: float) -> Tensor:
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    zxbcdt = h @ W["in"].t()
    z, xbc, dt = zxbcdt[:, :inner], zxbcdt[:, inner: 2 * inner + 2 * G * N], zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W["conv"], W["conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner: inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W["dt_bias"])                            # [T, H]
    decay = torch.exp(-torch.exp(W["A_log"]) * dt)              # [T, H]
    ys = []
    for i in range(H):
        g = i // (H // G)
        y = decayed_recurrence(C[:, g], B[:, g], dt[:, i: i + 1] * x[:, i], decay[:, i])
        ys.append(y + W["D"][i] * x[:, i])
    y = torch.stack(ys, dim=1).reshape(T, inner) * silu(z)
    return grouped_rms_norm(y, W["norm"], int(m["norm_groups"]), eps) @ W["o"].t()


# --------------------------------------------------------------------------------------
# feed-forward, per-layer token input
# --------------------------------------------------------------------------------------
def clamped_ff(h: Tensor, W: Dict[str, Tensor], limit: float) -> Tensor:
    g = (h @ W["gate"].t()).clamp(max=limit)
    u = (h @ W["up"].t()).clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W["down"].t()


def token_side_input(x: Tensor, e: Tensor, W: Dict[str, Tensor], eps: float) -> Tensor:
    """e [T, dim] is the layer's slice of the tokens' rows of the second table."""
    y = (gelu_tanh(x @ W["gate"].t()) * e) @ W["proj"].t()
    return rms_norm(y, W["norm"], eps)


# --------------------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------------------
def _sub(W: Dict[str, Tensor], prefix: str) -> Dict[str, Tensor]:
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def run_order(cfg: dict) -> List[tuple]:
    """(layer, pass) in the order they run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return ([(i, None) for i in range(a)] + [(i, t) for t in range(times) for i in range(a, b)]
            + [(i, None) for i in range(b, n)])


def forward(tokens: Sequence[int], weights: Dict[str, Tensor], cfg: dict, dtype=torch.float64,
            return_layers: bool = False):
    """Logits [T, vocab] of a whole sequence (and, on request, the stream after every layer run)."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    tok = torch.as_tensor(list(tokens), dtype=torch.long)
    T = tok.numel()
    positions = torch.arange(T)
    x = W["embed"][tok]
    side = cfg.get("token_side")
    loop = cfg.get("loop")
    streams = []
    for i, t in run_order(cfg):
        if t is not None and i == int(loop["start"]):
            x = x + W["loop.step"][t]
        layer, Wl = cfg["layers"][i], _sub(W, f"l{i}.")
        hn = rms_norm(x, Wl["norm1"], eps)
        if layer["type"] == "parallel":
            x = x + parallel_mixer(hn, _sub(Wl, "mix."), layer["mixer"], eps, positions)
        elif layer["type"] == "mamba2":
            x = x + state_space_mixer(hn, _sub(Wl, "mix."), layer["mixer"], eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            x = x + clamped_ff(rms_norm(x, Wl["norm2"], eps), _sub(Wl, "mlp."), float(layer["mlp"]["limit"]))
        if side:
            dim = int(side["dim"])
            e = W["side.embed"][tok][:, i * dim: (i + 1) * dim]
            x = x + token_side_input(x, e, _sub(Wl, "side."), eps)
        streams.append(x)
    logits = rms_norm(x, W["final.norm"], eps) @ W["embed"].t()
    if return_layers:
        return logits, torch.stack(streams)
    return logits
