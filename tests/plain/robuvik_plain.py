"""A plain, slow implementation of the Robuvik decoder in float64: one function per mechanism, whole sequences
at a time, no cache.  It shares no code with the package; the tests compare the engine with it.

    x_0    = E[token_p] + B[row_p],  row_p = (token_(p-1) * mul_prev + token_p * mul_cur) mod buckets,  row_0 = buckets
    layer:   h = N(x) w;  x <- x + mixer(h) + ff(h)                  (one norm, both sublayers read it)
    loop:    layers start .. stop-1 run `times` times; before pass t > 0, x <- x + x_0; before every pass x <- x + P[t]
    logits = W_head (N(x) w_final)

A model is a dict: {"config": the configuration as config.json holds it, "tensors": {name: float64 tensor}}.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotary_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """(f [dims / 2], magnitude): pair i turns by position * f_i, and sine and cosine are multiplied by the magnitude."""
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, f: torch.Tensor, magnitude: float, layout: str) -> torch.Tensor:
    """x [T, H, D]: the first 2 len(f) dims of every head turned by the position; `layout` 'interleaved' pairs
    (2i, 2i + 1), 'half' pairs (i, i + len(f))."""
    n = f.numel()
    a = positions.to(F64)[:, None] * f[None, :]
    cos, sin = (torch.cos(a) * magnitude)[:, None, :], (torch.sin(a) * magnitude)[:, None, :]
    out = x.clone()
    if layout == "interleaved":
        u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
        out[..., 0:2 * n:2] = u * cos - v * sin
        out[..., 1:2 * n:2] = v * cos + u * sin
    else:
        u, v = x[..., :n], x[..., n:2 * n]
        out[..., :n] = u * cos - v * sin
        out[..., n:2 * n] = v * cos + u * sin
    return out


def embedding(tokens: List[int], embed: torch.Tensor, bigram: Optional[torch.Tensor], cfg: dict) -> torch.Tensor:
    b = (cfg.get("embedding") or {}).get("bigram")
    if not b:
        return embed[torch.tensor(tokens)]
    rows = []
    for p, t in enumerate(tokens):
        rows.append(b["buckets"] if p == 0 else (tokens[p - 1] * b["mul_prev"] + t * b["mul_cur"]) % b["buckets"])
    return embed[torch.tensor(tokens)] + bigram[torch.tensor(rows)]


def softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: Optional[int],
                      sink: bool) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; query head h reads key head h // (H / G); position i sees j with
    0 <= i - j (< window); with `sink` the denominator has one more term exp(0)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[2]), dtype=F64)
    i = torch.arange(T)
    dist = i[:, None] - i[None, :]
    seen = dist >= 0
    if window is not None:
        seen &= dist < window
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, -math.inf)
        m = s.max(-1, keepdim=True).values
        if sink:
            m = m.clamp_min(0.0)
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True) + (torch.exp(-m) if sink else 0.0)
        out[:, h] = (e / den) @ v[:, g]
    return out


def attention_mixer(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[p + "q"].T + t[p + "q.b"]).view(T, H, D)
    k = (h @ t[p + "k"].T + t[p + "k.b"]).view(T, G, D)
    v = (h @ t[p + "v"].T + t[p + "v.b"]).view(T, G, Dv)
    rot = m.get("rot")
    pos = torch.arange(T)
    if rot:
        f, mag = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate(q, pos, f, mag, "half"), rotate(k, pos, f, mag, "half")
    window = (m.get("mask") or {}).get("size")
    o = softmax_attention(q, k, v, m["scale"], window, sink=True)
    return o.reshape(T, H * Dv) @ t[p + "o"].T


def latent_attention_mixer(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, Dr, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ t[p + "dq"].T, t[p + "dq.norm"], eps)
    q = (cq @ t[p + "uq"].T).view(T, H, D + Dr)
    z = h @ t[p + "dkv"].T
    c = rms_norm(z[:, :R], t[p + "dkv.norm"], eps)
    k_rot = z[:, R:].view(T, 1, Dr)
    rot = m["rot"]
    f, mag = rotary_frequencies(Dr, rot["base"], rot.get("scaling"))
    pos = torch.arange(T)
    q_rot = rotate(q[..., D:].contiguous(), pos, f, mag, "interleaved")
    k_rot = rotate(k_rot, pos, f, mag, "interleaved")
    k_plain = (c @ t[p + "uk"].T).view(T, H, D)
    v = (c @ t[p + "uv"].T).view(T, H, Dv)
    qq = torch.cat([q[..., :D], q_rot], -1)
    kk = torch.cat([k_plain, k_rot.expand(T, H, Dr)], -1)
    o = softmax_attention(qq, kk, v, m["scale"], None, sink=False).reshape(T, H * Dv)
    o = o * torch.sigmoid(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


def dense_ff(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return torch.relu(h @ t[p + "up"].T) ** 2 @ t[p + "down"].T


def gated_expert(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    g = h @ t[p + "gate"].T
    return (g * torch.sigmoid(g) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def router(h: torch.Tensor, w: torch.Tensor, top: int):
    """(ids [T, top], scores [T, top]): the `top` largest sigmoid scores (ties to the lower index), as they are."""
    s = torch.sigmoid(h @ w.T)
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.gather(s, 1, order)


def moe_ff(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    ids, w = router(h, t[p + "router"], mlp["router"]["top"])
    out = torch.zeros((h.shape[0], t[p + "e0.down"].shape[0]), dtype=F64)
    for tok in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[tok, j])
            out[tok] += gated_expert((w[tok, j] * h[tok])[None], t, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_expert(h, t, p + "shared.")
    return out


def layer_passes(cfg: dict):
    """[(layer index, pass number or None)] in the order the layers run."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    out = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        out += [(i, t) for i in range(loop["start"], loop["stop"])]
    return out + [(i, None) for i in range(loop["stop"], n)]


def forward(model: dict, tokens: List[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence; `streams` collects the residual stream after every layer run."""
    cfg, t = model["config"], model["tensors"]
    eps = cfg["norm"]["eps"]
    x0 = embedding(tokens, t["embed"], t.get("bigram"), cfg)
    x = x0.clone()
    loop = cfg.get("loop")
    for i, pas in layer_passes(cfg):
        if pas is not None and i == loop["start"]:
            if pas > 0:
                x = x + x0
            x = x + t["loop.step"][pas]
        layer = cfg["layers"][i]
        h = rms_norm(x, t[f"l{i}.norm1"], eps)
        if layer["type"] == "attention":
            a = attention_mixer(h, t, f"l{i}.mix.", layer["mixer"])
        elif layer["type"] == "latent_attention":
            a = latent_attention_mixer(h, t, f"l{i}.mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            a = a + (dense_ff(h, t, f"l{i}.mlp.") if mlp["kind"] == "dense" else moe_ff(h, t, f"l{i}.mlp.", mlp))
        x = x + a
        if streams is not None:
            streams.append(x.clone())
    return rms_norm(x, t["final.norm"], eps) @ t["head"].T
