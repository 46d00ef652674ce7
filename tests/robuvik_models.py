"""Small Robuvik models for the tests, their folders with random weights, and comparisons of the engine's logits
with the plain implementation's (tests/plain/robuvik_plain.py).

The models differ in every size and option:
  RA  width 64; (attention, dense), (latent attention, experts top 2 of 4 + shared), (attention, experts top 1 of 6, no
      shared expert); layers 1..2 run twice; attention 4 heads on 2 of keys 32 / values 16, 16 rotated dims with a
      stretched rotation whose band lies inside short contexts, a window of 10; latent attention 3 heads of 16 + 8
      rotated, values 24, latents 40 / 24; second attention 2 heads on 1, keys 24 / values 40 (a cache head of 48), all
      dims rotated without stretching, a window of 5 (shorter than a page)
  RB  width 96, no loop, no pair table; (latent attention, no feed-forward), (attention without window and without
      rotation, dense), (latent attention with a plain rotation, experts top 3 of 3)
  RC  width 50 (no multiple of 8), vocabulary 101; both layers run three times; 3 heads on 3, keys 10 / values 7, 4
      rotated dims, a window of 33; latent attention 2 heads of 6 + 4, values 5, latents 9 / 7; experts of width 9
  RE  RB with its first two layers run twice (a loop without a pair table)
  RF  two attention layers whose heads are rotated whole, keys and values 32 / 32 and 16 / 16, with and without window and
      stretching: the shapes whose single tokens take the fused product in bfloat16
  RD  sizes above what the matrix-core attention takes: keys 136 / values 24; a latent row of 200 + 16; a single layer
      that runs twice between two that run once
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch

from serve_amd.config.kotipel import LoopConfig
from serve_amd.config.robuvik import (BigramConfig, DenseConfig, ExpertsConfig, LatentAttentionConfig, RobuvikConfig,
                                      RobuvikLayerConfig, RotConfig, WindowAttentionConfig, YarnScaling)
from serve_amd.weights.loader import write_random_model
from tests.plain import robuvik_plain

L = RobuvikLayerConfig
ATT, LAT = WindowAttentionConfig, LatentAttentionConfig

RA = RobuvikConfig(vocab=150, width=64, eps=1e-5, bigram=BigramConfig(97, 5, 3), loop=LoopConfig(1, 3, 2), layers=(
    L(ATT(4, 2, 32, 16, 0.2, RotConfig(100.0, 16, YarnScaling(4.0, 32.0, 6.0, 1.5)), 10), DenseConfig(96)),
    L(LAT(3, 16, 8, 24, 40, 24, 0.2, RotConfig(50.0, 8, YarnScaling(3.0, 16.0, 4.0, 1.0))), ExpertsConfig(4, 2, 32, 48)),
    L(ATT(2, 1, 24, 40, 0.22, RotConfig(10000.0, 24, None), 5), ExpertsConfig(6, 1, 40, None)),
))

RB = RobuvikConfig(vocab=211, width=96, eps=1e-6, bigram=None, loop=None, layers=(
    L(LAT(6, 8, 16, 8, 24, 48, 0.25, RotConfig(300.0, 16, YarnScaling(2.0, 24.0, 8.0, 2.0))), None),
    L(ATT(6, 3, 16, 16, 0.25, None, None), DenseConfig(120)),
    L(LAT(2, 32, 4, 32, 64, 16, 0.15, RotConfig(1000.0, 4, None)), ExpertsConfig(3, 3, 24, 40)),
))

RC = RobuvikConfig(vocab=101, width=50, eps=1e-5, bigram=BigramConfig(13, 1, 101), loop=LoopConfig(0, 2, 3), layers=(
    L(ATT(3, 3, 10, 7, 0.4, RotConfig(50.0, 4, YarnScaling(8.0, 8.0, 2.0, 0.5)), 33), ExpertsConfig(5, 2, 9, 11)),
    L(LAT(2, 6, 4, 5, 9, 7, 0.4, RotConfig(20.0, 4, None)), DenseConfig(27)),
))

RD = RobuvikConfig(vocab=120, width=64, eps=1e-5, bigram=BigramConfig(1019, 29, 11), loop=LoopConfig(1, 2, 2), layers=(
    L(ATT(2, 1, 136, 24, 0.1, RotConfig(5000.0, 64, YarnScaling(2.0, 64.0, 16.0, 1.0)), 40), None),
    L(LAT(2, 24, 16, 16, 200, 32, 0.12, RotConfig(200.0, 16, YarnScaling(2.0, 64.0, 16.0, 1.0))), DenseConfig(64)),
    L(ATT(2, 2, 136, 24, 0.1, None, 7), ExpertsConfig(2, 1, 16, None)),
))

# RB with its first two layers run twice: passes that add the output of an embedding without a pair table
RE = RobuvikConfig(vocab=RB.vocab, width=RB.width, eps=RB.eps, bigram=None, loop=LoopConfig(0, 2, 2), layers=RB.layers)

# whole heads rotated, keys and values of one size that is a multiple of 16: in bfloat16, steps of few rows take the
# product whose epilogue adds the biases, rotates and writes the cache
RF = RobuvikConfig(vocab=130, width=64, eps=1e-5, bigram=BigramConfig(61, 3, 5), loop=LoopConfig(0, 1, 2), layers=(
    L(ATT(4, 2, 32, 32, 0.18, RotConfig(300.0, 32, YarnScaling(3.0, 24.0, 6.0, 1.0)), 9), DenseConfig(72)),
    L(ATT(3, 1, 16, 16, 0.25, RotConfig(40.0, 16, None), None), ExpertsConfig(4, 2, 24, None)),
))

MODELS = {"RA": (RA, 3), "RB": (RB, 4), "RC": (RC, 5), "RD": (RD, 6), "RE": (RE, 7), "RF": (RF, 8)}

# tables and the output matrix at a scale at which the stream and the logits are of order one
BASE = {r"^embed$": 40.0, r"^bigram$": 25.0, r"^head$": 6.0, r"^loop\.step$": 2.0}

# queries and keys drawn wider: scores of order one and more, so that the softmax picks keys instead of averaging them
# and a key lost or let in at a window's edge moves the logits by far more than the bfloat16 tolerance
SHARP = {r"mix\.(q|k|uq|uk)$": 4.0}

# per row of logits: root mean square of the difference over that of the row.  float32: a few ulp of the largest
# intermediate; bfloat16: 8 bits of mantissa at every product's input
TOLERANCE = {"float32": 2e-4, "bfloat16": 0.08}


def make_folder(tmp_path, name: str, config: Optional[RobuvikConfig] = None, seed=None, scales=None) -> str:
    cfg, s = MODELS.get(name, (config, seed))
    folder = os.path.join(str(tmp_path), f"robuvik_{name}")
    if not os.path.isdir(folder):
        write_random_model(folder, cfg if config is None else config, s if seed is None else seed,
                           scales=dict(BASE, **(scales or {})))
    return folder


def plain_weights(folder: str) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file
    return load_file(os.path.join(folder, "model.safetensors"))


def plain_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def plain_model(folder: str, config: Optional[dict] = None, weights: Optional[Dict[str, torch.Tensor]] = None) -> dict:
    w = weights or plain_weights(folder)
    return {"config": config or plain_config(folder), "tensors": {k: v.double() for k, v in w.items()}}


def plain_logits(folder: str, tokens: List[int], config: Optional[dict] = None,
                 weights: Optional[Dict[str, torch.Tensor]] = None) -> torch.Tensor:
    return robuvik_plain.forward(plain_model(folder, config, weights), tokens)


def row_distance(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row: the root mean square of the difference (its mean taken off) over that of the wanted row."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-12)


def assert_rows_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what: str = "") -> None:
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    dist = row_distance(got, want)
    bad = (dist > TOLERANCE[dtype]) | ~torch.isfinite(dist)
    if bad.any():
        i = int(bad.nonzero()[0])
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.numel()} rows differ; first row {i}: distance "
                             f"{dist[i].item():.3g}, allowed {TOLERANCE[dtype]:.3g}; worst {dist.max().item():.3g}")


def shaky_rows(folder: str, tokens: List[int], want: torch.Tensor) -> torch.Tensor:
    """Rows of the plain model's logits that rest on a close call (a router's choice between two experts whose scores
    nearly tie moves the token's own row and, through its keys and values, rows behind it).  Found by running the plain
    model twice more with every floating tensor disturbed by a relative 2^-9 (what storing a value in bfloat16 does):
    rows that move by a quarter of the tolerance."""
    out = torch.zeros(len(tokens), dtype=torch.bool)
    for k in range(2):
        g = torch.Generator().manual_seed(len(tokens) + 1000 * k)
        W = {n: (v.double() * (1 + 2.0 ** -9 * (2 * torch.rand(v.shape, generator=g, dtype=torch.float64) - 1))
                 if v.is_floating_point() else v) for n, v in plain_weights(folder).items()}
        moved = row_distance(robuvik_plain.forward({"config": plain_config(folder), "tensors": W}, tokens), want)
        out |= moved > 0.25 * TOLERANCE["bfloat16"]
    return out


def assert_matches_plain(got: torch.Tensor, folder: str, tokens: List[int], dtype: str, what: str = "", rows=None) -> None:
    """`got`: the engine's logits for all of `tokens`, or for the places `rows` among them.  float32: every row.
    bfloat16: the rows that are well conditioned in the plain model (`shaky_rows`; they must be the many)."""
    want = plain_logits(folder, tokens)
    keep = None
    if dtype == "bfloat16":
        keep = ~shaky_rows(folder, tokens, want)
    if rows is not None:
        want = want[rows]
        keep = None if keep is None else keep[rows]
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    got = got.detach().cpu()
    if keep is not None:
        assert len(keep) < 20 or keep.float().mean().item() >= 0.6, f"{what}: too many rows rest on close calls"
        assert torch.isfinite(got).all()
        got, want = got[keep], want[keep]
    assert_rows_close(got, want, dtype, what)


def engine_for(folder: str, dtype: str, num_pages=64, page_size=8, max_requests=4, **kw):
    from serve_amd.config.engine import EngineConfig
    from serve_amd.engine.engine import Engine
    cfg = EngineConfig(dtype=dtype, page_size=page_size, num_pages=num_pages, max_context=num_pages * page_size,
                       max_requests=max_requests, max_tokens_per_step=4096, prefill_chunk=4096, **kw)
    return Engine.from_folder(folder, cfg)


def run_portions(engine, rid, tokens, portions):
    """Feed `tokens` in the given portion sizes, wanting every position; returns [len, V]."""
    from serve_amd.engine.batch import Segment
    assert sum(portions) == len(tokens)
    assert engine.runner.admit(rid)
    rows, at = [], 0
    for n in portions:
        rows.append(engine.step([Segment(rid, tokens[at: at + n], list(range(n)))]))
        at += n
    engine.runner.release(rid)
    return torch.cat(rows, dim=0)
