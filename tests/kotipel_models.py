"""Small Kotipel models for the tests, their folders with random weights, and comparisons of the engine's logits
with the plain implementation's (tests/plain/kotipel_plain.py).

The models differ in every size and option:
  KA  width 64; (parallel, dense), (state space, no feed-forward), (parallel, dense); layers 1..2 run twice; token
      inputs of 8; attention 4 heads on 2 of keys 32 / values 16, 16 rotated dims with rescaled frequencies whose
      band lies inside short contexts; linear attention 2 heads of 16 x 32; state space 4 heads of 16, state 16, two
      groups, 4 taps, two norm groups
  KB  width 96, no loop, no token inputs; (state space, dense), (parallel, no feed-forward); 6 heads on one
      key/value head, keys 24 / values 40 (a cache head of 48), all 24 dims rotated, no rescaling; linear attention 3
      heads of 48 x 20; state space 3 heads of 32, state 8, 2 taps, three norm groups
  KC  width 50 (no multiple of 8), vocabulary 101; both layers run three times; token inputs of 5; 3 heads on 3,
      keys 10 / values 7, 4 rotated dims; one linear-attention head of 10 x 70; state space 2 heads of 9, state 5,
      two groups, a convolution of one tap (no convolution state)
  KD  heads above what the matrix-core attention takes: keys 136 / values 24; linear attention keys of 130; a state
      of 160; a single layer that runs twice between two that run once
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch

from serve_amd.config.kotipel import (ClampedDenseConfig, GatedAttentionConfig, KotipelConfig, KotipelLayerConfig,
                                      LinearAttentionConfig, LoopConfig, ParallelMixerConfig, RotScaling,
                                      StateSpaceMixerConfig)
from serve_amd.weights.loader import write_random_model
from tests.plain import kotipel_plain

L = KotipelLayerConfig


def par(heads, kv, dim, vdim, scale, rot, base, scaling, rheads, rdim, rvdim, tau, rank):
    return ParallelMixerConfig(GatedAttentionConfig(heads, kv, dim, vdim, scale, rot, base, scaling),
                               LinearAttentionConfig(rheads, rdim, rvdim, tau, rank))


KA = KotipelConfig(vocab=150, width=64, eps=1e-5, loop=LoopConfig(1, 3, 2), side_dim=8, layers=(
    L(par(4, 2, 32, 16, 0.2, 16, 100.0, RotScaling(4.0, 0.5, 3.0, 32.0), 2, 16, 32, 8.0, 8), ClampedDenseConfig(96, 0.7)),
    L(StateSpaceMixerConfig(4, 16, 16, 2, 4, 2), None),
    L(par(4, 2, 32, 16, 0.2, 16, 100.0, RotScaling(4.0, 0.5, 3.0, 32.0), 2, 16, 32, 8.0, 8), ClampedDenseConfig(80, 2.5)),
))

KB = KotipelConfig(vocab=211, width=96, eps=1e-6, loop=None, side_dim=None, layers=(
    L(StateSpaceMixerConfig(3, 32, 8, 1, 2, 3), ClampedDenseConfig(120, 1.5)),
    L(par(6, 1, 24, 40, 0.25, 24, 10000.0, None, 3, 48, 20, 2.0, 12), None),
))

KC = KotipelConfig(vocab=101, width=50, eps=1e-5, loop=LoopConfig(0, 2, 3), side_dim=5, layers=(
    L(par(3, 3, 10, 7, 0.4, 4, 50.0, None, 1, 10, 70, 1.0, 3), ClampedDenseConfig(30, 1.0)),
    L(StateSpaceMixerConfig(2, 9, 5, 2, 1, 1), ClampedDenseConfig(27, 0.9)),
))

KD = KotipelConfig(vocab=120, width=64, eps=1e-5, loop=LoopConfig(1, 2, 2), side_dim=4, layers=(
    L(StateSpaceMixerConfig(2, 64, 160, 1, 3, 2), None),
    L(par(2, 1, 136, 24, 0.1, 64, 5000.0, RotScaling(8.0, 1.0, 4.0, 64.0), 2, 130, 64, 16.0, 4), ClampedDenseConfig(64, 1.2)),
    L(StateSpaceMixerConfig(2, 64, 160, 1, 3, 2), None),
))

MODELS = {"KA": (KA, 3), "KB": (KB, 4), "KC": (KC, 5), "KD": (KD, 6)}

# the embedding at a scale at which the logits (the table is the output matrix too) are of order one
BASE = {r"^embed$": 12.0}

# per row of logits: root mean square of the difference over that of the row.  float32: a few ulp of the largest
# intermediate through two recurrences; bfloat16: 8 bits of mantissa at every product's input
TOLERANCE = {"float32": 2e-4, "bfloat16": 0.08}


def make_folder(tmp_path, name: str, config: Optional[KotipelConfig] = None, seed=None, scales=None) -> str:
    cfg, s = MODELS.get(name, (config, seed))
    folder = os.path.join(str(tmp_path), f"kotipel_{name}")
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


def plain_logits(folder: str, tokens: List[int], config: Optional[dict] = None,
                 weights: Optional[Dict[str, torch.Tensor]] = None) -> torch.Tensor:
    return kotipel_plain.forward(tokens, weights or plain_weights(folder), config or plain_config(folder),
                                 dtype=torch.float64)


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
    """Rows of the plain model's logits that rest on a badly conditioned step: the design divides small vectors by their
    own size (a token input whose gates are all nearly shut, the two mixers' outputs, the read-outs), and there one
    rounding of the inputs turns the result.  Found by running the plain model once more with every floating tensor
    disturbed by a relative 2^-9 (what storing a value in bfloat16 does): rows that move by a quarter of the tolerance."""
    g = torch.Generator().manual_seed(len(tokens))
    W = {k: (v.double() * (1 + 2.0 ** -9 * (2 * torch.rand(v.shape, generator=g, dtype=torch.float64) - 1))
             if v.is_floating_point() else v) for k, v in plain_weights(folder).items()}
    moved = row_distance(kotipel_plain.forward(tokens, W, plain_config(folder), dtype=torch.float64), want)
    return moved > 0.25 * TOLERANCE["bfloat16"]


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
        assert len(keep) < 20 or keep.float().mean().item() >= 0.7, f"{what}: too many rows are badly conditioned"
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
