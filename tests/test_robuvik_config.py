"""Robuvik without a GPU: the configuration's round trip and errors, tensor names and shapes, the run order of a
loop, cache and state requests, and the plain implementation against closed forms; and that each mechanism, left out or
moved by one, shifts the plain model's logits by far more than the tests' tolerance."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from serve_amd.config.llama import ConfigError
from serve_amd.config.robuvik import RobuvikConfig
from serve_amd.models.model import Model
from serve_amd.models.robuvik import build_robuvik_spec
from serve_amd.parts.standard import yarn_frequencies
from tests import robuvik_models as rm
from tests.plain import robuvik_plain as rp


@pytest.mark.parametrize("name", list(rm.MODELS))
def test_config_round_trip(name):
    cfg = rm.MODELS[name][0]
    d = cfg.to_hf_dict()
    assert d["architecture"] == "Robuvik"
    again = RobuvikConfig.from_hf_dict(d)
    assert again == cfg and again.to_hf_dict() == d


def test_optional_keys_may_be_absent():
    d = rm.RA.to_hf_dict()
    del d["loop"], d["embedding"]
    del d["layers"][0]["mixer"]["rot"]["scaling"], d["layers"][0]["mixer"]["mask"]
    del d["layers"][2]["mixer"]["rot"]
    del d["layers"][1]["mlp"]["shared"]
    d["layers"][0]["mlp"] = None
    cfg = RobuvikConfig.from_hf_dict(d)
    assert cfg.loop is None and cfg.bigram is None
    assert cfg.layers[0].mixer.rot.scaling is None and cfg.layers[0].mixer.window is None
    assert cfg.layers[2].mixer.rot is None and cfg.layers[1].mlp.shared_ff is None and cfg.layers[0].mlp is None
    spec = build_robuvik_spec(cfg)
    assert spec.pass_vectors is None and spec.embedding.kind == "token_embedding"
    assert [e.pass_vector for e in spec.run_order] == [None] * 3
    names = {r.checkpoint_name for r in Model(spec).weight_requests()}
    assert not names & {"loop.step", "bigram", "l0.mlp.up", "l1.mlp.shared.up"}


@pytest.mark.parametrize("change,message", [
    (lambda d: d["layers"][0].__setitem__("type", "other"), "not supported"),
    (lambda d: d["layers"][0]["mixer"].__setitem__("kv_heads", 3), "multiple"),
    (lambda d: d["layers"][0]["mixer"]["rot"].__setitem__("dims", 34), "fit"),
    (lambda d: d["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "even"),
    (lambda d: d["layers"][0]["mixer"]["mask"].__setitem__("size", 0), "positive"),
    (lambda d: d["layers"][1]["mixer"]["rot"].__setitem__("dims", 4), "whole rotated part"),
    (lambda d: d["layers"][1]["mixer"].pop("q_rank"), "lacks"),
    (lambda d: d["layers"][1]["mlp"]["router"].__setitem__("top", 5), "top"),
    (lambda d: d["layers"][1]["mlp"].__setitem__("kind", "other"), "not supported"),
    (lambda d: d["layers"][0]["mlp"].pop("ff"), "lacks"),
    (lambda d: d["loop"].__setitem__("stop", 4), "loop"),
    (lambda d: d["loop"].__setitem__("times", 0), "loop"),
    (lambda d: d["embedding"]["bigram"].__setitem__("buckets", 0), "buckets"),
    (lambda d: d["layers"][0]["mixer"]["rot"]["scaling"].__setitem__("factor", 0.0), "positive"),
])
def test_config_errors(change, message):
    d = copy.deepcopy(rm.RA.to_hf_dict())
    change(d)
    with pytest.raises(ConfigError, match=message):
        RobuvikConfig.from_hf_dict(d)


def test_tensor_names_run_order_cache_and_state():
    spec = build_robuvik_spec(rm.RA)
    model = Model(spec)
    names = {r.checkpoint_name: r.shape for r in model.weight_requests()}
    assert names["embed"] == (150, 64) and names["bigram"] == (98, 64) and names["loop.step"] == (2, 64)
    assert names["head"] == (150, 64) and names["final.norm"] == (64,) and names["l1.norm1"] == (64,)
    assert names["l0.mix.q"] == (128, 64) and names["l0.mix.k.b"] == (64,) and names["l0.mix.v"] == (32, 64)
    assert names["l0.mix.o"] == (64, 64) and names["l0.mlp.up"] == (96, 64)
    assert names["l1.mix.dq"] == (24, 64) and names["l1.mix.uq"] == (3 * 24, 24) and names["l1.mix.dkv"] == (48, 64)
    assert names["l1.mix.dkv.norm"] == (40,) and names["l1.mix.uk"] == (48, 40) and names["l1.mix.uv"] == (72, 40)
    assert names["l1.mix.g"] == (72, 64) and names["l1.mix.o"] == (64, 72)
    assert names["l1.mlp.router"] == (4, 64) and names["l1.mlp.e3.down"] == (64, 32) and names["l1.mlp.shared.gate"] == (48, 64)
    assert "l2.mlp.shared.gate" not in names and names["l2.mlp.e5.up"] == (40, 64)
    assert not [n for n in names if "norm2" in n]
    # l0, then (l1, l2) twice, every run on a cache layer of its own; the second pass adds the embedding again
    assert [(e.layer, e.cache, e.pass_vector, e.adds_embedding) for e in spec.run_order] == [
        (0, 0, None, False), (1, 1, 0, False), (2, 2, None, False), (1, 3, 1, True), (2, 4, None, False)]
    creq, sreq = model.cache_requests(), model.state_requests()
    assert [None if c is None else c.window for c in creq] == [10, None, 5, None, 5, None]
    assert [t.shape for t in creq[0].tensors] == [(2, 32), (2, 32)]          # keys 32, values 16: one padded head size
    assert [t.shape for t in creq[2].tensors] == [(1, 48), (1, 48)]          # keys 24, values 40
    assert [t.shape for t in creq[1].tensors] == [(1, 48), (1, 48)]          # a latent of 40 and 8 rotated dims
    # the last cache layer is the embedding's: the request's previous token
    assert creq[-1] is None and sreq[-1].shape == (1,) and sreq[-1].dtype == torch.int32 and all(s is None for s in sreq[:-1])
    assert len(Model(build_robuvik_spec(rm.RB)).cache_requests()) == 3       # (no pair table: no state)


def test_stretched_rotation_frequencies():
    """Both implementations against numbers worked out by hand: 8 dims, base 16, factor 4, original 32, fast 4, slow 1."""
    s = {"factor": 4.0, "original": 32.0, "fast": 4.0, "slow": 1.0}
    f, mag = rp.rotary_frequencies(8, 16.0, s)
    plain = [16.0 ** (-2 * i / 8) for i in range(4)]                         # 1, 1/2, 1/4, 1/8
    turn = lambda n: 8 * math.log(32.0 / (2 * math.pi * n)) / (2 * math.log(16.0))      # noqa: E731
    lo, hi = max(math.floor(turn(4.0)), 0), min(math.ceil(turn(1.0)), 7)
    assert (lo, hi) == (0, 3)
    want = [p / 4.0 * r + p * (1 - r) for p, r in zip(plain, [0.0, 1 / 3, 2 / 3, 1.0])]
    assert torch.allclose(f, torch.tensor(want, dtype=torch.float64), rtol=1e-12)
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    f2, mag2 = yarn_frequencies(8, 16.0, dict(s, rope_type="yarn"))
    assert torch.allclose(f2.double(), f, rtol=1e-6) and mag2 == pytest.approx(mag)
    f3, mag3 = rp.rotary_frequencies(8, 16.0, None)
    assert torch.allclose(f3, torch.tensor(plain, dtype=torch.float64)) and mag3 == 1.0


def test_plain_rotation_layouts_and_relative_scores():
    f, mag = rp.rotary_frequencies(4, 10.0, None)
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0]]], dtype=torch.float64)
    a = rp.rotate(x, torch.tensor([3]), f, 1.0, "interleaved")[0, 0]
    c0, s0, c1, s1 = math.cos(3 * f[0]), math.sin(3 * f[0]), math.cos(3 * f[1]), math.sin(3 * f[1])
    assert torch.allclose(a, torch.tensor([1 * c0 - 2 * s0, 2 * c0 + 1 * s0, 3 * c1 - 4 * s1, 4 * c1 + 3 * s1, 5.0], dtype=torch.float64))
    b = rp.rotate(x, torch.tensor([3]), f, 2.0, "half")[0, 0]
    assert torch.allclose(b, torch.tensor([2 * (1 * c0 - 3 * s0), 2 * (2 * c1 - 4 * s1), 2 * (3 * c0 + 1 * s0), 2 * (4 * c1 + 2 * s1), 5.0],
                                          dtype=torch.float64))
    # scores depend on the distance alone, and carry the magnitude twice
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 1, 4, generator=g, dtype=torch.float64), torch.randn(1, 1, 4, generator=g, dtype=torch.float64)
    s = [(rp.rotate(q, torch.tensor([p + 5]), f, 1.5, "half") * rp.rotate(k, torch.tensor([p]), f, 1.5, "half")).sum().item()
         for p in (0, 7, 100)]
    assert s[0] == pytest.approx(s[1]) and s[0] == pytest.approx(s[2])
    plain = (rp.rotate(q, torch.tensor([5]), f, 1.0, "half") * k).sum().item()
    assert s[0] == pytest.approx(1.5 ** 2 * plain)


def test_plain_softmax_with_sink_and_window():
    q = torch.zeros(4, 1, 2, dtype=torch.float64)
    k = torch.zeros(4, 1, 2, dtype=torch.float64)
    v = torch.arange(4, dtype=torch.float64).view(4, 1, 1) + 1.0
    out = rp.softmax_attention(q, k, v, 1.0, None, sink=True)[:, 0, 0]
    # all scores 0: every key and the sink weigh the same
    assert torch.allclose(out, torch.tensor([1 / 2, 3 / 3, 6 / 4, 10 / 5], dtype=torch.float64))
    out = rp.softmax_attention(q, k, v, 1.0, 2, sink=True)[:, 0, 0]         # itself and one token before it
    assert torch.allclose(out, torch.tensor([1 / 2, 3 / 3, 5 / 3, 7 / 3], dtype=torch.float64))
    out = rp.softmax_attention(q, k, v, 1.0, 2, sink=False)[:, 0, 0]
    assert torch.allclose(out, torch.tensor([1.0, 1.5, 2.5, 3.5], dtype=torch.float64))
    out = rp.softmax_attention(q, k, v, 1.0, 1, sink=False)[:, 0, 0]
    assert torch.allclose(out, torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=torch.float64))


def test_plain_router_embedding_and_feed_forwards():
    w = torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]], dtype=torch.float64)
    h = torch.tensor([[2.0, -1.0], [-3.0, 0.5]], dtype=torch.float64)
    ids, s = rp.router(h, w, 2)
    assert ids.tolist() == [[0, 2], [1, 2]]
    sig = lambda z: 1 / (1 + math.exp(-z))                                   # noqa: E731
    assert torch.allclose(s, torch.tensor([[sig(2.0), sig(1.0)], [sig(0.5), sig(-2.5)]], dtype=torch.float64))
    cfg = {"embedding": {"bigram": {"buckets": 7, "mul_prev": 3, "mul_cur": 5}}}
    E = torch.arange(10, dtype=torch.float64).view(10, 1)
    B = 100.0 * torch.arange(8, dtype=torch.float64).view(8, 1)
    x = rp.embedding([4, 9, 9, 0], E, B, cfg)[:, 0]
    assert x.tolist() == [4 + 700, 9 + 100 * ((4 * 3 + 9 * 5) % 7), 9 + 100 * ((9 * 3 + 9 * 5) % 7), 0 + 100 * ((9 * 3) % 7)]
    t = {"up": torch.tensor([[1.0], [-1.0]], dtype=torch.float64), "down": torch.tensor([[1.0, 10.0]], dtype=torch.float64)}
    assert rp.dense_ff(torch.tensor([[3.0], [-2.0]], dtype=torch.float64), t, "")[:, 0].tolist() == [9.0, 40.0]
    t = {"gate": torch.tensor([[1.0]], dtype=torch.float64), "up": torch.tensor([[2.0]], dtype=torch.float64),
         "down": torch.tensor([[1.0]], dtype=torch.float64)}
    assert rp.gated_expert(torch.tensor([[1.5]], dtype=torch.float64), t, "").item() == pytest.approx(1.5 * sig(1.5) * 3.0)
    assert rp.gelu_tanh(torch.tensor(1.0, dtype=torch.float64)).item() == pytest.approx(
        0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * 1.044715)))


def test_every_mechanism_shows_in_the_plain_logits(tmp_path):
    """Leaving a mechanism out, or moving a border by one, moves the plain model's logits by 300 times the float32
    tolerance and more (windows, passes, rotation and pair rows by more than twice the bfloat16 tolerance): a fault of
    that kind in the engine cannot hide behind the tolerances."""
    folder = rm.make_folder(tmp_path, "RAsharp", config=rm.RA, seed=3, scales=rm.SHARP)
    cfg, weights = rm.plain_config(folder), rm.plain_weights(folder)
    tokens = [(7 * i * i + 3 * i + 1) % 150 for i in range(40)]
    want = rm.plain_logits(folder, tokens)

    def moved(config=None, tensors=None, fn=None):
        if fn is not None:
            saved = {n: getattr(rp, n) for n in fn}
            for n, f in fn.items():
                setattr(rp, n, f)
        try:
            got = rm.plain_logits(folder, tokens, config, tensors)
        finally:
            if fn is not None:
                for n, f in saved.items():
                    setattr(rp, n, f)
        return rm.row_distance(got, want)[-12:].max().item()

    bound = 300 * rm.TOLERANCE["float32"]
    for layer, size in ((0, 9), (0, 11), (2, 4), (2, 6)):
        c = copy.deepcopy(cfg)
        c["layers"][layer]["mixer"]["mask"]["size"] = size
        assert moved(c) > 2 * rm.TOLERANCE["bfloat16"], f"window of layer {layer} at {size}"
    c = copy.deepcopy(cfg)
    c["loop"]["times"] = 1
    assert moved(c) > bound
    c = copy.deepcopy(cfg)
    del c["layers"][0]["mixer"]["rot"]["scaling"]
    assert moved(c) > bound
    c = copy.deepcopy(cfg)
    c["embedding"]["bigram"]["mul_prev"] += 1
    assert moved(c) > bound
    c = copy.deepcopy(cfg)
    c["layers"][1]["mlp"]["router"]["top"] = 1
    assert moved(c) > bound
    for name in ("l0.mix.k.b", "l1.mix.g", "l1.mlp.shared.down", "loop.step"):
        w = dict(weights)
        w[name] = torch.zeros_like(w[name])
        assert moved(tensors=w) > bound, name
    soft = rp.softmax_attention
    assert moved(fn={"softmax_attention": lambda q, k, v, s, w, sink: soft(q, k, v, s, w, False)}) > bound      # no sink
    rot = rp.rotate
    assert moved(fn={"rotate": lambda x, p, f, m, layout: rot(x, p, f, 1.0, layout)}) > bound           # no magnitude
    assert moved(fn={"rotate": lambda x, p, f, m, layout: rot(x, p, f, m, "half")}) > bound             # one layout for both
    emb = rp.embedding
    assert moved(fn={"embedding": lambda t, E, B, c: emb(t, E, torch.zeros_like(B), c)}) > bound        # no pair rows
    expert = rp.gated_expert

    def moe_out(h, t, p, mlp):                       # (the weights on the experts' outputs instead of their inputs)
        ids, w = rp.router(h, t[p + "router"], mlp["router"]["top"])
        out = torch.zeros((h.shape[0], t[p + "e0.down"].shape[0]), dtype=torch.float64)
        for tok in range(h.shape[0]):
            for j in range(ids.shape[1]):
                out[tok] += w[tok, j] * expert(h[tok][None], t, f"{p}e{int(ids[tok, j])}.")[0]
        return out + (expert(h, t, p + "shared.") if mlp.get("shared") else 0.0)
    assert moved(fn={"moe_ff": moe_out}) > bound
