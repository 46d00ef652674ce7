"""Kotipel without a GPU: the configuration's round trip and errors, tensor names and shapes, the run order of a
loop, cache and state requests, and the plain implementation against closed forms."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from serve_amd.config.kotipel import KotipelConfig
from serve_amd.config.llama import ConfigError
from serve_amd.models.kotipel import build_kotipel_spec
from serve_amd.models.model import Model
from tests import kotipel_models as km
from tests.plain import kotipel_plain as kp


@pytest.mark.parametrize("name", list(km.MODELS))
def test_config_round_trip(name):
    cfg = km.MODELS[name][0]
    d = cfg.to_hf_dict()
    assert d["architecture"] == "Kotipel"
    again = KotipelConfig.from_hf_dict(d)
    assert again == cfg and again.to_hf_dict() == d


def test_optional_keys_may_be_absent():
    d = km.KA.to_hf_dict()
    del d["loop"], d["token_side"]
    del d["layers"][0]["mixer"]["left"]["rot"]["scaling"]
    del d["layers"][2]["mixer"]["left"]["rot"]
    del d["layers"][0]["mixer"]["right"]["decay_rank"]
    cfg = KotipelConfig.from_hf_dict(d)
    assert cfg.loop is None and cfg.side_dim is None
    assert cfg.layers[0].mixer.left.rot_scaling is None and cfg.layers[2].mixer.left.rot_dims == 0
    assert cfg.layers[0].mixer.right.decay_rank is None
    spec = build_kotipel_spec(cfg)
    assert spec.pass_vectors is None and [e.pass_vector for e in spec.run_order] == [None] * 3
    model = Model(spec)
    names = {r.checkpoint_name: r.shape for r in model.weight_requests()}
    assert "loop.step" not in names and "side.embed" not in names and "l0.side.gate" not in names
    assert names["l0.mix.right.a1"] == (-1, 64) and names["l0.mix.right.a2"] == (32, -1)     # the checkpoint says


@pytest.mark.parametrize("change,message", [
    (lambda d: d["layers"][0].__setitem__("type", "other"), "not supported"),
    (lambda d: d["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 3), "multiple"),
    (lambda d: d["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 34), "rot"),
    (lambda d: d["layers"][1]["mixer"].__setitem__("groups", 3), "multiple"),
    (lambda d: d["layers"][1]["mixer"].pop("conv"), "lacks"),
    (lambda d: d["loop"].__setitem__("stop", 4), "loop"),
    (lambda d: d["loop"].__setitem__("times", 0), "loop"),
    (lambda d: d["layers"][0]["mlp"].__setitem__("kind", "moe"), "not supported"),
    (lambda d: d["layers"][0]["mlp"].pop("limit"), "lacks"),
    (lambda d: d["layers"][0]["mixer"]["right"].__setitem__("tau", 0.0), "positive"),
])
def test_config_errors(change, message):
    d = copy.deepcopy(km.KA.to_hf_dict())
    change(d)
    with pytest.raises(ConfigError, match=message):
        KotipelConfig.from_hf_dict(d)


def test_tensor_names_run_order_cache_and_state():
    model = Model(build_kotipel_spec(km.KA))
    names = {r.checkpoint_name: tuple(r.shape) for r in model.weight_requests()}
    assert names["embed"] == (150, 64) and names["side.embed"] == (150, 24) and names["loop.step"] == (2, 64)
    assert names["l0.mix.left.q"] == (128, 64) and names["l0.mix.left.k"] == (64, 64) and names["l0.mix.left.v"] == (32, 64)
    assert names["l0.mix.left.q.norm"] == (128,) and names["l0.mix.left.k.norm"] == (64,) and names["l0.mix.left.g"] == (4, 64)
    assert names["l0.mix.left.o"] == (64, 64) and names["l0.mix.left.out"] == (64,) and names["l0.mix.right.out"] == (64,)
    assert names["l0.mix.right.q"] == (32, 64) and names["l0.mix.right.v"] == (64, 64) and names["l0.mix.right.norm"] == (32,)
    assert names["l0.mix.right.a1"] == (8, 64) and names["l0.mix.right.a2"] == (32, 8) and names["l0.mix.right.a2.b"] == (32,)
    assert names["l1.mix.in"] == (2 * 64 + 2 * 2 * 16 + 4, 64) and names["l1.mix.conv"] == (128, 4)
    assert names["l1.mix.conv.b"] == (128,) and names["l1.mix.norm"] == (64,) and names["l1.mix.D"] == (4,)
    assert names["l2.mlp.gate"] == (80, 64) and names["l2.side.gate"] == (8, 64) and names["l2.side.proj"] == (64, 8)
    assert "l1.mlp.gate" not in names and "l1.norm2" not in names and "head" not in names
    # layers 1 and 2 run twice, each run on a cache layer of its own; a pass begins with its vector
    order = [(e.layer, e.cache, e.pass_vector) for e in model.spec.run_order]
    assert order == [(0, 0, None), (1, 1, 0), (2, 2, None), (1, 3, 1), (2, 4, None)]
    caches, states = model.cache_requests(), model.state_requests()
    assert [c is not None for c in caches] == [True, False, True, False, True]
    assert caches[0].tensors[0].shape == (2, 32) and caches[0].window is None          # keys 32, values 16: heads of 32
    assert all(s is not None and s.dtype == torch.float32 for s in states)
    assert states[1].shape[0] >= 4 * 16 * 16 + 3 * 128 and states[0].shape[0] >= 2 * 16 * 32
    assert model.graph_safe()


def test_random_weights_need_the_decay_rank():
    from serve_amd.weights.loader import random_tensors
    d = km.KB.to_hf_dict()
    del d["layers"][1]["mixer"]["right"]["decay_rank"]
    model = Model(build_kotipel_spec(KotipelConfig.from_hf_dict(d)))
    with pytest.raises(ValueError, match="checkpoint"):
        list(random_tensors(model, 1))


# ---------------------------------------------------------------------------------------------
# the plain implementation against closed forms
# ---------------------------------------------------------------------------------------------
def test_plain_rotary_frequencies():
    f = kp.rotary_frequencies(8, 10000.0, None)
    assert f == pytest.approx([1.0, 0.1, 0.01, 0.001])
    s = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    g = kp.rotary_frequencies(8, 10000.0, s)
    # wavelengths 6.3 (< 16: kept), 62.8 (between 16 and 64: blended), 628 and 6283 (> 64: divided)
    assert g[0] == 1.0 and g[2] == pytest.approx(0.01 / 8) and g[3] == pytest.approx(0.001 / 8)
    smooth = (64 / (2 * math.pi / 0.1) - 1.0) / 3.0
    assert g[1] == pytest.approx((1 - smooth) * 0.1 / 8 + smooth * 0.1)


def test_plain_rotation_keeps_scores_relative():
    torch.manual_seed(0)
    f = kp.rotary_frequencies(6, 100.0, None)
    q, k = torch.randn(1, 1, 8, dtype=torch.float64), torch.randn(1, 1, 8, dtype=torch.float64)
    a = (kp.rotate(q, torch.tensor([7]), f) * kp.rotate(k, torch.tensor([3]), f)).sum()
    b = (kp.rotate(q, torch.tensor([104]), f) * kp.rotate(k, torch.tensor([100]), f)).sum()
    assert a.item() == pytest.approx(b.item(), abs=1e-9)
    assert torch.equal(kp.rotate(q, torch.tensor([9]), f)[..., 6:], q[..., 6:])           # dims beyond the rotated ones


def test_plain_recurrence_closed_form():
    T, dk, dv = 6, 3, 2
    torch.manual_seed(1)
    q, k, v = (torch.randn(T, n, dtype=torch.float64) for n in (dk, dk, dv))
    a = torch.rand(T, dk, dtype=torch.float64)
    o = kp.decayed_recurrence(q, k, v, a)
    for t in range(T):
        want = torch.zeros(dv, dtype=torch.float64)
        for s in range(t + 1):
            w = torch.ones(dk, dtype=torch.float64)
            for r in range(s + 1, t + 1):
                w = w * a[r]
            want += ((q[t] * w * k[s]).sum()) * v[s]
        assert torch.allclose(o[t], want, atol=1e-12)
    one = torch.rand(T, dtype=torch.float64)
    assert torch.allclose(kp.decayed_recurrence(q, k, v, one), kp.decayed_recurrence(q, k, v, one[:, None].expand(T, dk)))


def test_plain_convolution_and_feed_forward():
    x = torch.arange(12, dtype=torch.float64).view(6, 2)
    w = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]], dtype=torch.float64)
    y = kp.causal_conv(x, w, torch.tensor([0.5, 0.0], dtype=torch.float64))
    assert y[0].tolist() == [0.5, 1.0] and y[2, 0].item() == 0.5 + 100 * 4 + 10 * 2 + 0 and y[5, 1].item() == 11.0
    W = {"gate": torch.tensor([[1.0]]), "up": torch.tensor([[1.0]]), "down": torch.tensor([[1.0]])}
    out = kp.clamped_ff(torch.tensor([[5.0], [-5.0]]), W, 2.0)
    assert out[0, 0].item() == pytest.approx(2.0 / (1 + math.exp(-1.702 * 2.0)) * 3.0)
    assert out[1, 0].item() == pytest.approx(-5.0 / (1 + math.exp(1.702 * 5.0)) * (-2.0 + 1.0))


def test_plain_loop_and_losing_the_state_show():
    """What the tests on the GPU rest on: a pass vector left out, a layer's token input left out, or a recurrence
    that starts from zeros in the middle of a sequence moves the logits by far more than the tolerances."""
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        folder = km.make_folder(tmp, "KA")
        W, cfg = km.plain_weights(folder), km.plain_config(folder)
        tokens = [(7 * i + 3) % 150 for i in range(40)]
        want = km.plain_logits(folder, tokens)
        no_step = dict(W)
        no_step["loop.step"] = torch.zeros_like(W["loop.step"])
        assert km.row_distance(km.plain_logits(folder, tokens, weights=no_step), want).min() > 2 * km.TOLERANCE["bfloat16"]
        no_side = dict(W)
        no_side["side.embed"] = torch.zeros_like(W["side.embed"])
        assert km.row_distance(km.plain_logits(folder, tokens, weights=no_side), want).min() > 2 * km.TOLERANCE["bfloat16"]
        once = copy.deepcopy(cfg)
        once["loop"]["times"] = 1
        assert km.row_distance(km.plain_logits(folder, tokens, once), want).min() > 2 * km.TOLERANCE["bfloat16"]
        tail = km.plain_logits(folder, tokens[20:])          # state and keys of the first half lost
        assert km.row_distance(tail, want[20:]).min() > 2 * km.TOLERANCE["bfloat16"]
