"""The Robuvik decoder through the engine against the plain implementation, float32 and bfloat16: whole prompts and
first tokens; prompt then token by token; portions down to two tokens; unequal requests in one batch against each
alone, with pages and slots that are freed and used again; windows' edges with sharp scores, in prompts and in
decoding; a far key among hundreds, at page borders; long decoding; greedy generation through the scheduler; the trace
runner as a program; and the kernels alone."""
from __future__ import annotations

import os
import random
from types import SimpleNamespace

import pytest
import torch

from tests import robuvik_models as rm
from tests.plain import robuvik_plain as rp

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
NAMES = ["RA", "RB", "RC", "RD", "RF"]


def tokens_for(n, seed, vocab):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts_and_first_tokens(tmp_path, name, dtype):
    folder = rm.make_folder(tmp_path, name)
    engine = rm.engine_for(folder, dtype)
    vocab = rm.MODELS[name][0].vocab
    for n in (1, 2, 3, 5, 61):
        tokens = tokens_for(n, 100 + n, vocab)
        got = rm.run_portions(engine, f"r{n}", tokens, [n])
        rm.assert_matches_plain(got, folder, tokens, dtype, f"{name} whole {n}")
    engine.runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_token_by_token(tmp_path, name, dtype):
    folder = rm.make_folder(tmp_path, name)
    engine = rm.engine_for(folder, dtype)
    vocab = rm.MODELS[name][0].vocab
    tokens = tokens_for(84, 7, vocab)
    got = rm.run_portions(engine, "r", tokens, [84 - 45] + [1] * 45)
    rm.assert_matches_plain(got, folder, tokens, dtype, f"{name} prompt + 45 single tokens")
    got = rm.run_portions(engine, "s", tokens[:30], [1] * 30)             # from the very first token on
    rm.assert_matches_plain(got, folder, tokens, dtype, f"{name} token by token from the start", rows=slice(0, 30))
    if dtype == "float32":
        whole = rm.run_portions(engine, "w", tokens, [84])
        assert rm.row_distance(got, whole[:30]).max().item() <= 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES + ["RE"])
def test_portions_of_changing_size(tmp_path, name, dtype):
    folder = rm.make_folder(tmp_path, name)
    engine = rm.engine_for(folder, dtype)
    vocab = rm.MODELS[name][0].vocab
    tokens = tokens_for(73, 8, vocab)
    for portions in ([7, 2, 16, 3, 2, 9, 2, 11, 5, 4, 1, 1, 2, 8], [2] * 10 + [53], [1, 3, 69], [40, 33]):
        got = rm.run_portions(engine, "r", tokens, portions)
        rm.assert_matches_plain(got, folder, tokens, dtype, f"{name} portions {portions}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_windows_edges_with_sharp_scores(tmp_path, dtype):
    """Queries and keys drawn wide, so that a key just inside or just outside a window (10 and 5 tokens, a page holds 4)
    carries weight: the plain model moves by more than twice the bfloat16 tolerance when a window is one off (see
    test_robuvik_config.py).  Portions that end before, at and behind the windows' edges, and single tokens far
    beyond them; pages that the windows have passed go back to the pool on the way."""
    folder = rm.make_folder(tmp_path, "RAsharp", config=rm.RA, seed=3, scales=rm.SHARP)
    engine = rm.engine_for(folder, dtype, num_pages=48, page_size=4)
    tokens = tokens_for(90, 21, rm.RA.vocab)
    for portions in ([90], [4, 1, 5, 1, 9, 10, 11, 2, 3] + [1] * 44, [9, 2] + [1] * 30 + [49], [5] * 18):
        got = rm.run_portions(engine, "r", tokens, portions)
        rm.assert_matches_plain(got, folder, tokens, dtype, f"sharp windows, portions {portions[:9]}...")
    engine.runner.cache.check_invariants()


def mixed_trace(rng, reqs, max_live=4):
    """Up to `max_live` live requests; portions of some beside single tokens of others; staggered."""
    fed = {k: 0 for k in reqs}
    order, live, steps, nxt = list(reqs), [], [], 0
    while nxt < len(order) or live:
        while len(live) < max_live and nxt < len(order) and (not live or rng.random() < 0.6):
            live.append(order[nxt])
            nxt += 1
        entries, ended = [], []
        for k in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue                         # left out of this step, goes on later
            n = min(len(reqs[k]) - fed[k], rng.choice([1, 1, 1, 2, 3, 5, 8, 13]))
            entries.append((k, reqs[k][fed[k]: fed[k] + n]))
            fed[k] += n
            if fed[k] == len(reqs[k]):
                ended.append(k)
                live.remove(k)
        if entries:
            steps.append((entries, ended))
    return steps


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_requests_together_with_pages_and_slots_used_again(tmp_path, name, dtype):
    from serve_amd.engine.batch import Segment
    folder = rm.make_folder(tmp_path, name)
    lengths = [23, 41, 9, 30, 17, 2, 36, 1, 40, 28, 33, 5]
    # four live requests of at most 41 tokens: pool and slots are far fewer than the requests need together
    engine = rm.engine_for(folder, dtype, num_pages=4 * 11 + 1, page_size=4, max_requests=4)
    vocab = rm.MODELS[name][0].vocab
    reqs = {f"q{i}": tokens_for(n, 300 + i, vocab) for i, n in enumerate(lengths)}
    steps = mixed_trace(random.Random(13), reqs)
    rows = {k: [] for k in reqs}
    slots_seen, pages_seen = {}, {}
    for entries, ended in steps:
        segs = []
        for k, toks in entries:
            if k not in engine.runner.cache:
                assert engine.runner.admit(k)
                slots_seen.setdefault(engine.runner.cache.slot_of(k), []).append(k)
            segs.append(Segment(k, toks, list(range(len(toks)))))
        logits = engine.step(segs)
        at = 0
        for k, toks in entries:
            rows[k].append(logits[at: at + len(toks)])
            at += len(toks)
            for page in engine.runner.cache.block_table(k, 0):
                pages_seen.setdefault(page, set()).add(k)
        for k in ended:
            engine.runner.release(k)
        engine.runner.cache.check_invariants()
    assert any(len(v) > 1 for v in slots_seen.values()), "no slot was used twice"
    assert any(len(v) > 1 for v in pages_seen.values()), "no page went from one request to another"
    for k, toks in reqs.items():
        rm.assert_matches_plain(torch.cat(rows[k]), folder, toks, dtype, f"{name} request {k} in the mix")


def far_key_model(tmp_path, n, far):
    """One attention layer without a window and an embedding table made so that one score stands out: the row of token
    1 is set so that, behind the layer's norm, its query matrix (the queries' bias is zero here) and the rotation to
    position n - 1, the queries of both heads point along the rotated key of token 0 at position `far`.  A sequence that
    ends in token 1 and holds token 0 once, at `far`, then reads that key with nearly all of its weight.  The pair rows
    are zero, so that a token's row does not depend on the one before it."""
    from safetensors.torch import save_file
    cfg = rm.RobuvikConfig(vocab=90, width=64, eps=1e-5, bigram=rm.BigramConfig(11, 2, 3), loop=None, layers=(
        rm.L(rm.ATT(2, 1, 16, 16, 3.0, rm.RotConfig(1000.0, 8, rm.YarnScaling(2.0, 256.0, 4.0, 1.0)), None), None),))
    folder = rm.make_folder(tmp_path, f"far{far}", config=cfg, seed=11, scales={r"^bigram$": 0.0, r"q\.b$": 0.0, r"mix\.o$": 4.0})
    W = {k: v.double() for k, v in rm.plain_weights(folder).items()}
    f, mag = rp.rotary_frequencies(8, 1000.0, cfg.layers[0].mixer.rot.scaling.to_dict())
    h0 = rp.rms_norm(W["embed"][0:1], W["l0.norm1"], 1e-5)
    k0 = (h0 @ W["l0.mix.k"].T + W["l0.mix.k.b"]).view(1, 1, 16)
    k_at = rp.rotate(k0, torch.tensor([far]), f, mag, "half")
    q_plain = rp.rotate(k_at, torch.tensor([-(n - 1)]), f, 1.0, "half")[0, 0]      # turning it to n - 1 gives k_at's direction
    h1 = torch.linalg.pinv(W["l0.mix.q"]) @ torch.cat([q_plain, q_plain])
    row = h1 / W["l0.norm1"]
    out = rm.plain_weights(folder)
    out["embed"][1] = (0.8 * row / row.pow(2).mean().sqrt()).to(out["embed"].dtype)     # (as large as the other rows)
    save_file({k: v.contiguous() for k, v in out.items()}, os.path.join(folder, "model.safetensors"))
    return folder


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_among_hundreds(tmp_path, dtype):
    rng = random.Random(5)
    n = 420
    for far in (3, 37, 203):                  # in the first page, further on, and the last key of a page (page size 4)
        folder = far_key_model(tmp_path, n, far)
        with_key = [rng.randrange(2, 90) for _ in range(n - 1)] + [1]
        with_key[far] = 0
        without = list(with_key)
        without[far] = 2
        want = rm.plain_logits(folder, with_key)[-1:]
        # losing that one key would move the last row by far more than the tolerance
        assert rm.row_distance(rm.plain_logits(folder, without)[-1:], want).item() > 2 * rm.TOLERANCE["bfloat16"]
        engine = rm.engine_for(folder, dtype, num_pages=120, page_size=4)
        got = rm.run_portions(engine, "r", with_key, [n - 3, 1, 1, 1])[-1:]
        rm.assert_rows_close(got, want, dtype, f"key {far} of {n}, read by a token decoded alone")
        got = rm.run_portions(engine, "r", with_key, [200, 220])[-1:]
        rm.assert_rows_close(got, want, dtype, f"key {far} of {n}, read from a portion")


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_attention_over_hundreds_of_keys_with_sharp_scores(tmp_path, dtype):
    """Latent attention has no window: with queries and keys drawn wide every query puts its weight on a few keys
    anywhere in the 300 tokens before it, so keys lost far back, or at a page's border, would show in many rows."""
    cfg = rm.RobuvikConfig(vocab=97, width=64, eps=1e-5, bigram=rm.BigramConfig(31, 3, 2), loop=None, layers=(
        rm.L(rm.LAT(4, 16, 8, 16, 32, 24, 0.3, rm.RotConfig(200.0, 8, rm.YarnScaling(2.0, 64.0, 8.0, 1.0))), None),))
    folder = rm.make_folder(tmp_path, "latsharp", config=cfg, seed=17, scales=dict(rm.SHARP, **{r"mix\.o$": 3.0}))
    tokens = tokens_for(300, 41, 97)
    want = rm.plain_logits(folder, tokens)
    soft = rp.softmax_attention
    try:                                        # (what losing the keys more than 100 back would do to the last rows)
        rp.softmax_attention = lambda q, k, v, scale, window, sink: soft(q, k, v, scale, 100, sink)
        short = rm.plain_logits(folder, tokens)
    finally:
        rp.softmax_attention = soft
    assert rm.row_distance(short[-50:], want[-50:]).median().item() > 2 * rm.TOLERANCE["bfloat16"]
    engine = rm.engine_for(folder, dtype, num_pages=90, page_size=4)
    got = rm.run_portions(engine, "r", tokens, [250] + [1] * 30 + [20])
    rm.assert_matches_plain(got, folder, tokens, dtype, "sharp latent attention over 300 keys")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["RA", "RB"])
def test_long_decoding(tmp_path, name, dtype):
    folder = rm.make_folder(tmp_path, name)
    engine = rm.engine_for(folder, dtype, num_pages=80)
    vocab = rm.MODELS[name][0].vocab
    tokens = tokens_for(260, 31, vocab)
    got = rm.run_portions(engine, "r", tokens, [4] + [1] * 256)
    rm.assert_matches_plain(got, folder, tokens, dtype, f"{name} 256 single tokens")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["RA", "RC"])
def test_greedy_generation_through_the_scheduler(tmp_path, name, dtype):
    """`generate` (scheduler, mixed steps, graphs, steps launched ahead of the host) picks the tokens the plain model
    picks, as long as the plain model's choice is clear."""
    from serve_amd.engine.engine import Request
    folder = rm.make_folder(tmp_path, name)
    engine = rm.engine_for(folder, dtype, num_pages=128, page_size=8, max_requests=3)
    vocab = rm.MODELS[name][0].vocab
    prompts = [tokens_for(n, 50 + n, vocab) for n in (5, 19, 1, 33, 8)]
    new = 12
    reqs = [Request(torch.tensor(p), len(p), new) for p in prompts]
    out = engine.generate(reqs, temperature=0.0, return_logits="all")
    compared = 0
    for p, o in zip(prompts, out):
        assert o.error is None and len(o.generated_tokens) == new
        seq = list(p)
        for i, tok in enumerate(o.generated_tokens.tolist()):
            row = rm.plain_logits(folder, seq)[-1]
            top2 = row.topk(2).values
            if (top2[0] - top2[1]).item() < (1e-3 if dtype == "float32" else 0.15) * row.std().item():
                break                            # the plain model's own choice is a close call: stop comparing
            assert tok == int(row.argmax()), f"{name}: token {i} after a prompt of {len(p)}"
            if dtype == "float32":
                rm.assert_rows_close(o.logits[i: i + 1], row[None], dtype, f"{name} logits of generated token {i}")
            seq.append(tok)
            compared += 1
    assert compared >= (new if dtype == "float32" else 5)
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.free_slots() == 3
    # without the logits the scheduler samples on the device and replays decode steps from graphs, and the embedding
    # takes the tokens (and the ones before them) from the device: the same tokens
    again = engine.generate([Request(torch.tensor(p), len(p), new) for p in prompts], temperature=0.0)
    if dtype == "float32":
        assert [o.generated_tokens.tolist() for o in again] == [o.generated_tokens.tolist() for o in out]


@pytest.mark.parametrize("dtype", DTYPES)
def test_traces_through_the_program(tmp_path, dtype):
    """`bin/trace_run` as a child process on a model folder: whole prompts, prompt then single tokens, portions, and a
    mix of four live requests (four state slots, pages for 256 tokens), against the plain model."""
    import json
    import subprocess
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    name = "RA"
    folder = rm.make_folder(tmp_path, name)
    vocab = rm.MODELS[name][0].vocab
    reqs, steps = {}, []

    def feed(key, n, portions, seed):
        reqs[key] = tokens_for(n, seed, vocab)
        at = 0
        for j, m in enumerate(portions):
            steps.append(([(key, reqs[key][at: at + m])], [key] if j == len(portions) - 1 else []))
            at += m
        assert at == n
    feed("whole", 50, [50], 1)
    feed("tail", 70, [30] + [1] * 40, 2)
    feed("cut", 61, [7, 2, 16, 3, 2, 9, 2, 11, 5, 4], 3)
    mixed = {f"m{i}": tokens_for(n, 40 + i, vocab) for i, n in enumerate([23, 41, 9, 30, 17, 2, 36, 12, 40])}
    reqs.update(mixed)
    steps.extend(mixed_trace(random.Random(5), mixed))
    lines = [json.dumps({"step": i, "entries": [{"id": k, "tokens": t, "want": list(range(len(t)))} for k, t in entries],
                         "end": ended}) for i, (entries, ended) in enumerate(steps)]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                           "--max-tokens", "256"], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(steps))]
    rows = {k: [] for k in reqs}
    for i, (entries, _) in enumerate(steps):
        arr = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(sum(len(t) for _, t in entries), vocab))
        at = 0
        for k, t in entries:
            rows[k].append(arr[at: at + len(t)])
            at += len(t)
    assert sum(len(t) for t in reqs.values()) > 256          # pages went from request to request
    for k, t in reqs.items():
        rm.assert_matches_plain(torch.cat(rows[k]), folder, t, dtype, f"trace request {k}")


# ---------------------------------------------------------------------------------------------
# the kernels alone
# ---------------------------------------------------------------------------------------------
def _step(lens, slots, positions0, tokens, dev="cuda"):
    """A step's index arrays for segments of the given lengths: what the embedding's kernel reads."""
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    seg = [i for i, n in enumerate(lens) for _ in range(n)]
    pos = [p + j for p, n in zip(positions0, lens) for j in range(n)]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)          # noqa: E731
    return SimpleNamespace(token_ids=i32(tokens), positions=i32(pos), seg_of_token=i32(seg), cu_q=i32(cu),
                           state_slots=i32(slots), src_row=None, prev_tokens=None)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d", [50, 64, 512])
def test_pair_embedding_over_steps(dtype, d):
    """Two requests over three steps (a portion, single tokens, a portion that starts a new request in a slot that was
    used before), a segment of no request, and tokens that come from the device."""
    from serve_amd import ops
    V, buckets, mp, mc = 37, 11, 5, 3
    g = torch.Generator().manual_seed(d)
    E = torch.randn(V, d, generator=g).to(dtype).cuda()
    B = torch.randn(buckets + 1, d, generator=g).to(dtype).cuda()
    last = torch.full((3, 1), 7, dtype=torch.int32, device="cuda")          # (stale values: position 0 must not read them)

    def want(seqs):
        rows = []
        for prev, toks, pos0 in seqs:
            for j, t in enumerate(toks):
                p = prev if j == 0 else toks[j - 1]
                r = buckets if pos0 + j == 0 or p is None else (p * mp + t * mc) % buckets
                rows.append(E[t].float() + B[r].float())
        return torch.stack(rows)

    a, b, c = [3, 36, 0, 5, 5], [9, 1, 2], [30, 31]
    x, keep = torch.empty(6, d, device="cuda"), torch.empty(6, d, device="cuda")
    ops.pair_embed(E, B, _step([4, 2], [2, 0], [0, 0], a[:4] + b[:2]), last, x, mp, mc, keep)
    assert torch.equal(x, want([(None, a[:4], 0), (None, b[:2], 0)])) and torch.equal(keep, x)
    assert last[:, 0].tolist() == [b[1], 7, a[3]]
    # single tokens, one of them sampled on the device (its id in the step's array is a placeholder), and an inert row
    step = _step([1, 1, 1], [0, -1, 2], [2, 5, 4], [b[2], 8, 0])
    step.src_row = torch.tensor([-1, -1, 1], dtype=torch.int32, device="cuda")
    step.prev_tokens = torch.tensor([0, a[4], 0], dtype=torch.int32, device="cuda")
    x = torch.empty(3, d, device="cuda")
    ops.pair_embed(E, B, step, last, x, mp, mc)
    assert torch.equal(x, want([(b[1], b[2:3], 2), (None, [8], 5), (a[3], a[4:5], 4)]))
    assert last[:, 0].tolist() == [b[2], 7, a[4]]
    # a new request in slot 2 (its first token reads nothing of the slot's past), the other goes on with a portion
    x = torch.empty(4, d, device="cuda")
    ops.pair_embed(E, B, _step([2, 2], [2, 0], [0, 3], c + [4, 4]), last, x, mp, mc)
    assert torch.equal(x, want([(None, c, 0), (b[2], [4, 4], 3)]))
    assert last[:, 0].tolist() == [4, 7, c[1]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv,Dp,rot,adjacent,T", [
    (4, 2, 32, 16, 32, 16, False, 11), (6, 1, 24, 40, 48, 24, False, 11), (3, 3, 10, 7, 16, 4, True, 11),
    (2, 1, 136, 24, 144, 64, False, 11), (2, 2, 16, 16, 16, 0, False, 11), (5, 5, 8, 8, 16, 8, True, 11),
    (4, 2, 32, 16, 32, 16, False, 300), (8, 2, 64, 64, 64, 64, False, 1100), (2, 1, 48, 40, 48, 32, False, 600)])
def test_bias_rope_kv_write(dtype, H, G, D, Dv, Dp, rot, adjacent, T):
    """Both kernels (an element a thread; for bfloat16 at sizes that are multiples of 8, eight dims a thread and the
    values through LDS, with 1, 2, 4 and 8 tokens a workgroup), with and without biases, with slots that store nothing."""
    from serve_amd import ops
    page = 4
    P = (T + 30) // page + 2
    g = torch.Generator().manual_seed(H * D + rot + T)
    cols = H * D + G * (D + Dv)
    z = torch.randn(T, cols + (8 if H % 2 == 0 else 5), generator=g).to(dtype).cuda()       # (rows wider than what is read)
    bias = torch.randn(cols, generator=g).cuda()
    pos_l = [0, 1, 2, 3, 40, 41, 42, 300, 7, 8, 9] if T == 11 else [(5 * t) % 310 for t in range(T)]
    slot_l = [0, 1, 2, 3, 20, 21, 22, -1, 9, 10, 11] if T == 11 else [-1 if t % 97 == 5 else t + 12 for t in range(T)]
    pos = torch.tensor(pos_l, dtype=torch.int32, device="cuda")
    slots = torch.tensor(slot_l, dtype=torch.int32, device="cuda")
    f, mag = (rp.rotary_frequencies(rot, 100.0, {"factor": 3.0, "original": 16.0, "fast": 4.0, "slow": 1.0})
              if rot else (torch.zeros(0, dtype=torch.float64), 1.0))
    inv = f.float().cuda()
    for with_bias in (True, False):
        k_pages = torch.full((P, G, page, Dp), 9.0, dtype=dtype, device="cuda")
        v_pages = torch.full((P, G, Dp, page), 9.0, dtype=dtype, device="cuda")
        q = torch.full((T, H * Dp), 9.0, dtype=dtype, device="cuda")
        ops.bias_rope_kv_write(z, q, pos, slots, k_pages, v_pages, bias if with_bias else None, inv if rot else None,
                               rot, adjacent, mag, H, G, D, Dv)
        zz = z[:, :cols].double().cpu() + (bias.double().cpu() if with_bias else 0.0)
        layout = "interleaved" if adjacent else "half"
        wq = rp.rotate(zz[:, : H * D].reshape(T, H, D), pos.cpu(), f, mag, layout) if rot else zz[:, : H * D].reshape(T, H, D)
        wk = zz[:, H * D: (H + G) * D].reshape(T, G, D)
        wk = rp.rotate(wk, pos.cpu(), f, mag, layout) if rot else wk
        wv = zz[:, (H + G) * D:].reshape(T, G, Dv)
        # (float32: the angle itself, position times frequency, is rounded to 24 bits)
        tol = dict(atol=1e-4, rtol=2e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)
        qq = q.view(T, H, Dp).double().cpu()
        assert torch.allclose(qq[..., :D], wq, **tol) and (qq[..., D:] == 0).all()
        stored = [t for t in range(T) if slot_l[t] >= 0]
        st = torch.tensor([slot_l[t] for t in stored])
        kk = k_pages.double().cpu()[st // page, :, st % page]                    # [n, G, Dp]
        vv = v_pages.double().cpu()[st // page, :, :, st % page]                 # [n, G, Dp]
        assert torch.allclose(kk[..., :D], wk[stored], **tol) and (kk[..., D:] == 0).all()
        assert torch.allclose(vv[..., :Dv], wv[stored], **tol) and (vv[..., Dv:] == 0).all()
        # slots that nobody named are untouched
        used = torch.zeros(P * page, dtype=torch.bool)
        used[st] = True
        free = (~used).nonzero()[:, 0]
        assert (k_pages.cpu()[free // page, :, free % page] == 9).all()
        assert (v_pages.cpu()[free // page, :, :, free % page] == 9).all()
        q2 = torch.empty_like(q)
        ops.bias_rope_kv_write(z, q2, pos, None, None, None, bias if with_bias else None, inv if rot else None, rot,
                               adjacent, mag, H, G, D, Dv)
        assert torch.equal(q2, q)


@pytest.mark.parametrize("M", [1, 5, 40, 128])
@pytest.mark.parametrize("H,G,D", [(4, 2, 32), (3, 1, 16), (8, 2, 64), (2, 2, 128)])
def test_fused_product_with_biases_and_a_stretched_rotation(M, H, G, D):
    """The bfloat16 product whose epilogue adds biases to the fp32 sums, rotates whole heads with a magnitude and
    writes queries, keys and values to their places, against the plain computation."""
    from serve_amd import ops
    K, page, P = 64, 4, 40
    g = torch.Generator().manual_seed(M + D)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn((H + 2 * G) * D, K, generator=g) / K ** 0.5).to(torch.bfloat16).cuda()
    bias = torch.randn((H + 2 * G) * D, generator=g).cuda()
    pos = torch.tensor([(7 * t) % 150 for t in range(M)], dtype=torch.int32, device="cuda")
    slot_l = [-1 if t % 11 == 3 else t + 6 for t in range(M)]
    slots = torch.tensor(slot_l, dtype=torch.int32, device="cuda")
    f, mag = rp.rotary_frequencies(D, 100.0, {"factor": 3.0, "original": 16.0, "fast": 4.0, "slow": 1.0})
    assert ops.qkv_rope_available(a, w, torch.empty(0, dtype=torch.bfloat16, device="cuda"), D, D, False)
    k_pages = torch.full((P, G, page, D), 9.0, dtype=torch.bfloat16, device="cuda")
    v_pages = torch.full((P, G, D, page), 9.0, dtype=torch.bfloat16, device="cuda")
    q = torch.empty((M, H * D), dtype=torch.bfloat16, device="cuda")
    ops.qkv_rope_bf16(a, w, q, pos, f.float().cuda(), slots, k_pages, v_pages, H, G, D, page, bias, mag)
    z = a.double().cpu() @ w.double().cpu().T + bias.double().cpu()
    wq = rp.rotate(z[:, : H * D].reshape(M, H, D), pos.cpu(), f, mag, "half")
    wk = rp.rotate(z[:, H * D: (H + G) * D].reshape(M, G, D), pos.cpu(), f, mag, "half")
    wv = z[:, (H + G) * D:].reshape(M, G, D)
    tol = dict(atol=3e-2, rtol=2e-2)
    assert torch.allclose(q.view(M, H, D).double().cpu(), wq, **tol)
    stored = [t for t in range(M) if slot_l[t] >= 0]
    st = torch.tensor([slot_l[t] for t in stored])
    assert torch.allclose(k_pages.double().cpu()[st // page, :, st % page], wk[stored], **tol)
    assert torch.allclose(v_pages.double().cpu()[st // page, :, :, st % page], wv[stored], **tol)
    used = torch.zeros(P * page, dtype=torch.bool)
    used[st] = True
    free = (~used).nonzero()[:, 0]
    assert (k_pages.cpu()[free // page, :, free % page] == 9).all() and (v_pages.cpu()[free // page, :, :, free % page] == 9).all()


def _plain_experts(h, router_w, wg, wu, wd, top):
    """Sigmoid scores, the largest `top`, each expert applied to score * h; float64."""
    ids, s = rp.router(h, router_w, top)
    out = torch.zeros((h.shape[0], wd.shape[1]), dtype=torch.float64)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            x = s[t, j] * h[t]
            a = x @ wg[e].T
            out[t] += ((a * torch.sigmoid(a)) * (x @ wu[e].T)) @ wd[e].T
    return ids, s, out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,top,d,F", [(5, 4, 2, 64, 32), (40, 6, 1, 64, 40), (40, 5, 2, 50, 9), (700, 8, 2, 64, 64),
                                         (16, 3, 3, 96, 24), (300, 70, 4, 32, 16)])
def test_experts_weighted_on_their_inputs_by_sigmoid_scores(dtype, T, E, top, d, F):
    """Every path of the experts' kernels (routing inside the grouping kernel for few tokens, the matrix-core kernels
    for tiles of 16 and of 64 rows, the vector kernels for float32 and for sizes the matrix cores do not take) with the
    router's sigmoid scores on the experts' inputs, against the plain sum."""
    from serve_amd import ops
    g = torch.Generator().manual_seed(T + E)
    h = torch.randn(T, d, generator=g).to(dtype)
    rw = (0.05 * torch.randn(E, d, generator=g)).to(dtype)         # (scores around one half)
    wg = (torch.randn(E, F, d, generator=g) / d ** 0.5).to(dtype)
    wu = (torch.randn(E, F, d, generator=g) / d ** 0.5).to(dtype)
    wd = (torch.randn(E, d, F, generator=g) / F ** 0.5).to(dtype)
    logits = (h.double() @ rw.double().T).float().cuda()
    ids_w, s_w, want = _plain_experts(h.double(), rw.double(), wg.double(), wu.double(), wd.double(), top)
    # rows whose choice is clear in float32 (the logits were rounded once)
    srt = torch.sort(logits.double().cpu(), dim=-1, descending=True).values
    clear = torch.ones(T, dtype=torch.bool) if top == E else (srt[:, top - 1] - srt[:, top]) > 1e-4
    ids = torch.empty((T, top), dtype=torch.int32, device="cuda")
    wts = torch.empty((T, top), dtype=torch.float32, device="cuda")
    yk = torch.empty((T * top, d), dtype=torch.float32, device="cuda")
    gate_up = torch.stack([wg, wu]).cuda().contiguous()
    hc, wdc = h.cuda(), wd.cuda().contiguous()
    if T <= ops.MOE_ROUTE_INSIDE:
        ops.moe_experts(hc, ids, gate_up[0], gate_up[1], wdc, yk, logits, wts, "sigmoid", 1.0, "silu", 0.0, True)
    else:
        ops.moe_route(logits, E, top, ids, wts, "sigmoid", 1.0)
        ops.moe_experts(hc, ids, gate_up[0], gate_up[1], wdc, yk, weights=wts, weight_inputs=True)
    y = torch.empty((T, d), dtype=torch.float32, device="cuda")
    ops.moe_combine(yk, None, None, None, E, y)
    assert torch.equal(ids.cpu()[clear].long(), ids_w[clear])
    assert torch.allclose(wts.cpu()[clear].double(), s_w[clear], atol=1e-6)
    err = (y.cpu().double() - want)[clear].norm(dim=-1) / want[clear].norm(dim=-1).clamp_min(1e-9)
    assert err.max().item() < (2e-5 if dtype == torch.float32 else 2e-2), err.max().item()
    # the same scores on the outputs instead give another result: the two places are told apart
    ops.moe_combine(yk, wts, None, None, E, y)
    assert ((y.cpu().double() - want)[clear].norm(dim=-1) / want[clear].norm(dim=-1)).median().item() > 0.05


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_stream_add_with_a_second_array_the_squared_relu_and_the_output_gate(dtype):
    from serve_amd import ops
    g = torch.Generator().manual_seed(1)
    for T, d in ((3, 50), (70, 64), (5, 2304)):
        x = torch.randn(T, d, generator=g).cuda()
        y = torch.randn(2, T, d, generator=g).cuda()
        vec, extra = torch.randn(d, generator=g).cuda(), torch.randn(T, d, generator=g).cuda()
        want = x + y[0] + y[1] + extra + vec
        h = torch.empty(T, d, dtype=dtype, device="cuda")
        ops.stream_add(x, y, vec, h, extra)
        assert torch.allclose(x, want, atol=1e-6) and torch.equal(h, x.to(dtype))
        want = x + extra
        ops.stream_add(x, None, None, None, extra)
        assert torch.allclose(x, want, atol=1e-6)
    for n in (7, 4096):
        a = torch.randn(3, n, generator=g).to(dtype).cuda()
        want = (a.float().clamp_min(0) ** 2).to(dtype)
        assert torch.equal(ops.activation(a.clone(), "relu_squared"), want)
        gate = torch.randn(3, n, generator=g).to(dtype).cuda()
        want = (a.float() * torch.sigmoid(gate.float())).to(dtype)
        assert torch.allclose(ops.sigmoid_mul(a.clone(), gate).float(), want.float(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-6,
                              atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_kernels_with_a_magnitude(dtype):
    """The latent cache write and the queries' tail with a rotation whose sine and cosine are stretched."""
    from serve_amd import ops
    T, R, dr, Dp, page, H, K = 7, 20, 8, 32, 4, 3, 12
    g = torch.Generator().manual_seed(2)
    z = torch.randn(T, R + dr, generator=g).to(dtype).cuda()
    w = (1 + 0.1 * torch.randn(R, generator=g)).cuda()
    pos = torch.tensor([0, 1, 5, 9, 100, 3, 4], dtype=torch.int32, device="cuda")
    slots = torch.tensor([0, 1, 2, 3, 8, 9, -1], dtype=torch.int32, device="cuda")
    f, mag = rp.rotary_frequencies(dr, 50.0, {"factor": 4.0, "original": 16.0, "fast": 4.0, "slow": 1.0})
    inv = f.float().cuda()
    k_pages = torch.zeros((4, 1, page, Dp), dtype=dtype, device="cuda")
    v_pages = torch.zeros((4, 1, Dp, page), dtype=dtype, device="cuda")
    ops.latent_kv_write(z, w, pos, inv, slots, k_pages, v_pages, 1e-5, R, dr, mag)
    zz = z.double().cpu()
    c = rp.rms_norm(zz[:, :R], w.double().cpu(), 1e-5)
    kr = rp.rotate(zz[:, R:].view(T, 1, dr), pos.cpu(), f, mag, "half")[:, 0]
    tol = dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)
    for t in range(T - 1):
        s = int(slots[t])
        row = k_pages[s // page, 0, s % page].double().cpu()
        assert torch.allclose(row[:R], c[t], **tol) and torch.allclose(row[R: R + dr], kr[t], **tol) and (row[R + dr:] == 0).all()
        assert torch.allclose(v_pages[s // page, 0, :R, s % page].double().cpu(), c[t], **tol)
    q = torch.randn(T, H * (K + dr), generator=g).to(dtype).cuda()
    wk = (torch.randn(H, K, R, generator=g) / K ** 0.5).to(dtype).cuda()
    out = torch.empty((T, H * Dp), dtype=dtype, device="cuda")
    ops.head_linear(q, H * (K + dr), K + dr, wk, out, H * Dp, Dp, T, pos, inv, dr, Dp - R, mag)
    qq = q.double().cpu().view(T, H, K + dr)
    want = torch.einsum("thk,hkr->thr", qq[..., :K], wk.double().cpu())
    tail = rp.rotate(qq[..., K:].contiguous(), pos.cpu(), f, mag, "half")
    oo = out.double().cpu().view(T, H, Dp)
    assert torch.allclose(oo[..., :R], want, **tol) and torch.allclose(oo[..., R: R + dr], tail, **tol)
    assert (oo[..., R + dr:] == 0).all()
