"""The Kotipel decoder through the engine against the plain implementation, float32 and bfloat16: whole prompts and
first tokens; prompt then token by token; portions down to two tokens; unequal requests in one batch against each
alone, with pages and slots that are freed and used again; a far key among hundreds, at page borders, in prompts and
in decoding; long decoding; greedy generation through the scheduler; the trace runner as a program; and the kernels
alone."""
from __future__ import annotations

import os
import random
from types import SimpleNamespace

import pytest
import torch

from tests import kotipel_models as km
from tests.plain import kotipel_plain as kp

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
NAMES = ["KA", "KB", "KC", "KD"]


def tokens_for(n, seed, vocab):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts_and_first_tokens(tmp_path, name, dtype):
    folder = km.make_folder(tmp_path, name)
    engine = km.engine_for(folder, dtype)
    vocab = km.MODELS[name][0].vocab
    for n in (1, 2, 3, 5, 61):
        tokens = tokens_for(n, 100 + n, vocab)
        got = km.run_portions(engine, f"r{n}", tokens, [n])
        km.assert_matches_plain(got, folder, tokens, dtype, f"{name} whole {n}")
    engine.runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_token_by_token(tmp_path, name, dtype):
    folder = km.make_folder(tmp_path, name)
    engine = km.engine_for(folder, dtype)
    vocab = km.MODELS[name][0].vocab
    tokens = tokens_for(84, 7, vocab)
    got = km.run_portions(engine, "r", tokens, [84 - 45] + [1] * 45)
    km.assert_matches_plain(got, folder, tokens, dtype, f"{name} prompt + 45 single tokens")
    got = km.run_portions(engine, "s", tokens[:30], [1] * 30)             # from the very first token on
    km.assert_matches_plain(got, folder, tokens, dtype, f"{name} token by token from the start", rows=slice(0, 30))
    if dtype == "float32":
        whole = km.run_portions(engine, "w", tokens, [84])
        assert km.row_distance(got, whole[:30]).max().item() <= 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(tmp_path, name, dtype):
    folder = km.make_folder(tmp_path, name)
    engine = km.engine_for(folder, dtype)
    vocab = km.MODELS[name][0].vocab
    tokens = tokens_for(73, 8, vocab)
    for portions in ([7, 2, 16, 3, 2, 9, 2, 11, 5, 4, 1, 1, 2, 8], [2] * 10 + [53], [1, 3, 69], [40, 33]):
        got = km.run_portions(engine, "r", tokens, portions)
        km.assert_matches_plain(got, folder, tokens, dtype, f"{name} portions {portions}")


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
    folder = km.make_folder(tmp_path, name)
    lengths = [23, 41, 9, 30, 17, 2, 36, 1, 40, 28, 33, 5]
    # four live requests of at most 41 tokens: pool and slots are far fewer than the requests need together
    engine = km.engine_for(folder, dtype, num_pages=4 * 11 + 1, page_size=4, max_requests=4)
    vocab = km.MODELS[name][0].vocab
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
        km.assert_matches_plain(torch.cat(rows[k]), folder, toks, dtype, f"{name} request {k} in the mix")


def far_key_model(tmp_path, n, far):
    """One parallel layer and an embedding table made so that one score of the softmax attention stands out: the row
    of token 1 is set so that, behind the layer's first norm, its query matrix, the norm over the projection and the
    rotation to position n - 1, the queries of both heads point along the rotated key of token 0 at position `far`.  A
    sequence that ends in token 1 and holds token 0 once, at `far`, then reads that key with nearly all of its weight."""
    from safetensors.torch import save_file
    from serve_amd.config.kotipel import KotipelConfig, KotipelLayerConfig, RotScaling
    cfg = KotipelConfig(vocab=90, width=64, eps=1e-5, loop=None, side_dim=None, layers=(
        KotipelLayerConfig(km.par(2, 1, 16, 16, 3.0, 8, 1000.0, RotScaling(2.0, 1.0, 4.0, 256.0), 1, 16, 16, 4.0, 4), None),))
    folder = km.make_folder(tmp_path, f"far{far}", config=cfg, seed=11)
    W = {k: v.double() for k, v in km.plain_weights(folder).items()}
    left = cfg.layers[0].mixer.left.to_dict()
    f = kp.rotary_frequencies(8, 1000.0, left["rot"]["scaling"])
    h0 = kp.rms_norm(W["embed"][0:1], W["l0.norm1"], 1e-5)
    k0 = kp.rms_norm(h0 @ W["l0.mix.left.k"].T, W["l0.mix.left.k.norm"], 1e-5).view(1, 1, 16)
    k_at = kp.rotate(k0, torch.tensor([far]), f)
    q_plain = kp.rotate(k_at, torch.tensor([-(n - 1)]), f)[0, 0]         # rotating it to n - 1 gives k_at
    want_q = torch.cat([q_plain, q_plain]) / W["l0.mix.left.q.norm"]
    h1 = torch.linalg.pinv(W["l0.mix.left.q"]) @ want_q
    row = h1 / W["l0.norm1"]
    out = km.plain_weights(folder)
    out["embed"][1] = (row / row.pow(2).mean().sqrt()).to(out["embed"].dtype)
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
        want = km.plain_logits(folder, with_key)[-1:]
        # losing that one key would move the last row by far more than the tolerance
        assert km.row_distance(km.plain_logits(folder, without)[-1:], want).item() > 2 * km.TOLERANCE["bfloat16"]
        engine = km.engine_for(folder, dtype, num_pages=120, page_size=4)
        got = km.run_portions(engine, "r", with_key, [n - 3, 1, 1, 1])[-1:]
        km.assert_rows_close(got, want, dtype, f"key {far} of {n}, read by a token decoded alone")
        got = km.run_portions(engine, "r", with_key, [200, 220])[-1:]
        km.assert_rows_close(got, want, dtype, f"key {far} of {n}, read from a portion")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["KA", "KB"])
def test_long_decoding(tmp_path, name, dtype):
    folder = km.make_folder(tmp_path, name)
    engine = km.engine_for(folder, dtype, num_pages=80)
    vocab = km.MODELS[name][0].vocab
    tokens = tokens_for(260, 31, vocab)
    got = km.run_portions(engine, "r", tokens, [4] + [1] * 256)
    km.assert_matches_plain(got, folder, tokens, dtype, f"{name} 256 single tokens")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["KA", "KC"])
def test_greedy_generation_through_the_scheduler(tmp_path, name, dtype):
    """`generate` (scheduler, mixed steps, graphs, steps launched ahead of the host) picks the tokens the plain model
    picks, as long as the plain model's choice is clear."""
    from serve_amd.engine.engine import Request
    folder = km.make_folder(tmp_path, name)
    engine = km.engine_for(folder, dtype, num_pages=128, page_size=8, max_requests=3)
    vocab = km.MODELS[name][0].vocab
    prompts = [tokens_for(n, 50 + n, vocab) for n in (5, 19, 1, 33, 8)]
    new = 12
    reqs = [Request(torch.tensor(p), len(p), new) for p in prompts]
    out = engine.generate(reqs, temperature=0.0, return_logits="all")
    compared = 0
    for p, o in zip(prompts, out):
        assert o.error is None and len(o.generated_tokens) == new
        seq = list(p)
        for i, tok in enumerate(o.generated_tokens.tolist()):
            row = km.plain_logits(folder, seq)[-1]
            top2 = row.topk(2).values
            if (top2[0] - top2[1]).item() < (1e-3 if dtype == "float32" else 0.15):
                break                            # the plain model's own choice is a close call: stop comparing
            assert tok == int(row.argmax()), f"{name}: token {i} after a prompt of {len(p)}"
            if dtype == "float32":
                km.assert_rows_close(o.logits[i: i + 1], row[None], dtype, f"{name} logits of generated token {i}")
            seq.append(tok)
            compared += 1
    assert compared >= new
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.free_slots() == 3
    # without the logits the scheduler samples on the device and replays decode steps from graphs: the same tokens
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
    name = "KA"
    folder = km.make_folder(tmp_path, name)
    vocab = km.MODELS[name][0].vocab
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
        km.assert_matches_plain(torch.cat(rows[k]), folder, t, dtype, f"trace request {k}")


# ---------------------------------------------------------------------------------------------
# the kernels alone
# ---------------------------------------------------------------------------------------------
def _ctx(lens, slots):
    T = sum(lens)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    seg = [i for i, n in enumerate(lens) for _ in range(n)]
    dev = dict(dtype=torch.int32, device="cuda")
    return SimpleNamespace(num_tokens=T, num_segments=len(lens), max_q_len=max(lens), q_lens=list(lens),
                           seg_of_token=torch.tensor(seg, **dev), cu_q=torch.tensor(cu, **dev),
                           state_slots=torch.tensor(slots, **dev))


# steps of two requests and a segment of nobody's: short ones go token by token, the others sixteen tokens a pass
# (and the longest are cut into pieces that run side by side, with a chain of states between two passes)
SCAN_STEPS = {"short": [[4, 1, 3], [1, 5, 2]], "mid": [[9, 1, 3], [1, 21, 2]], "long": [[33, 1, 16], [1, 64, 7], [47, 3, 1]],
              "pieces": [[300, 1, 20], [1, 415, 7], [130, 3, 129]]}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("per_channel", [True, False])
@pytest.mark.parametrize("decays", ["mild", "strong"])
@pytest.mark.parametrize("steps", sorted(SCAN_STEPS))
@pytest.mark.parametrize("dk,dv,H,Hk", [(16, 32, 4, 2), (32, 64, 2, 2), (10, 70, 1, 1), (48, 20, 3, 1), (130, 16, 2, 1),
                                        (256, 128, 1, 1), (5, 9, 2, 2), (128, 64, 2, 1), (64, 128, 2, 2)])
def test_decay_scan_over_steps(dk, dv, H, Hk, per_channel, dtype, steps, decays):
    """Two requests over several steps (portions, single tokens) and a segment without a request, against the plain
    recurrence over the whole sequences: the state carries over between the two kernels, lies where it is asked to,
    and nothing else is written.  `strong`: decays down to e^-30 a token, which a pass of sixteen cannot factor."""
    from serve_amd import ops
    torch.manual_seed(dk + dv)
    lens = SCAN_STEPS[steps]
    total = [sum(n[0] for n in lens), sum(n[1] for n in lens)]
    rnd = lambda *s: torch.randn(*s).to(dtype).double()   # noqa: E731  (values the storage type holds)
    q = [rnd(n, Hk * dk) for n in total]
    k = [rnd(n, Hk * dk) for n in total]
    v = [rnd(n, H * dv) for n in total]
    span = 0.7 if decays == "mild" else 30.0
    la = [-(torch.rand(n, H, dk, dtype=torch.float64) if per_channel else torch.rand(n, H, dtype=torch.float64)) ** 3 * span
          for n in total]
    la = [x.float().double() for x in la]            # the logarithms are what the kernel gets
    a = [torch.exp(x) for x in la]
    scale = 0.37
    want = []
    for r in range(2):
        outs = [kp.decayed_recurrence(q[r].view(-1, Hk, dk)[:, i // (H // Hk)] * scale, k[r].view(-1, Hk, dk)[:, i // (H // Hk)],
                                      v[r].view(-1, H, dv)[:, i], a[r][:, i]) for i in range(H)]
        want.append(torch.stack(outs, dim=1).reshape(-1, H * dv))
    need = ops.decay_scan_state_floats(H, dk, dv)
    off = 7
    state = torch.zeros(3, off + need + 5, dtype=torch.float32, device="cuda")
    at, got = [0, 0], [[], []]
    for step in range(len(lens)):
        n = lens[step]
        cat = lambda xs, w: torch.cat([xs[0][at[0]: at[0] + n[0]], xs[1][at[1]: at[1] + n[1]],   # noqa: E731
                                       torch.ones(n[2], w, dtype=torch.float64)])
        wide = torch.cat([cat(q, Hk * dk), cat(k, Hk * dk), cat(v, H * dv)], dim=1).to(dtype).cuda()      # rows inside wider rows
        dec = torch.cat([la[0][at[0]: at[0] + n[0]], la[1][at[1]: at[1] + n[1]], -torch.ones((n[2],) + tuple(a[0].shape[1:]), dtype=torch.float64)])
        ctx = _ctx(n, [2, 0, -1])
        out = torch.full((sum(n), H * dv), 7.0, dtype=torch.float32, device="cuda")
        ops.decay_scan(wide[:, : Hk * dk], wide[:, Hk * dk: 2 * Hk * dk], wide[:, 2 * Hk * dk:], dec.float().cuda().contiguous(),
                       state, off, ctx, out, H, Hk, dk, dv, q_scale=scale)
        got[0].append(out[: n[0]].cpu())
        got[1].append(out[n[0]: n[0] + n[1]].cpu())
        at = [at[0] + n[0], at[1] + n[1]]
    for r in range(2):
        g = torch.cat(got[r]).double()
        assert torch.allclose(g, want[r], atol=2e-5 * want[r].abs().max().item(), rtol=2e-4), \
            f"request {r}: max diff {(g - want[r]).abs().max().item():.3g} at row {(g - want[r]).abs().max(dim=1).values.argmax().item()}"
    assert state[1].abs().max().item() == 0.0, "a slot that no segment named was written"
    assert state[:, :off].abs().max().item() == 0.0 and state[:, off + need:].abs().max().item() == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv,Dp,rot", [(4, 2, 32, 16, 32, 16), (6, 1, 24, 40, 48, 24), (3, 3, 10, 7, 16, 4),
                                             (2, 1, 136, 24, 144, 64), (2, 2, 16, 16, 16, 0)])
def test_row_norm_rope_kv_write_and_head_gate(dtype, H, G, D, Dv, Dp, rot):
    from serve_amd import ops
    torch.manual_seed(D)
    T, page, P = 11, 4, 9
    width = H * D + G * (D + Dv) + H
    wide = torch.randn(T, width + 5, device="cuda").to(dtype)             # rows inside wider rows
    z = wide[:, :width]
    wq, wk = torch.rand(H * D, device="cuda") + 0.5, torch.rand(G * D, device="cuda") + 0.5
    freq = torch.tensor(kp.rotary_frequencies(rot, 100.0, None), dtype=torch.float32, device="cuda") if rot else None
    positions = torch.tensor([0, 1, 2, 3, 4, 5, 6, 7, 300, 301, 1302], dtype=torch.int32, device="cuda")
    slots = torch.tensor([5, 6, 7, 8, 20, 21, 22, 23, -1, 1, 35], dtype=torch.int32, device="cuda")
    k_pages = torch.full((P, G, page, Dp), 7.0, device="cuda").to(dtype)
    v_pages = torch.full((P, G, Dp, page), 7.0, device="cuda").to(dtype)
    q = torch.full((T, H * Dp), 7.0, device="cuda").to(dtype)
    eps = 1e-5
    ops.row_norm_rope_kv_write(z, q, positions, slots, k_pages, v_pages, wq, wk, eps, freq, rot, H, G, D, Dv)
    x = z.double().cpu()
    f = freq.double().cpu().tolist() if rot else []
    pos = positions.cpu().long()
    want_q = kp.rotate(kp.rms_norm(x[:, : H * D], wq.double().cpu(), eps).view(T, H, D), pos, f)
    want_k = kp.rotate(kp.rms_norm(x[:, H * D: (H + G) * D], wk.double().cpu(), eps).view(T, G, D), pos, f)
    want_v = x[:, (H + G) * D: (H + G) * D + G * Dv].view(T, G, Dv)
    tol = dict(atol=2e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=1e-2)
    got_q = q.double().cpu().view(T, H, Dp)
    assert torch.allclose(got_q[:, :, :D], want_q, **tol) and (got_q[:, :, D:] == 0).all()
    kpg, vpg = k_pages.double().cpu(), v_pages.double().cpu()
    written = set()
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        pg, off = divmod(s, page)
        written.add((pg, off))
        assert torch.allclose(kpg[pg, :, off, :D], want_k[t], **tol) and (kpg[pg, :, off, D:] == 0).all()
        assert torch.equal(vpg[pg, :, :Dv, off], want_v[t]) and (vpg[pg, :, Dv:, off] == 0).all()
    for pg in range(P):
        for off in range(page):
            if (pg, off) not in written:
                assert (kpg[pg, :, off] == 7.0).all() and (vpg[pg, :, :, off] == 7.0).all(), "a slot that no token named was written"
    q2 = torch.empty_like(q)
    ops.row_norm_rope_kv_write(z, q2, positions, None, None, None, wq, wk, eps, freq, rot, H, G, D, Dv)     # queries alone
    assert torch.equal(q2, q)
    # the output gate per head, from the last H columns of the same rows
    a = torch.randn(T, H * Dp, device="cuda").to(dtype)
    want = a.double().cpu().view(T, H, Dp) * torch.sigmoid(x[:, width - H:])[:, :, None]
    ops.head_gate(a, z, width - H, H)
    assert torch.allclose(a.double().cpu().view(T, H, Dp), want, atol=1e-6 if dtype == torch.float32 else 2e-2, rtol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d", [50, 64, 2304])
def test_stream_kernels(dtype, d):
    """stream_add, dual_norm_mix and gelu_mul_rows against their formulas."""
    from serve_amd import ops
    torch.manual_seed(d)
    T = 7
    x = torch.randn(T, d, device="cuda")
    parts = torch.randn(3, T, d, device="cuda")
    vec = torch.randn(d, device="cuda")
    want = x.double() + parts.double().sum(0) + vec.double()
    h = torch.empty(T, d, device="cuda", dtype=dtype)
    ops.stream_add(x, parts, vec, h)
    assert torch.allclose(x.double(), want, atol=1e-5) and torch.allclose(h.double(), want, atol=1e-5 if dtype == torch.float32 else 5e-2)
    y = torch.randn(T, d, device="cuda").to(dtype)
    before = x.double().clone()
    ops.stream_add(x, y, None, None)
    assert torch.allclose(x.double(), before + y.double(), atol=1e-5)
    ops.stream_add(x, None, vec, None)
    assert torch.allclose(x.double(), before + y.double() + vec.double(), atol=1e-5)
    a, b = torch.randn(2, T, d, device="cuda") * 3, torch.randn(T, d, device="cuda").to(dtype)
    wa, wb = torch.rand(d, device="cuda") + 0.5, torch.rand(d, device="cuda") + 0.5
    out = torch.empty(T, d, device="cuda")
    ops.dual_norm_mix(a, b, wa, wb, 0.5, 0.25, 1e-5, out)
    want = 0.5 * kp.rms_norm(a.double().sum(0), wa.double(), 1e-5) + 0.25 * kp.rms_norm(b.double(), wb.double(), 1e-5)
    assert torch.allclose(out.double(), want, atol=1e-5, rtol=1e-5)
    n, V = 24, 31
    z = torch.randn(T, n, device="cuda").to(dtype)
    table = torch.randn(V, 3 * n + 1, device="cuda").to(dtype)
    tokens = torch.tensor([0, 30, 5, 5, 17, 2, 9], dtype=torch.int32, device="cuda")
    g = torch.empty_like(z)
    ops.gelu_mul_rows(z, table, n + 1, tokens, g)
    want = kp.gelu_tanh(z.double()) * table.double()[tokens.long(), n + 1: 2 * n + 1]
    assert torch.allclose(g.double(), want, atol=1e-6 if dtype == torch.float32 else 3e-2, rtol=1e-2)
    src = torch.tensor([-1, 1, -1, 0, -1, -1, -1], dtype=torch.int32, device="cuda")
    prev = torch.tensor([8, 3], dtype=torch.int32, device="cuda")
    ops.gelu_mul_rows(z, table, 0, tokens, g, src, prev)
    ids = tokens.long().clone()
    ids[1], ids[3] = 3, 8
    want = kp.gelu_tanh(z.double()) * table.double()[ids, :n]
    assert torch.allclose(g.double(), want, atol=1e-6 if dtype == torch.float32 else 3e-2, rtol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("lens", [[[9, 1], [1, 6]], [[290, 1], [3, 270]]], ids=["short", "long"])
@pytest.mark.parametrize("H,P,N,G,taps,norm_groups", [(4, 16, 16, 2, 4, 2), (3, 32, 8, 1, 2, 3), (2, 9, 5, 2, 1, 1), (5, 64, 16, 1, 16, 1)])
def test_state_space_kernels_in_two_steps(dtype, H, P, N, G, taps, norm_groups, lens):
    """ssm_prepare, conv_state_update, decay_scan and gated_group_norm over two steps against the plain mixer's
    inner part over the whole sequences (the convolution's last inputs and the state carry over).  `long`: steps of
    more than 256 tokens, whose preparation takes runs of eight tokens (inside a segment from loaded windows, at a
    segment's first tokens and where two segments meet one by one)."""
    from serve_amd import ops
    torch.manual_seed(P)
    inner, C = H * P, H * P + 2 * G * N
    total = [lens[0][0] + lens[1][0], lens[0][1] + lens[1][1]]
    zx = [torch.randn(n, inner + C).to(dtype).double() for n in total]
    dt = [torch.randn(n, H).float().double() for n in total]
    f64 = lambda *s: torch.randn(*s).float().double()   # noqa: E731
    conv_w, conv_b = f64(C, taps) * 0.5, f64(C) * 0.1
    A_log, dt_bias, D, norm_w = -torch.rand(H).double(), -torch.rand(H).double(), f64(H), 1 + 0.1 * f64(inner)
    eps = 1e-5
    want = []
    for r in range(2):
        xbc = kp.silu(kp.causal_conv(zx[r][:, inner:], conv_w, conv_b))
        x, B, Cm = xbc[:, :inner].view(-1, H, P), xbc[:, inner: inner + G * N].view(-1, G, N), xbc[:, inner + G * N:].view(-1, G, N)
        step = kp.softplus(dt[r] + dt_bias)
        decay = torch.exp(-torch.exp(A_log) * step)
        ys = [kp.decayed_recurrence(Cm[:, i // (H // G)], B[:, i // (H // G)], step[:, i: i + 1] * x[:, i], decay[:, i])
              + D[i] * x[:, i] for i in range(H)]
        y = torch.stack(ys, dim=1).reshape(-1, inner) * kp.silu(zx[r][:, :inner])
        want.append(kp.grouped_rms_norm(y, norm_w, norm_groups, eps))
    scan = ops.decay_scan_state_floats(H, N, P)
    state = torch.zeros(3, scan + (taps - 1) * C, dtype=torch.float32, device="cuda")
    c = lambda t: t.float().cuda().contiguous()   # noqa: E731
    at, got = [0, 0], [[], []]
    for s in range(2):
        n = lens[s]
        rows = torch.cat([zx[r][at[r]: at[r] + n[r]] for r in range(2)]).to(dtype).cuda()
        raw = c(torch.cat([dt[r][at[r]: at[r] + n[r]] for r in range(2)]))
        T = rows.shape[0]
        ctx = _ctx(n, [2, 0])
        xbc, v, decay = (torch.empty(T, w, dtype=torch.float32, device="cuda") for w in (C, inner, H))
        ops.ssm_prepare(rows, inner, c(conv_w), c(conv_b), state, scan, raw, c(A_log), c(dt_bias), ctx, xbc, v, decay, H, P, taps)
        ops.conv_state_update(rows, inner, C, state, scan, ctx, taps)
        o = torch.empty(T, inner, dtype=torch.float32, device="cuda")
        ops.decay_scan(xbc[:, inner + G * N:], xbc[:, inner: inner + G * N], v, decay, state, 0, ctx, o, H, G, N, P)
        y = torch.empty(T, inner, dtype=dtype, device="cuda")
        ops.gated_group_norm(o, rows, 0, c(norm_w), inner // norm_groups, True, eps, y, skip_x=xbc, skip_d=c(D), head_dim=P)
        got[0].append(y[: n[0]].cpu())
        got[1].append(y[n[0]:].cpu())
        at = [at[0] + n[0], at[1] + n[1]]
    tol = dict(atol=2e-4, rtol=2e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)
    for r in range(2):
        g = torch.cat(got[r]).double()
        assert torch.allclose(g, want[r], **tol), f"request {r}: max diff {(g - want[r]).abs().max().item():.3g}"
    assert state[1].abs().max().item() == 0.0, "a slot that no segment named was written"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gla_decay_and_the_norm_behind_the_read_out(dtype):
    from serve_amd import ops
    torch.manual_seed(3)
    T, H, Dv, C = 9, 3, 20, 48
    z = torch.randn(T, C, device="cuda") * 4
    bias = torch.randn(C, device="cuda") * 3
    out = torch.empty_like(z)
    ops.gla_decay(z, bias, 4.0, out)                                             # the decay's logarithm
    want = torch.sigmoid(z.double() + bias.double()) ** 0.25
    assert torch.allclose(torch.exp(out.double()), want, atol=1e-6, rtol=1e-5)
    big = torch.tensor([[-200.0, 200.0]], device="cuda")
    ops.gla_decay(big, None, 2.0, big)
    assert big[0, 0].item() == -100.0 and big[0, 1].item() == 0.0               # (no overflow on either side)
    o = torch.randn(T, H * Dv, device="cuda")
    rows = torch.randn(T, 11 + H * Dv, device="cuda").to(dtype)
    w = torch.rand(Dv, device="cuda") + 0.5
    y = torch.empty(T, H * Dv, device="cuda", dtype=dtype)
    ops.gated_group_norm(o, rows, 11, w, Dv, False, 1e-5, y)
    want = (kp.rms_norm(o.double().view(T, H, Dv), w.double(), 1e-5).reshape(T, H * Dv) * kp.silu(rows.double()[:, 11:])).cpu()
    assert torch.allclose(y.double().cpu(), want, atol=1e-5 if dtype == torch.float32 else 3e-2, rtol=1e-2)
