"""`Kotipel`: a decoder whose layers are listed one by one in config.json, as a `ModelSpec`.

A layer is pre-norm, x <- x + mixer(N_1(x)); x <- x + ff(N_2(x)) (the second half only if the layer has a
feed-forward), and, where the model has per-layer token inputs, ends with x <- x + N_s(P (gelu(G x) * e)), e being the
layer's slice of a second embedding row of the token.  The mixer is "parallel" (a softmax attention with queries and
keys normed over the whole projection, rotary positions and an output gate per head, beside a gated linear attention;
their normed outputs are averaged) or "mamba2" (a selective state-space mixer).  The feed-forward is gated with a
clamped swish.  Layers `loop.start .. loop.stop - 1` run `loop.times` times in a row with the same weights, every pass
on a cache and state of its own, and before every pass one row of `loop.step` is added to the stream.  The output
matrix is the embedding table.

Tensor names: `embed`, `side.embed`, `loop.step`, `l<i>.norm1|norm2`, `l<i>.mix.*`, `l<i>.mlp.gate|up|down`,
`l<i>.side.gate|proj|norm`, `final.norm`.
"""
from __future__ import annotations

from ..config.kotipel import KotipelConfig, ParallelMixerConfig
from ..config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..registry import register_architecture


def _rope_scaling(s):
    """The configuration's names for the frequency rescaling -> the rotary part's."""
    if s is None:
        return None
    return {"rope_type": "llama3", "factor": s.factor, "low_freq_factor": s.low, "high_freq_factor": s.high,
            "original_max_position_embeddings": s.original}


def build_kotipel_spec(cfg: KotipelConfig) -> ModelSpec:
    d = cfg.width
    n_layers = len(cfg.layers)
    side_width = 0 if cfg.side_dim is None else cfg.side_dim * n_layers
    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m, mlp = f"l{i}.", layer.mixer, layer.mlp
        norm = PartSpec("rmsnorm", {"size": d, "eps": cfg.eps})
        weights = {"mixer_norm.weight": p + "norm1"}
        if isinstance(m, ParallelMixerConfig):
            l, r = m.left, m.right
            position = None
            if l.rot_dims:
                position = PartSpec("rope", {"head_dim": l.dim, "rot_dim": l.rot_dims, "theta": l.rot_base,
                                             "scaling": _rope_scaling(l.rot_scaling), "pairing": "half"})
            left = PartSpec("gated_rotary_attention", {
                "hidden_size": d, "num_heads": l.heads, "num_kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim,
                "scale": l.scale, "eps": cfg.eps, "position": position, "out_gate": True})
            right = PartSpec("gated_linear_attention", {
                "hidden_size": d, "heads": r.heads, "dim": r.dim, "vdim": r.vdim, "tau": r.tau, "eps": cfg.eps,
                "decay_rank": r.decay_rank})          # (None: the checkpoint's tensors say it)
            mixer = PartSpec("parallel", {"hidden_size": d, "eps": cfg.eps, "left": left, "right": right})
            names = (["left." + n for n in ("q", "k", "v", "q.norm", "k.norm", "g", "o", "out")]
                     + ["right." + n for n in ("q", "k", "v", "g", "o", "norm", "a1", "a2", "a2.b", "out")])
        else:
            mixer = PartSpec("state_space", {"hidden_size": d, "heads": m.heads, "vdim": m.vdim, "state": m.state,
                                             "groups": m.groups, "conv": m.conv, "norm_groups": m.norm_groups,
                                             "eps": cfg.eps})
            names = ["in", "conv", "conv.b", "dt_bias", "A_log", "D", "norm", "o"]
        weights.update({"mixer." + n: p + "mix." + n for n in names})
        parts = {"mixer": mixer, "mixer_norm": norm}
        if mlp is not None:
            parts.update(ffn_norm=norm, ffn=PartSpec("gated", {"hidden_size": d, "intermediate_size": mlp.ff,
                                                               "activation": "clamped_swish", "limit": mlp.limit}))
            weights.update({"ffn_norm.weight": p + "norm2", "ffn.gate_proj.weight": p + "mlp.gate",
                            "ffn.up_proj.weight": p + "mlp.up", "ffn.down_proj.weight": p + "mlp.down"})
        if cfg.side_dim is not None:
            parts["token_input"] = PartSpec("gated_side_embedding", {
                "hidden_size": d, "vocab_size": cfg.vocab, "table_width": side_width, "offset": i * cfg.side_dim,
                "dim": cfg.side_dim, "eps": cfg.eps})
            weights.update({"token_input.gate": p + "side.gate", "token_input.proj": p + "side.proj",
                            "token_input.norm": p + "side.norm", "token_input.table": "side.embed"})
        layers.append(LayerSpec(parts=parts, weights=weights, arrangement="prenorm_residual"))
    # every run of a layer works on a cache layer of its own
    run_order = []
    for c, (i, t) in enumerate(cfg.passes()):
        first = t is not None and i == cfg.loop.start
        run_order.append(RunEntry(layer=i, cache=c, writes_cache=True, pass_vector=t if first else None))
    weights = {"embedding.weight": "embed", "final_norm.weight": "final.norm", "lm_head.weight": "embed"}
    if side_width:
        weights["embedding.side"] = "side.embed"
    pass_vectors = None
    if cfg.loop is not None:
        pass_vectors = PartSpec("pass_vectors", {"rows": cfg.loop.times, "hidden_size": d})
        weights["pass_vectors.weight"] = "loop.step"
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=d,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": d, "side_width": side_width}),
        layers=layers, run_order=run_order,
        final_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.eps}),
        lm_head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": d, "tied": True,
                                         "shares": "embedding.weight"}),
        weights=weights, pass_vectors=pass_vectors,
        # a layer without feed-forward may still carry the norm in front of one: nothing reads it
        ignored_weight_patterns=[r"l\d+\.norm2"],
    )


register_architecture("Kotipel", KotipelConfig.from_hf_dict, build_kotipel_spec)
