"""`Robuvik`: a decoder whose layers are listed one by one in config.json, as a `ModelSpec`.

The embedding adds a second row, chosen by a hash of the previous and the current token, to the token's own.  A layer
has ONE norm, and its mixer and feed-forward both read that norm's output: x <- x + mixer(N(x)) + ff(N(x)).  The mixer
is "attention" (grouped-query attention with biases, a rotation of part of every head, a sliding window and a softmax
whose denominator has one more term exp(0)) or "latent_attention" (queries through a normed latent, one normed latent
and one rotated key part per token for all heads, an element-wise output gate).  The feed-forward is absent, dense with
the square of relu, or a mixture of experts whose sigmoid scores multiply the chosen experts' inputs, plus a shared
expert.  Layers `loop.start .. loop.stop - 1` run `loop.times` times in a row with the same weights, every pass on a
cache of its own; before every pass one row of `loop.step` is added to the stream, and before every pass but the first
the embedding's output as well.

Tensor names: `embed`, `bigram`, `loop.step`, `l<i>.norm1`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`, `head`.
"""
from __future__ import annotations

from ..config.robuvik import DenseConfig, ExpertsConfig, RobuvikConfig, WindowAttentionConfig
from ..config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..registry import register_architecture


def _position(rot, head_dim: int, pairing: str):
    if rot is None:
        return None
    scaling = None
    if rot.scaling is not None:
        s = rot.scaling
        scaling = {"rope_type": "yarn", "factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
    return PartSpec("rope", {"head_dim": head_dim, "rot_dim": rot.dims, "theta": rot.base, "scaling": scaling,
                             "pairing": pairing})


def build_robuvik_spec(cfg: RobuvikConfig) -> ModelSpec:
    d = cfg.width
    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m, mlp = f"l{i}.", layer.mixer, layer.mlp
        weights = {"norm.weight": p + "norm1"}
        if isinstance(m, WindowAttentionConfig):
            mixer = PartSpec("rotary_attention", {
                "hidden_size": d, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
                "scale": m.scale, "position": _position(m.rot, m.dim, "half"), "bias": True, "sink": 0.0,
                "window": m.window})
            names = ["q", "k", "v", "q.b", "k.b", "v.b", "o"]
        else:
            mixer = PartSpec("latent_attention", {
                "hidden_size": d, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim,
                "kv_rank": m.kv_rank, "scale": m.scale, "eps": cfg.eps,
                "position": _position(m.rot, m.rot_dim, "adjacent"), "q_rank": m.q_rank, "out_gate": True})
            names = ["dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "g", "o"]
        weights.update({"mixer." + n: p + "mix." + n for n in names})
        parts = {"mixer": mixer, "norm": PartSpec("rmsnorm", {"size": d, "eps": cfg.eps})}
        if isinstance(mlp, DenseConfig):
            parts["ffn"] = PartSpec("dense", {"hidden_size": d, "intermediate_size": mlp.ff,
                                              "activation": "relu_squared"})
            weights.update({"ffn.up": p + "mlp.up", "ffn.down": p + "mlp.down"})
        elif isinstance(mlp, ExpertsConfig):
            parts["ffn"] = PartSpec("routed_experts", {
                "hidden_size": d, "experts": mlp.experts, "top": mlp.top, "expert_size": mlp.ff,
                "shared_size": mlp.shared_ff, "shared_gate": False, "activation": "silu",
                "router_softmax": "sigmoid", "weight_inputs": True})
            names = ["router"] + [f"e{e}.{n}" for e in range(mlp.experts) for n in ("gate", "up", "down")]
            if mlp.shared_ff is not None:
                names += ["shared.gate", "shared.up", "shared.down"]
            weights.update({"ffn." + n: p + "mlp." + n for n in names})
        layers.append(LayerSpec(parts=parts, weights=weights, arrangement="parallel_residual"))
    # every run of a layer works on a cache layer of its own
    run_order = []
    for c, (i, t) in enumerate(cfg.passes()):
        first = t is not None and i == cfg.loop.start
        run_order.append(RunEntry(layer=i, cache=c, writes_cache=True, pass_vector=t if first else None,
                                  adds_embedding=first and t > 0))
    weights = {"embedding.weight": "embed", "final_norm.weight": "final.norm", "lm_head.weight": "head"}
    if cfg.bigram is not None:
        embedding = PartSpec("pair_embedding", {"vocab_size": cfg.vocab, "hidden_size": d, "buckets": cfg.bigram.buckets,
                                                "mul_prev": cfg.bigram.mul_prev, "mul_cur": cfg.bigram.mul_cur})
        weights["embedding.pairs"] = "bigram"
    else:
        embedding = PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": d})
    pass_vectors = None
    if cfg.loop is not None:
        pass_vectors = PartSpec("pass_vectors", {"rows": cfg.loop.times, "hidden_size": d})
        weights["pass_vectors.weight"] = "loop.step"
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=d, embedding=embedding,
        layers=layers, run_order=run_order,
        final_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.eps}),
        lm_head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": d, "tied": False, "shares": None}),
        weights=weights, pass_vectors=pass_vectors,
    )


register_architecture("Robuvik", RobuvikConfig.from_hf_dict, build_robuvik_spec)
