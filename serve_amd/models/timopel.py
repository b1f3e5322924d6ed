"""`Timopel`: a decoder of attention layers that are listed one by one in config.json, as a `ModelSpec`.

With one constant c (`residual_mult`) and plain RMS norms N a layer is

    x <- x + c * N_1b(mixer(N_1(x)));   x <- x + c * N_2b(ff(N_2(x)))

(the second half only if the layer has a feed-forward).  The mixer is a grouped-query attention without
rotation whose queries and keys are normed per head, with a query temperature that grows with the
position, a learned sink in every head's softmax, and values that are blended with those of the first
layer that takes part in the blending (`v_mix`).  The feed-forward is absent, dense and gated (gelu, tanh
form), or a mixture of experts with clamped gates, routed by the renormalised softmax over all experts,
plus an optional shared expert.  The embedding is scaled on its way into the stream; the output matrix is
the embedding table itself.

Tensor names: `embed`, `l<i>.norm1|norm1b|norm2|norm2b`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`.
"""
from __future__ import annotations

from ..config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..config.timopel import ClampedMoeConfig, GatedDenseConfig, TimopelConfig
from ..registry import register_architecture


def build_timopel_spec(cfg: TimopelConfig) -> ModelSpec:
    d = cfg.width
    layers, run_order = [], []
    source = None                          # the first layer that takes part in the blending of values
    for i, layer in enumerate(cfg.layers):
        p, m, mlp = f"l{i}.", layer.mixer, layer.mlp
        before = PartSpec("rmsnorm", {"size": d, "eps": cfg.eps})
        after = PartSpec("scaled_output_rmsnorm", {"size": d, "eps": cfg.eps, "constant_scale": cfg.residual_mult})
        blend = "none"
        if m.v_mix:
            blend = "source" if source is None else "blend"
            source = i if source is None else source
        mixer = PartSpec("qk_norm_attention", {
            "hidden_size": d, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
            "scale": m.scale, "eps": cfg.eps, "q_temp_coef": m.q_temp.coef if m.q_temp else 0.0,
            "q_temp_every": m.q_temp.every if m.q_temp else 0, "sink": True, "v_blend": blend})
        names = ["q", "k", "v", "q.norm", "k.norm", "sink", "o"] + (["vmix"] if m.v_mix else [])
        weights = {"mixer_norm.weight": p + "norm1", "mixer_out_norm.weight": p + "norm1b"}
        weights.update({"mixer." + n: p + "mix." + n for n in names})
        parts = {"mixer": mixer, "mixer_norm": before, "mixer_out_norm": after}
        if mlp is not None:
            weights.update({"ffn_norm.weight": p + "norm2", "ffn_out_norm.weight": p + "norm2b"})
            parts.update(ffn_norm=before, ffn_out_norm=after)
            if isinstance(mlp, GatedDenseConfig):
                parts["ffn"] = PartSpec("gated", {"hidden_size": d, "intermediate_size": mlp.ff, "activation": "gelu_tanh"})
                weights.update({"ffn.gate_proj.weight": p + "mlp.gate", "ffn.up_proj.weight": p + "mlp.up",
                                "ffn.down_proj.weight": p + "mlp.down"})
            else:
                assert isinstance(mlp, ClampedMoeConfig)
                parts["ffn"] = PartSpec("routed_experts", {
                    "hidden_size": d, "experts": mlp.experts, "top": mlp.top, "expert_size": mlp.expert_ff,
                    "shared_size": mlp.shared_ff, "shared_gate": False, "activation": "clamped_swish",
                    "limit": mlp.expert_limit, "shared_limit": mlp.shared_limit, "router_softmax": "all",
                    "router_scale": mlp.router_scale})
                names = ["router"] + [f"e{e}.{n}" for e in range(mlp.experts) for n in ("gate", "up", "down")]
                if mlp.shared_ff is not None:
                    names += ["shared.gate", "shared.up", "shared.down"]
                weights.update({"ffn." + n: p + "mlp." + n for n in names})
        layers.append(LayerSpec(parts=parts, weights=weights, arrangement="sandwich_residual"))
        run_order.append(RunEntry(layer=i, cache=i, writes_cache=True))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=d,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": cfg.embedding_scale}),
        layers=layers, run_order=run_order,
        final_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.eps}),
        lm_head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": d, "tied": True,
                                         "shares": "embedding.weight"}),
        weights={"embedding.weight": "embed", "final_norm.weight": "final.norm", "lm_head.weight": "embed"},
        # a checkpoint may carry the blending scalar of a layer that does not blend, and the feed-forward's norms of
        # a layer without feed-forward: nothing reads them
        ignored_weight_patterns=[r"l\d+\.mix\.vmix", r"l\d+\.norm2b?"],
    )


register_architecture("Timopel", TimopelConfig.from_hf_dict, build_timopel_spec)
