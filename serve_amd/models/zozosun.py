"""`Zozosun`: a decoder whose layers are listed one by one in config.json, as a `ModelSpec`.

A layer is x <- x + ls1 * N1(mixer(x)); x <- x + ls2 * N2(ff(x)): the norm sits on the sublayer's
output, its weight is stored around zero (applied as 1 + w), and a layer scale multiplies the normed
output.  The mixer is a gated delta rule ("delta") or a latent attention with a sliding window
("latent_attention"), which may read an earlier layer's cache (`kv_from`); the feed-forward is
absent, dense (gelu, tanh form) or a mixture of experts with an optional gated shared expert.  The
model ends with the same kind of norm (`final.norm`) and the output matrix `head`.

Tensor names: `embed`, `l<i>.norm1|norm2|ls1|ls2`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`, `head`.
"""
from __future__ import annotations

from typing import Dict

from ..config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..config.zozosun import DeltaMixerConfig, DenseMlpConfig, LatentMixerConfig, MoeMlpConfig, ZozosunConfig
from ..registry import register_architecture


def build_zozosun_spec(cfg: ZozosunConfig) -> ModelSpec:
    d = cfg.width
    layers, run_order = [], []
    cache_of: Dict[int, int] = {}          # layer that keeps a cache or state -> its cache layer
    # how many keys a latent cache must keep: the longest window among the layers that read it
    retain: Dict[int, object] = {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, LatentMixerConfig):
            owner = i if m.kv_from is None else m.kv_from
            if owner not in retain:
                retain[owner] = m.window
            elif retain[owner] is not None:
                retain[owner] = None if m.window is None else max(retain[owner], m.window)
    for i, layer in enumerate(cfg.layers):
        p, m, mlp = f"l{i}.", layer.mixer, layer.mlp
        norm = PartSpec("scaled_output_rmsnorm", {"size": d, "eps": cfg.eps, "offset": 1.0})
        weights = {"mixer_norm.weight": p + "norm1", "mixer_norm.scale": p + "ls1"}
        if isinstance(m, DeltaMixerConfig):
            mixer = PartSpec("gated_delta", {"hidden_size": d, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                                             "vdim": m.vdim, "conv": m.conv, "eps": cfg.eps})
            names = ["q", "q.conv", "k", "k.conv", "v", "v.conv", "b", "a", "A_log", "dt_bias", "norm", "g", "o"]
            owner = i
        else:
            own = m.kv_from is None
            owner = i if own else m.kv_from
            mixer = PartSpec("latent_attention", {
                "hidden_size": d, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim,
                "kv_rank": m.kv_rank, "scale": m.scale, "eps": cfg.eps, "window": m.window,
                "retain": retain[owner] if own else None, "own_kv": own,
                "position": PartSpec("rope", {"head_dim": m.rot_dim, "rot_dim": m.rot_dim, "theta": m.rot_base,
                                              "scaling": None, "pairing": "half"})})
            names = ["q"] + (["dkv", "dkv.norm"] if own else []) + ["uk", "uv", "o"]
        weights.update({"mixer." + n: p + "mix." + n for n in names})
        parts = {"mixer": mixer, "mixer_norm": norm}
        if mlp is not None:
            weights.update({"ffn_norm.weight": p + "norm2", "ffn_norm.scale": p + "ls2"})
            parts["ffn_norm"] = norm
            if isinstance(mlp, DenseMlpConfig):
                parts["ffn"] = PartSpec("dense", {"hidden_size": d, "intermediate_size": mlp.ff, "activation": "gelu_tanh"})
                names = ["up", "down"]
            else:
                assert isinstance(mlp, MoeMlpConfig)
                parts["ffn"] = PartSpec("routed_experts", {"hidden_size": d, "experts": mlp.experts, "top": mlp.top,
                                                           "expert_size": mlp.expert_ff, "shared_size": mlp.shared_ff,
                                                           "shared_gate": True})
                names = ["router"] + [f"e{e}.{n}" for e in range(mlp.experts) for n in ("gate", "up", "down")]
                if mlp.shared_ff is not None:
                    names += ["shared.gate", "shared.up", "shared.down", "shared.sg"]
            weights.update({"ffn." + n: p + "mlp." + n for n in names})
        layers.append(LayerSpec(parts=parts, weights=weights, arrangement="postnorm_residual"))
        if owner == i:
            cache_of[i] = len(cache_of)
        run_order.append(RunEntry(layer=i, cache=cache_of[owner], writes_cache=owner == i))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=d,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": d}),
        layers=layers, run_order=run_order,
        final_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.eps, "offset": 1.0}),
        lm_head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": d, "tied": False, "shares": None}),
        weights={"embedding.weight": "embed", "final_norm.weight": "final.norm", "lm_head.weight": "head"},
    )


register_architecture("Zozosun", ZozosunConfig.from_hf_dict, build_zozosun_spec)
