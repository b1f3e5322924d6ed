"""Typed configuration of the Timopel decoder, read from config.json's own keys.

config.json gives `vocab`, `width`, `norm.eps`, `residual_mult`, `embedding.scale` and `layers`, a
list whose entries name the layer's mixer (`type`: "attention"), the mixer's sizes and constants
(`mixer`: heads, kv_heads, dim, vdim, scale, q_temp {coef, every}, v_mix) and its feed-forward
(`mlp`: null, {"kind": "dense", "ff"} or {"kind": "moe", "router": {"experts", "top", "scale"},
"expert": {"ff", "limit"}, "shared": {"ff", "limit"} or absent}).  Layers differ from each other;
nothing about them stands in code.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple, Union

from .llama import ConfigError
from .zozosun import _need


@dataclass(frozen=True)
class QueryTemperature:
    """Queries at position p are multiplied by 1 + coef * ln(floor((p + 1) / every) + 1)."""

    coef: float
    every: int

    def to_dict(self) -> Dict[str, Any]:
        return {"coef": self.coef, "every": self.every}


@dataclass(frozen=True)
class SinkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp: Optional[QueryTemperature]
    v_mix: bool

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "SinkAttentionConfig":
        _need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
        qt = m.get("q_temp")
        if qt is not None:
            _need(qt, ("coef", "every"), where + ".q_temp")
            qt = QueryTemperature(float(qt["coef"]), int(qt["every"]))
            if qt.every <= 0:
                raise ConfigError(f"{where}.q_temp.every must be positive")
        c = SinkAttentionConfig(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                                qt, bool(m.get("v_mix", False)))
        if min(c.heads, c.kv_heads, c.dim, c.vdim) <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"{where}: sizes must be positive and heads a multiple of kv_heads")
        return c

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads}
        if self.q_temp is not None:
            d["q_temp"] = self.q_temp.to_dict()
        d.update(scale=self.scale, v_mix=self.v_mix, vdim=self.vdim)
        return d


@dataclass(frozen=True)
class GatedDenseConfig:
    ff: int

    def to_dict(self) -> Dict[str, Any]:
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class ClampedMoeConfig:
    experts: int
    top: int
    router_scale: float
    expert_ff: int
    expert_limit: float
    shared_ff: Optional[int] = None
    shared_limit: Optional[float] = None

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"expert": {"ff": self.expert_ff, "limit": self.expert_limit}, "kind": "moe",
                             "router": {"experts": self.experts, "scale": self.router_scale, "top": self.top}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return d


def _mlp_from_dict(mlp: Optional[Dict[str, Any]], where: str):
    if mlp is None:
        return None
    kind = mlp.get("kind")
    if kind == "dense":
        _need(mlp, ("ff",), where)
        if int(mlp["ff"]) <= 0:
            raise ConfigError(f"{where}.ff must be positive")
        return GatedDenseConfig(int(mlp["ff"]))
    if kind == "moe":
        _need(mlp, ("router", "expert"), where)
        _need(mlp["router"], ("experts", "top"), where + ".router")
        _need(mlp["expert"], ("ff", "limit"), where + ".expert")
        shared = mlp.get("shared")
        if shared:
            _need(shared, ("ff", "limit"), where + ".shared")
        c = ClampedMoeConfig(int(mlp["router"]["experts"]), int(mlp["router"]["top"]),
                             float(mlp["router"].get("scale", 1.0)), int(mlp["expert"]["ff"]),
                             float(mlp["expert"]["limit"]), None if not shared else int(shared["ff"]),
                             None if not shared else float(shared["limit"]))
        if not 0 < c.top <= c.experts or c.expert_ff <= 0 or (c.shared_ff is not None and c.shared_ff <= 0):
            raise ConfigError(f"{where}: 0 < top <= experts and positive widths are needed")
        if c.expert_limit <= 0 or (c.shared_limit is not None and c.shared_limit <= 0):
            raise ConfigError(f"{where}: the experts' limits must be positive")
        return c
    raise ConfigError(f"{where}.kind={kind!r} is not supported (known: 'dense', 'moe')")


@dataclass(frozen=True)
class TimopelLayerConfig:
    mixer: SinkAttentionConfig
    mlp: Union[None, GatedDenseConfig, ClampedMoeConfig]

    type = "attention"

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class TimopelConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    embedding_scale: float
    layers: Tuple[TimopelLayerConfig, ...]

    architecture = "Timopel"

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @staticmethod
    def from_hf_dict(d: Dict[str, Any]) -> "TimopelConfig":
        _need(d, ("vocab", "width", "norm", "layers", "residual_mult", "embedding"), "config.json")
        _need(d["norm"], ("eps",), "config.json norm")
        _need(d["embedding"], ("scale",), "config.json embedding")
        layers: List[TimopelLayerConfig] = []
        for i, layer in enumerate(d["layers"]):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            if layer["type"] != "attention":
                raise ConfigError(f"{where}.type={layer['type']!r} is not supported (known: 'attention')")
            layers.append(TimopelLayerConfig(SinkAttentionConfig.from_dict(layer["mixer"], where + ".mixer"),
                                             _mlp_from_dict(layer.get("mlp"), where + ".mlp")))
        cfg = TimopelConfig(int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), float(d["residual_mult"]),
                            float(d["embedding"]["scale"]), tuple(layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.eps <= 0 or not self.layers:
            raise ConfigError("vocab, width and norm.eps must be positive, and there must be layers")
        blend = [l.mixer for l in self.layers if l.mixer.v_mix]
        for m in blend[1:]:
            if (m.kv_heads, m.vdim) != (blend[0].kv_heads, blend[0].vdim):
                raise ConfigError("layers that blend their values with the first such layer's need its kv_heads and vdim")

    def to_hf_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.eps},
                "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
