"""Typed configuration of the Zozosun decoder, read from config.json's own keys.

config.json gives `vocab`, `width`, `norm.eps` and `layers`, a list whose entries name the layer's
mixer (`type`: "delta" or "latent_attention"), the mixer's sizes and constants (`mixer`) and its
feed-forward (`mlp`: null, {"kind": "dense", "ff"} or {"kind": "moe", "router": {"experts", "top"},
"expert": {"ff"}, "shared": {"ff"} or absent}).  Layers differ from each other; nothing about them
stands in code.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple, Union

from .llama import ConfigError


def _need(d: Dict[str, Any], keys, where: str) -> None:
    missing = [k for k in keys if k not in d]
    if missing:
        raise ConfigError(f"{where} lacks the keys {missing}")


@dataclass(frozen=True)
class DeltaMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "DeltaMixerConfig":
        _need(m, ("heads", "kv_heads", "dim", "vdim", "conv"), where)
        c = DeltaMixerConfig(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), int(m["conv"]))
        if min(c.heads, c.kv_heads, c.dim, c.vdim, c.conv) <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"{where}: sizes must be positive and heads a multiple of kv_heads")
        return c

    def to_dict(self) -> Dict[str, Any]:
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    window: Optional[int]
    kv_from: Optional[int] = None

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "LatentMixerConfig":
        _need(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"), where)
        rot = m["rot"]
        _need(rot, ("base", "dims"), where + ".rot")
        if int(rot["dims"]) != int(m["rot_dim"]):
            raise ConfigError(f"{where}: rot.dims {rot['dims']} must equal rot_dim {m['rot_dim']} (the whole shared "
                              "key part is rotated)")
        mask = m.get("mask")
        window = None if not mask else int(mask["size"])
        kv_from = m.get("kv_from")
        c = LatentMixerConfig(int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]),
                              float(m["scale"]), float(rot["base"]), window, None if kv_from is None else int(kv_from))
        if min(c.heads, c.dim, c.vdim, c.kv_rank) <= 0 or c.rot_dim < 0 or c.rot_dim % 2:
            raise ConfigError(f"{where}: sizes must be positive and rot_dim even")
        if c.scale <= 0 or c.rot_base <= 0 or (c.window is not None and c.window <= 0):
            raise ConfigError(f"{where}: scale, rot.base and mask.size must be positive")
        return c

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        d.update(kv_rank=self.kv_rank)
        if self.window is not None:
            d["mask"] = {"size": self.window}
        d.update(rot={"base": self.rot_base, "dims": self.rot_dim}, rot_dim=self.rot_dim, scale=self.scale, vdim=self.vdim)
        return d


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int

    def to_dict(self) -> Dict[str, Any]:
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class MoeMlpConfig:
    experts: int
    top: int
    expert_ff: int
    shared_ff: Optional[int] = None

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"expert": {"ff": self.expert_ff}, "kind": "moe",
                             "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


def _mlp_from_dict(mlp: Optional[Dict[str, Any]], where: str):
    if mlp is None:
        return None
    kind = mlp.get("kind")
    if kind == "dense":
        _need(mlp, ("ff",), where)
        if int(mlp["ff"]) <= 0:
            raise ConfigError(f"{where}.ff must be positive")
        return DenseMlpConfig(int(mlp["ff"]))
    if kind == "moe":
        _need(mlp, ("router", "expert"), where)
        _need(mlp["router"], ("experts", "top"), where + ".router")
        _need(mlp["expert"], ("ff",), where + ".expert")
        shared = mlp.get("shared")
        c = MoeMlpConfig(int(mlp["router"]["experts"]), int(mlp["router"]["top"]), int(mlp["expert"]["ff"]),
                         None if not shared else int(shared["ff"]))
        if not 0 < c.top <= c.experts or c.expert_ff <= 0 or (c.shared_ff is not None and c.shared_ff <= 0):
            raise ConfigError(f"{where}: 0 < top <= experts and positive widths are needed")
        return c
    raise ConfigError(f"{where}.kind={kind!r} is not supported (known: 'dense', 'moe')")


@dataclass(frozen=True)
class ZozosunLayerConfig:
    mixer: Union[DeltaMixerConfig, LatentMixerConfig]
    mlp: Union[None, DenseMlpConfig, MoeMlpConfig]

    @property
    def type(self) -> str:
        return "delta" if isinstance(self.mixer, DeltaMixerConfig) else "latent_attention"

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class ZozosunConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[ZozosunLayerConfig, ...]

    architecture = "Zozosun"

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @staticmethod
    def from_hf_dict(d: Dict[str, Any]) -> "ZozosunConfig":
        _need(d, ("vocab", "width", "norm", "layers"), "config.json")
        _need(d["norm"], ("eps",), "config.json norm")
        layers: List[ZozosunLayerConfig] = []
        for i, layer in enumerate(d["layers"]):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            if layer["type"] == "delta":
                mixer = DeltaMixerConfig.from_dict(layer["mixer"], where + ".mixer")
            elif layer["type"] == "latent_attention":
                mixer = LatentMixerConfig.from_dict(layer["mixer"], where + ".mixer")
            else:
                raise ConfigError(f"{where}.type={layer['type']!r} is not supported (known: 'delta', 'latent_attention')")
            layers.append(ZozosunLayerConfig(mixer, _mlp_from_dict(layer.get("mlp"), where + ".mlp")))
        cfg = ZozosunConfig(int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), tuple(layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.eps <= 0 or not self.layers:
            raise ConfigError("vocab, width and norm.eps must be positive, and there must be layers")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if isinstance(m, LatentMixerConfig) and m.kv_from is not None:
                j = m.kv_from
                if not 0 <= j < i or not isinstance(self.layers[j].mixer, LatentMixerConfig):
                    raise ConfigError(f"layers[{i}].mixer.kv_from={j} must name an earlier latent-attention layer")
                src = self.layers[j].mixer
                if src.kv_from is not None:
                    raise ConfigError(f"layers[{i}].mixer.kv_from={j}: that layer keeps no cache of its own")
                if (src.kv_rank, src.rot_dim, src.rot_base) != (m.kv_rank, m.rot_dim, m.rot_base):
                    raise ConfigError(f"layers[{i}] reads the cache of layer {j}: kv_rank, rot_dim and rot.base must be equal")

    def to_hf_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                "norm": {"eps": self.eps}, "vocab": self.vocab, "width": self.width}
