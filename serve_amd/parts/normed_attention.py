"""Grouped-query attention without a rotation, whose queries and keys are normed per head:

    q = N(W_q h) * w_qn * temp(p),   k = N(W_k h) * w_kn,   v = W_v h        N(y) = y / sqrt(mean(y^2) + eps)
    temp(p) = 1 + coef * ln(floor((p + 1) / every) + 1)      (the "query temperature"; optional)
    weights = exp(q . k * scale) / (sum over seen keys + exp(sink_h))          (the "sink"; optional)

Positions enter through the causal mask and the temperature alone.  Keys have `dim` dims, values
`vdim`: the cache and the attention kernels work on one padded head size (the places behind are zeros),
so the framework's paged attention kernels run unchanged, with the sink as one more argument.

Value blending across layers (`v_blend`): the layer that is the "source" leaves its values of the step's
tokens on the step's context; a layer that is set to "blend" stores and attends over
(1 - lambda) v + lambda v_source, lambda being its own stored scalar.  Which layer is which is the
model builder's business.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops, trace
from ..registry import register_part
from .base import LayerCache, ParamRequest, Part, Runtime, StepCost, TokenCacheRequest, kv_cache_request
from .linear import linear
from .standard import _prepare_products

V_BLEND = ("none", "source", "blend")
SHARED_VALUES = "first_values"          # the name under which the source layer's values travel on the step's context


def padded_head_size(dim: int, vdim: int) -> int:
    """The head size of the cache: the larger of the two, up to a multiple of 16."""
    return -(-max(dim, vdim) // 16) * 16


class QKNormAttention(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, scale: float,
                 eps: float, q_temp_coef: float = 0.0, q_temp_every: int = 0, sink: bool = False,
                 v_blend: str = "none", window: Optional[int] = None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if v_blend not in V_BLEND:
            raise ValueError(f"v_blend must be one of {V_BLEND}")
        if q_temp_every < 0:
            raise ValueError("q_temp_every must not be negative (0: no query temperature)")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.scale, self.eps = int(dim), int(vdim), float(scale), float(eps)
        self.q_temp_coef, self.q_temp_every = float(q_temp_coef), int(q_temp_every)
        self.sink, self.v_blend, self.window = bool(sink), v_blend, window
        self.head_size = padded_head_size(self.dim, self.vdim)
        if self.head_size > ops.SIMPLE_ATTENTION_MAX_HEAD_DIM:
            raise ValueError(f"head sizes up to {ops.SIMPLE_ATTENTION_MAX_HEAD_DIM} are taken, got {self.head_size}")

    def param_requests(self) -> List[ParamRequest]:
        d, H, G, D, Dv = self.hidden_size, self.num_heads, self.num_kv_heads, self.dim, self.vdim
        out = [ParamRequest("q", (H * D, d), init="normal:0.08"), ParamRequest("k", (G * D, d), init="normal:0.08"),
               ParamRequest("v", (G * Dv, d), init="normal:0.08"),
               ParamRequest("q.norm", (D,), init="ones_normal:0.2"), ParamRequest("k.norm", (D,), init="ones_normal:0.2")]
        if self.v_blend != "none":
            # (read by the blending layers only: the source layer's may be missing)
            out.append(ParamRequest("vmix", (), init="uniform:0.2:0.6", optional=self.v_blend == "source"))
        if self.sink:
            out.append(ParamRequest("sink", (H,), init="normal:1.0"))
        return out + [ParamRequest("o", (d, H * Dv), init="normal:0.08")]

    def cache_request(self) -> TokenCacheRequest:
        return kv_cache_request(self.num_kv_heads, self.head_size, self.window)

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        """The four projections, and scores (dim) and weighted values (vdim) over the keys each token sees."""
        cost = super().step_cost(tokens, context_before)
        if self.window:
            keys = sum(min(context_before + j + 1, self.window) for j in range(tokens))
        else:
            keys = tokens * context_before + tokens * (tokens + 1) // 2
        cost.flops += 2.0 * self.num_heads * (self.dim + self.vdim) * keys
        return cost

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        H, Dv, Dp = self.num_heads, self.vdim, self.head_size
        parts = [tensors["q"], tensors["k"], tensors["v"]]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        self.wqkv = torch.cat([p.to(dt) for p in parts], dim=0).contiguous()         # one product for q, k and v
        wo = tensors["o"]
        if Dp != Dv:
            # the attention's output rows hold Dp places a head, of which the last Dp - Dv are zeros
            padded = torch.zeros((self.hidden_size, H, Dp), dtype=wo.dtype, device=wo.device)
            padded[:, :, :Dv] = wo.view(self.hidden_size, H, Dv)
            wo = padded.view(self.hidden_size, H * Dp)
        self.wo = wo.contiguous()
        self.q_norm = tensors["q.norm"].float().contiguous()
        self.k_norm = tensors["k.norm"].float().contiguous()
        self.sinks = tensors["sink"].float().contiguous() if self.sink else None
        self.blend = float(tensors["vmix"].float()) if self.v_blend == "blend" else 0.0
        _prepare_products(rt, self.wqkv)

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        H, G, D, Dv, Dp = self.num_heads, self.num_kv_heads, self.dim, self.vdim, self.head_size
        T = h.shape[0]
        grp = ctx.groups[cache.group]
        if cache.k_pages.shape[-1] != Dp:
            raise ValueError(f"the cache keeps heads of {cache.k_pages.shape[-1]}, this layer works on {Dp}")
        with trace.span("write_to_cache"):
            qkv = linear(h, self.wqkv)
            first = None
            if self.v_blend == "blend":
                first = ctx.shared.get(SHARED_VALUES)
                if first is None:
                    raise RuntimeError("a layer that blends its values ran before the layer whose values it blends with")
            q = self.rt.empty((T, H * Dp))
            ops.qk_norm_kv_write(qkv, q, ctx.positions, grp.slots if writes_cache else None, cache.k_pages,
                                 cache.v_pages, self.q_norm, self.k_norm, self.eps, H, G, D, Dv, self.q_temp_coef,
                                 self.q_temp_every, first, self.blend)
            if self.v_blend == "source":
                ctx.shared[SHARED_VALUES] = qkv[:, (H + G) * D:]         # (a view: the rows stay alive with it)
        attn = self.rt.empty((T, H * Dp))
        with trace.span("attention"):
            ops.paged_attention(q, H * Dp, attn, cache.k_pages, cache.v_pages, grp.block_table, ctx, H, self.scale,
                                self.window, self.sinks)
        return linear(attn, self.wo, partial_ok=True)      # the following norm adds the parts


register_part("mixer", "qk_norm_attention", QKNormAttention)
