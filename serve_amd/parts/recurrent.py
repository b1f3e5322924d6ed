"""A recurrent mixer: the gated delta rule.

Per head, with a state matrix S [dim, vdim] per request (fp32, zero at admission):

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

q and k (kv_heads x dim) and v (heads x vdim) are projections of the layer's input that pass a
short causal convolution over time (one filter per channel, `conv` taps, the last on the current
token, zeros before the start) and silu; q and k are then unit vectors per head (x / sqrt(sum x^2 +
1e-6)), q also times dim^-1/2; beta = sigmoid(W_b h); g = exp(-exp(A_log) softplus(W_a h + dt_bias)),
one per head.  Head i reads q/k head i // (heads / kv_heads).  The read-out is divided by its root
mean square over vdim, times a weight shared by the heads, times silu(W_g h), then projected back.

State per request: S of every head and the convolution's last conv - 1 inputs, one fp32 row.
"""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from ..registry import register_part
from .base import LayerCache, ParamRequest, Part, Runtime, StateRequest, StepCost
from .linear import linear
from .standard import _prepare_products


class GatedDeltaMixer(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, conv: int, eps: float):
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if not (0 < dim <= ops.DELTA_MAX_DIM and 0 < vdim <= ops.DELTA_MAX_DIM and 1 <= conv <= ops.DELTA_MAX_TAPS):
            raise ValueError(f"the delta rule's kernels take head sizes up to {ops.DELTA_MAX_DIM} and up to "
                             f"{ops.DELTA_MAX_TAPS} taps; got dim {dim}, vdim {vdim}, conv {conv}")
        self.hidden_size, self.heads, self.kv_heads = int(hidden_size), int(heads), int(kv_heads)
        self.dim, self.vdim, self.taps, self.eps = int(dim), int(vdim), int(conv), float(eps)
        self.channels = 2 * self.kv_heads * self.dim + self.heads * self.vdim      # what the convolution sees

    def param_requests(self) -> List[ParamRequest]:
        d, H, Hk, dk, dv, taps = self.hidden_size, self.heads, self.kv_heads, self.dim, self.vdim, self.taps
        return [ParamRequest("q", (Hk * dk, d), init="normal:0.06"), ParamRequest("q.conv", (Hk * dk, taps), init="normal:0.6"),
                ParamRequest("k", (Hk * dk, d), init="normal:0.06"), ParamRequest("k.conv", (Hk * dk, taps), init="normal:0.6"),
                ParamRequest("v", (H * dv, d), init="normal:0.06"), ParamRequest("v.conv", (H * dv, taps), init="normal:0.6"),
                ParamRequest("b", (H, d), init="normal:0.06"), ParamRequest("a", (H, d), init="normal:0.06"),
                ParamRequest("A_log", (H,), init="uniform:-4:0"), ParamRequest("dt_bias", (H,), init="uniform:-3.5:-1.5"),
                ParamRequest("norm", (dv,), init="ones_normal:0.15"), ParamRequest("g", (H * dv, d), init="normal:0.09"),
                ParamRequest("o", (d, H * dv), init="normal:0.07")]

    def state_request(self) -> StateRequest:
        return StateRequest((self.heads * self.dim * self.vdim + (self.taps - 1) * self.channels,), torch.float32)

    def step_cost(self, tokens: int, context_before: int = 0) -> StepCost:
        """The projections, and per token and head three passes over S (decay and S^T k, the rank-one
        update, S^T q): 6 dim vdim flops."""
        cost = super().step_cost(tokens, context_before)
        cost.flops += 6.0 * tokens * self.heads * self.dim * self.vdim
        return cost

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        big = [tensors[n] for n in ("q", "k", "v", "g")]
        dt = big[0].dtype if all(t.dtype == big[0].dtype for t in big) else torch.float32
        self.w_in = torch.cat([t.to(dt) for t in big], dim=0).contiguous()        # one product: q | k | v | gate
        small = [tensors["b"], tensors["a"]]
        self.w_ba = torch.cat([t.to(dt) for t in small], dim=0).contiguous()      # beta's and the decay's logits
        self.conv_w = torch.cat([tensors[n].float() for n in ("q.conv", "k.conv", "v.conv")], dim=0).contiguous()
        self.A_log = tensors["A_log"].float().contiguous()
        self.dt_bias = tensors["dt_bias"].float().contiguous()
        self.norm_w = tensors["norm"].float().contiguous()
        self.wo = tensors["o"]
        _prepare_products(rt, self.w_in)

    def forward(self, h: torch.Tensor, ctx, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        if cache.state is None:
            raise ValueError("the delta rule needs its per-request state")
        z = linear(h, self.w_in)
        ba = linear(h, self.w_ba, out_dtype=torch.float32)          # what enters the recurrence stays fp32
        y = self.rt.empty((h.shape[0], self.heads * self.vdim))
        ops.delta_rule(z, self.conv_w, ba, self.A_log, self.dt_bias, self.norm_w, cache.state, ctx, y, self.eps,
                       self.heads, self.kv_heads, self.dim, self.vdim, self.taps)
        return linear(y, self.wo, partial_ok=True)


register_part("mixer", "gated_delta", GatedDeltaMixer)
