"""Plain, slow, cache-free implementation of the Timopel decoder.

One function per mechanism, written from the design's equations, whole sequences on the CPU,
in the dtype it is given (float64 as the oracle).  It shares no code with the `serve_amd`
package: the tests compare the engine with it.

Notation.  h [T, d] is a sublayer's input, W["<name>"] a checkpoint tensor stored [out, in].
With a constant c (`residual_mult`) and N_w(y) = y / sqrt(mean(y^2) + eps) * w a layer is

    x <- x + c * N_1b(mixer(N_1(x)));   x <- x + c * N_2b(ff(N_2(x)))      (the second half only with a feed-forward)

so every sublayer has a norm in front of it and one behind it.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

Tensor = torch.Tensor


# --------------------------------------------------------------------------------------
# elementwise pieces
# --------------------------------------------------------------------------------------
def rms_norm(y: Tensor, w: Tensor, eps: float) -> Tensor:
    """y / sqrt(mean(y^2) + eps) * w over the last axis, eps inside the root, plain weight."""
    return y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z: Tensor) -> Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def clamped_swish_gate(g: Tensor, u: Tensor, limit: float) -> Tensor:
    """The experts' activation: the gate is cut from above, the other branch from both sides and
    shifted by one:  min(g, L) * sigmoid(1.702 min(g, L)) * (clamp(u, -L, L) + 1)."""
    g = g.clamp(max=limit)
    u = u.clamp(min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


# --------------------------------------------------------------------------------------
# mixer 'attention'
# --------------------------------------------------------------------------------------
def query_temperature(positions: Tensor, coef: float, every: int) -> Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1) per position p: 1 for the first every - 1 positions,
    then growing in steps."""
    steps = torch.div(positions + 1, every, rounding_mode="floor")
    return 1.0 + coef * torch.log(steps.to(torch.float64) + 1.0)


def sink_softmax(scores: Tensor, sink: Tensor) -> Tensor:
    """Weights over the keys (last axis) when the denominator also holds exp(sink): the weights of a
    row sum to less than one.  scores [..., keys] with -inf where a key is not seen; sink broadcasts
    against scores[..., 0]."""
    m = torch.maximum(scores.max(-1).values, sink)
    e = torch.exp(scores - m[..., None])
    return e / (e.sum(-1) + torch.exp(sink - m))[..., None]


def attention(h: Tensor, W: Dict[str, Tensor], mixer: dict, eps: float, v_first: Optional[Tensor],
              mixes: bool) -> (Tensor, Tensor):
    """The whole mixer over one sequence from position 0.  Returns (output [T, d], the values that
    were used [T, G, vdim]).  `mixes`: blend the values with `v_first` (the values of the first layer
    that takes part in the blending) by the layer's scalar `vmix`."""
    T = h.shape[0]
    H, G, D, Dv = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    q = (h @ W["q"].T).view(T, H, D)
    k = (h @ W["k"].T).view(T, G, D)
    v = (h @ W["v"].T).view(T, G, Dv)
    q = rms_norm(q, W["q.norm"], eps)
    k = rms_norm(k, W["k.norm"], eps)
    qt = mixer.get("q_temp")
    if qt:
        q = q * query_temperature(torch.arange(T), float(qt["coef"]), int(qt["every"])).to(q.dtype)[:, None, None]
    if mixes:
        lam = W["vmix"].to(v.dtype)
        v = (1.0 - lam) * v + lam * v_first
    seen = torch.ones(T, T, dtype=torch.bool).tril()
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(mixer["scale"])
        s = s.masked_fill(~seen, -math.inf)
        p = sink_softmax(s, W["sink"][head].to(s.dtype))
        out[:, head] = p @ v[:, g]
    return out.reshape(T, H * Dv) @ W["o"].T, v


# --------------------------------------------------------------------------------------
# feed-forwards
# --------------------------------------------------------------------------------------
def dense_ff(h: Tensor, W: Dict[str, Tensor]) -> Tensor:
    return (gelu_tanh(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


def expert_ff(h: Tensor, W: Dict[str, Tensor], prefix: str, limit: float) -> Tensor:
    a = clamped_swish_gate(h @ W[prefix + "gate"].T, h @ W[prefix + "up"].T, limit)
    return a @ W[prefix + "down"].T


def route(z: Tensor, top: int, scale: float) -> (Tensor, Tensor):
    """z [T, E] router logits -> (ids [T, top], weights [T, top]): softmax over all experts, the `top`
    largest, their scores over their sum (+ 1e-20), times `scale`.  Ties go to the lower index."""
    s = torch.softmax(z, dim=-1)
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top]
    chosen = torch.gather(s, 1, order)
    return order, chosen / (chosen.sum(-1, keepdim=True) + 1e-20) * scale


def moe_ff(h: Tensor, W: Dict[str, Tensor], mlp: dict, margins: Optional[list] = None) -> Tensor:
    """`margins` (a list) receives per token (position, lead of the last chosen logit over the first that is
    left out, as a share of the logits' spread): how clear the router's choice is."""
    r = mlp["router"]
    z = h @ W["router"].T
    ids, wts = route(z, int(r["top"]), float(r["scale"]))
    if margins is not None and int(r["top"]) < z.shape[1]:
        v = torch.sort(z, dim=-1, descending=True).values
        lead = (v[:, int(r["top"]) - 1] - v[:, int(r["top"])]) / (v[:, 0] - v[:, -1]).clamp_min(1e-30)
        margins.extend((t, float(m)) for t, m in enumerate(lead))
    out = torch.zeros_like(h)
    limit = float(mlp["expert"]["limit"])
    for e in range(z.shape[1]):
        took = ids == e                                   # [T, top]: which tokens chose expert e, and at which place
        rows = took.any(-1)
        if rows.any():
            out[rows] += (wts * took).sum(-1, keepdim=True)[rows] * expert_ff(h[rows], W, f"e{e}.", limit)
    if mlp.get("shared"):
        out = out + expert_ff(h, W, "shared.", float(mlp["shared"]["limit"]))
    return out


# --------------------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------------------
def _sub(W: Dict[str, Tensor], prefix: str) -> Dict[str, Tensor]:
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def forward(tokens: Sequence[int], weights: Dict[str, Tensor], cfg: dict, dtype=torch.float64,
            return_layers: bool = False, margins: Optional[list] = None):
    """Logits [T, vocab] of one sequence from position 0 (and the stream after every layer).  `margins`: see moe_ff."""
    W = {k: v.to(dtype) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    c = float(cfg["residual_mult"])
    x = W["embed"][torch.tensor(list(tokens))] * float(cfg["embedding"]["scale"])
    v_first = None
    streams: List[Tensor] = []
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "attention":
            raise ValueError(f"layer {i}: unknown mixer {layer['type']!r}")
        L = _sub(W, f"l{i}.")
        mixer = layer["mixer"]
        takes_part = bool(mixer.get("v_mix"))
        y, v = attention(rms_norm(x, L["norm1"], eps), _sub(L, "mix."), mixer, eps, v_first,
                         takes_part and v_first is not None)
        if takes_part and v_first is None:
            v_first = v
        x = x + c * rms_norm(y, L["norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, L["norm2"], eps)
            M = _sub(L, "mlp.")
            if mlp["kind"] == "dense":
                y = dense_ff(h, M)
            elif mlp["kind"] == "moe":
                y = moe_ff(h, M, mlp, margins)
            else:
                raise ValueError(f"layer {i}: unknown feed-forward {mlp['kind']!r}")
            x = x + c * rms_norm(y, L["norm2b"], eps)
        streams.append(x)
    logits = rms_norm(x, W["final.norm"], eps) @ W["embed"].T
    return (logits, torch.stack(streams)) if return_layers else logits
