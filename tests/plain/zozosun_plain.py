"""Plain, slow, cache-free implementation of the Zozosun decoder.

One function per mechanism, written from the design's equations, whole sequences on the CPU,
in the dtype it is given (float64 as the oracle).  It shares no code with the `serve_amd`
package: the tests compare the engine with it.

Notation.  h [T, d] is a sublayer's input, W["<name>"] a checkpoint tensor stored [out, in].
A layer is   x <- x + ls1 * N1(mixer(x));  x <- x + ls2 * N2(ff(x))   with
N(y) = y / sqrt(mean(y^2) + eps) * (1 + w): the norm sits on the sublayer's output and its weight
is stored around zero.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch

Tensor = torch.Tensor


# --------------------------------------------------------------------------------------
# elementwise pieces
# --------------------------------------------------------------------------------------
def rms(y: Tensor, eps: float) -> Tensor:
    """y / sqrt(mean(y^2) + eps) over the last axis, eps inside the root."""
    return y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps)


def norm_around_zero(y: Tensor, w: Tensor, eps: float) -> Tensor:
    """The layer's and the model's norm: weight stored as w, applied as 1 + w."""
    return rms(y, eps) * (1.0 + w)


def gelu_tanh(z: Tensor) -> Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: Tensor) -> Tensor:
    return z * torch.sigmoid(z)


def softplus(z: Tensor) -> Tensor:
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


# --------------------------------------------------------------------------------------
# mixer 'delta': gated delta rule
# --------------------------------------------------------------------------------------
def short_conv(x: Tensor, w: Tensor) -> Tensor:
    """Causal convolution over time, one filter per channel: x [T, C], w [C, taps]; the last
    column of w multiplies the current token, the one before it the previous token, and so on;
    before the start of the sequence there are zeros."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                out[t] += w[:, j] * x[s]
    return out


def unit_vectors(x: Tensor) -> Tensor:
    """x / sqrt(sum(x^2) + 1e-6) over the last axis."""
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)


def delta_recurrence(q: Tensor, k: Tensor, v: Tensor, beta: Tensor, g: Tensor) -> Tensor:
    """One head, token by token.  q, k [T, dk]; v [T, dv]; beta, g [T].
    S [dk, dv] starts at zero;  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, dk = q.shape
    dv = v.shape[1]
    S = torch.zeros(dk, dv, dtype=q.dtype)
    out = torch.zeros(T, dv, dtype=q.dtype)
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.t() @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.t() @ q[t]
    return out


def delta_mixer(h: Tensor, W: Dict[str, Tensor], p: str, m: dict, eps: float) -> Tensor:
    """h [T, d] -> [T, d].  p = '<layer>.mix.'; m = the layer's 'mixer' entry of config.json."""
    H, Hk, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(short_conv(h @ W[p + "q"].t(), W[p + "q.conv"])).view(T, Hk, dk)
    k = silu(short_conv(h @ W[p + "k"].t(), W[p + "k.conv"])).view(T, Hk, dk)
    v = silu(short_conv(h @ W[p + "v"].t(), W[p + "v.conv"])).view(T, H, dv)
    q = unit_vectors(q) * dk ** -0.5
    k = unit_vectors(k)
    beta = torch.sigmoid(h @ W[p + "b"].t())                                   # [T, H]
    g = torch.exp(-torch.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].t() + W[p + "dt_bias"]))
    gate = silu(h @ W[p + "g"].t()).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    rep = H // Hk
    for i in range(H):
        o = delta_recurrence(q[:, i // rep], k[:, i // rep], v[:, i], beta[:, i], g[:, i])
        out[:, i] = rms(o, eps) * W[p + "norm"] * gate[:, i]
    return out.reshape(T, H * dv) @ W[p + "o"].t()


# --------------------------------------------------------------------------------------
# mixer 'latent_attention'
# --------------------------------------------------------------------------------------
def rotate(x: Tensor, positions: Tensor, base: float) -> Tensor:
    """Rotary encoding of the whole last axis (size n): dimension i is paired with i + n/2;
    (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * base^(-2i/n)."""
    n = x.shape[-1]
    half = n // 2
    f = torch.tensor([base ** (-2.0 * i / n) for i in range(half)], dtype=x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :]                # [T, half]
    while a.dim() < x.dim():
        a = a.unsqueeze(1)
    u, v = x[..., :half], x[..., half:]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a)], dim=-1)


def latent_and_rotated_key(h: Tensor, W: Dict[str, Tensor], p: str, m: dict, eps: float) -> Tuple[Tensor, Tensor]:
    """What a latent-attention layer keeps per token: c [T, kv_rank] (normed, plain weight) and
    the one rotated key part [T, rot_dim] that all heads share."""
    r = m["kv_rank"]
    T = h.shape[0]
    z = h @ W[p + "dkv"].t()
    c = rms(z[:, :r], eps) * W[p + "dkv.norm"]
    kr = rotate(z[:, r:], torch.arange(T), m["rot"]["base"])
    return c, kr


def latent_attention(h: Tensor, W: Dict[str, Tensor], p: str, m: dict, c: Tensor, kr: Tensor) -> Tensor:
    """h [T, d] -> [T, d] given the latents c and rotated key parts kr of the same tokens (its own
    layer's, or those of the layer named by 'kv_from')."""
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].t()).view(T, H, dn + dr)
    qn, qr = q[..., :dn], rotate(q[..., dn:], torch.arange(T), m["rot"]["base"])
    kn = (c @ W[p + "uk"].t()).view(T, H, dn)
    val = (c @ W[p + "uv"].t()).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", qn, kn) + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = i - j >= 0
    if m.get("mask"):                                  # a sliding window: itself and the size - 1 tokens before it
        seen = seen & (i - j < m["mask"]["size"])
    scores = scores.masked_fill(~seen, float("-inf"))
    out = torch.einsum("hij,jhd->ihd", torch.softmax(scores, dim=-1), val)
    return out.reshape(T, H * dv) @ W[p + "o"].t()


# --------------------------------------------------------------------------------------
# feed-forward
# --------------------------------------------------------------------------------------
def dense_ff(h: Tensor, W: Dict[str, Tensor], p: str) -> Tensor:
    return gelu_tanh(h @ W[p + "up"].t()) @ W[p + "down"].t()


def gated_expert(h: Tensor, W: Dict[str, Tensor], p: str) -> Tensor:
    return (silu(h @ W[p + "gate"].t()) * (h @ W[p + "up"].t())) @ W[p + "down"].t()


def moe_ff(h: Tensor, W: Dict[str, Tensor], p: str, mlp: dict, margins: Optional[list] = None) -> Tensor:
    """Every token takes its `top` experts with the largest router logits, weighted by the softmax
    over those logits alone; a shared expert, if there is one, is added for every token, times
    sigmoid(W_sg h)."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ W[p + "router"].t()                                     # [T, E]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: -float(z[t, e]))
        chosen = order[:top]
        if margins is not None and top < E:
            # by how much the last chosen logit leads the first that is left out, in units of the logits' spread
            margins.append((t, float((z[t, order[top - 1]] - z[t, order[top]]) / z[t].std().clamp_min(1e-12))))
        w = torch.softmax(z[t, chosen], dim=0)
        for wi, e in zip(w, chosen):
            out[t] += wi * gated_expert(h[t:t + 1], W, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ W[p + "shared.sg"].t()) * gated_expert(h, W, p + "shared.")
    return out


# --------------------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------------------
def forward(tokens: Sequence[int], weights: Dict[str, Tensor], cfg: dict, dtype=torch.float64,
            return_layers: bool = False, margins: Optional[list] = None):
    """Logits [T, vocab] of one sequence (and, on request, the residual stream after every layer).
    `margins` receives (token, margin) of every routing decision: how clearly the experts were chosen."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(list(tokens), dtype=torch.long)]
    kept: Dict[int, Tuple[Tensor, Tensor]] = {}
    streams: List[Tensor] = []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        if layer["type"] == "delta":
            y = delta_mixer(x, W, p + "mix.", m, eps)
        elif layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = latent_and_rotated_key(x, W, p + "mix.", m, eps)
                src = i
            y = latent_attention(x, W, p + "mix.", m, *kept[src])
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        x = x + norm_around_zero(y, W[p + "norm1"], eps) * W[p + "ls1"]
        mlp = layer.get("mlp")
        if mlp is not None:
            y = dense_ff(x, W, p + "mlp.") if mlp["kind"] == "dense" else moe_ff(x, W, p + "mlp.", mlp, margins)
            x = x + norm_around_zero(y, W[p + "norm2"], eps) * W[p + "ls2"]
        streams.append(x)
    logits = norm_around_zero(x, W["final.norm"], eps) @ W["head"].t()
    return (logits, torch.stack(streams)) if return_layers else logits
