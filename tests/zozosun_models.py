"""Small Zozosun configurations for the tests, and helpers that compare the engine with the plain
implementation.  The configurations differ from each other in every size, in the order of their
layers and in which optional pieces they have; several values that a model may happen to make equal
(heads and kv_heads, dim and vdim, rot_dim and dim, top 1) are unequal in one and equal in another.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch

from serve_amd.config.zozosun import (DeltaMixerConfig, DenseMlpConfig, LatentMixerConfig, MoeMlpConfig,
                                      ZozosunConfig, ZozosunLayerConfig)
from serve_amd.weights.loader import write_random_model
from tests.plain import zozosun_plain


def _delta(heads, kv_heads, dim, vdim, conv):
    return DeltaMixerConfig(heads, kv_heads, dim, vdim, conv)


def _latent(heads, dim, rot_dim, vdim, rank, window, scale=0.2, base=10000.0, kv_from=None):
    return LatentMixerConfig(heads, dim, rot_dim, vdim, rank, scale, base, window, kv_from)


L = ZozosunLayerConfig

# mixed: both mixers, both feed-forwards, a layer without feed-forward, a layer that reads another's
# cache with a longer window than the layer that writes it
ZA = ZozosunConfig(vocab=200, width=64, eps=1e-5, layers=(
    L(_delta(4, 2, 16, 24, 3), DenseMlpConfig(96)),
    L(_latent(3, 16, 8, 24, 40, 20), MoeMlpConfig(6, 2, 32, 48)),
    L(_latent(2, 8, 8, 16, 40, 33, scale=0.3, kv_from=1), None),
    L(_delta(2, 2, 40, 16, 2), MoeMlpConfig(5, 1, 24, None)),
))

# cache rows wider than the matrix-core attention takes, head sizes of the delta rule above 64 in both
# directions, one kv head for six heads, a window shorter than a page, three of four experts
ZB = ZozosunConfig(vocab=333, width=96, eps=1e-6, layers=(
    L(_latent(5, 24, 16, 16, 150, 9, scale=0.15, base=500.0), DenseMlpConfig(80)),
    L(_delta(6, 1, 72, 80, 4), None),
    L(_latent(4, 12, 16, 20, 150, 5, scale=0.25, base=500.0, kv_from=0), MoeMlpConfig(4, 3, 40, 24)),
))

# the delta rule alone: no paged cache at all
ZD = ZozosunConfig(vocab=128, width=48, eps=1e-5, layers=(
    L(_delta(3, 3, 24, 24, 4), DenseMlpConfig(64)),
    L(_delta(2, 1, 32, 48, 1), None),
))

# latent attention alone, more heads than a matrix-core tile has rows, one layer that sees every key
ZL = ZozosunConfig(vocab=150, width=80, eps=1e-5, layers=(
    L(_latent(20, 8, 4, 8, 28, None, scale=0.35), None),
    L(_latent(2, 24, 16, 40, 56, 17, scale=0.2, base=300000.0), DenseMlpConfig(72)),
))

# sizes that no kernel's vector path takes: a width that is no multiple of 4, odd head sizes and widths of
# experts, a cache row of 290 (above the tiled attention kernels), one tap more than the others
ZO = ZozosunConfig(vocab=101, width=50, eps=1e-5, layers=(
    L(_delta(3, 1, 10, 7, 5), MoeMlpConfig(3, 2, 9, 5)),
    L(_latent(3, 6, 10, 5, 270, 11, scale=0.3), DenseMlpConfig(30)),
    L(_latent(1, 5, 10, 9, 270, 4, scale=0.3, kv_from=1), None),
))

MODELS = {"ZA": (ZA, 3), "ZB": (ZB, 4), "ZD": (ZD, 5), "ZL": (ZL, 6), "ZO": (ZO, 7)}

# queries and the keys' up-projections drawn wide: scores of order one, so that softmax picks keys and a
# window that is one token off, a wrong rotation or a wrong head shows in the logits
SHARP = {r"\.mix\.(q|uk)$": 3.0}
# the embedding and the output matrix at a scale at which the stream and the logits are of order one
BASE = {r"^embed$": 40.0, r"^head$": 3.0}

# per row of logits: root mean square of the difference over that of the row.  float32: a few ulp of the largest
# intermediate; bfloat16: 8 bits of mantissa at every product's input, through sharp softmaxes and routers in
# models only 48 to 96 wide (a window or a page that is off by one moves rows by 0.3 and more, see the tests)
TOLERANCE = {"float32": 2e-4, "bfloat16": 0.15}


def make_folder(tmp_path, name: str, sharp: bool = False, config: Optional[ZozosunConfig] = None, seed=None) -> str:
    cfg, s = MODELS.get(name, (config, seed))
    folder = os.path.join(str(tmp_path), f"zozosun_{name}{'_sharp' if sharp else ''}")
    if not os.path.isdir(folder):
        write_random_model(folder, cfg if config is None else config, s if seed is None else seed,
                           scales=dict(BASE, **SHARP) if sharp else BASE)
    return folder


def plain_weights(folder: str) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file
    return load_file(os.path.join(folder, "model.safetensors"))


def plain_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def plain_logits(folder: str, tokens: List[int], config: Optional[dict] = None) -> torch.Tensor:
    return zozosun_plain.forward(tokens, plain_weights(folder), config or plain_config(folder), dtype=torch.float64)


def row_distance(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row: the root mean square of the difference (its mean taken off) over that of the wanted row."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-12)


def assert_rows_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what: str = "") -> None:
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    dist = row_distance(got, want)
    bad = (dist > TOLERANCE[dtype]) | ~torch.isfinite(dist)
    if bad.any():
        i = int(bad.nonzero()[0])
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.numel()} rows differ; first row {i}: distance "
                             f"{dist[i].item():.3g}, allowed {TOLERANCE[dtype]:.3g}; worst {dist.max().item():.3g}")


def fragile_rows(folder: str, tokens: List[int], draws: int = 3, rel: float = 2.0 ** -8) -> torch.Tensor:
    """Which rows of the plain model's logits rest on a close call: they jump by the bfloat16 tolerance
    when the embedding table is disturbed by about one bfloat16 rounding (rows that respond smoothly move by a
    tenth of that).  (The design has such places by
    itself: a read-out that is divided by its own size keeps the sign of a sum that may lie near zero, and
    a router chooses.)  A comparison in bfloat16 leaves these rows out."""
    weights, cfg = plain_weights(folder), plain_config(folder)
    base = zozosun_plain.forward(tokens, weights, cfg, dtype=torch.float64)
    out = torch.zeros(len(tokens), dtype=torch.bool)
    g = torch.Generator().manual_seed(len(tokens))
    for _ in range(draws):
        w = dict(weights)
        w["embed"] = weights["embed"].double() * (1.0 + rel * torch.randn(weights["embed"].shape, generator=g, dtype=torch.float64))
        out |= row_distance(zozosun_plain.forward(tokens, w, cfg, dtype=torch.float64), base) > TOLERANCE["bfloat16"]
    return out


def kept_rows(got: torch.Tensor, folder: str, tokens: List[int], dtype: str, what: str = "", rows=None,
              config: Optional[dict] = None):
    """(engine's rows, plain model's rows) that a comparison may use.  `got`: the engine's logits for all of
    `tokens`, or for the places `rows` among them.  float32: every row; bfloat16: every row that does not rest
    on a close call (at most a sixth of them may)."""
    want = plain_logits(folder, tokens, config)
    keep = torch.ones(len(tokens), dtype=torch.bool)
    if dtype == "bfloat16":
        keep = ~fragile_rows(folder, tokens)
        assert (~keep).float().mean().item() <= 1 / 6 or len(tokens) < 6, f"{what}: too many rows rest on close calls"
    if rows is not None:
        want, keep = want[rows], keep[rows]
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    return got[keep.to(got.device)], want[keep]


def assert_close_but_few(got: torch.Tensor, want: torch.Tensor, dtype: str, what: str = "") -> None:
    """float32: every row.  bfloat16, from twenty rows on: one row in fifty (and one more) may still sit on a call
    that the disturbances did not reach; a fault of a window, a page, a state or a batch moves rows by the dozen."""
    if dtype == "bfloat16" and len(want) >= 20:
        dist = row_distance(got, want)
        order = dist.argsort(descending=True)[len(want) // 50 + 1:]
        got, want = got[order.to(got.device)], want[order]
    assert_rows_close(got, want, dtype, what)


def assert_matches_plain(got: torch.Tensor, folder: str, tokens: List[int], dtype: str, what: str = "",
                         rows=None, config: Optional[dict] = None) -> None:
    assert_close_but_few(*kept_rows(got, folder, tokens, dtype, what, rows, config), dtype, what)


def engine_for(folder: str, dtype: str, num_pages=64, page_size=8, max_requests=4, **kw):
    from serve_amd.config.engine import EngineConfig
    from serve_amd.engine.engine import Engine
    cfg = EngineConfig(dtype=dtype, page_size=page_size, num_pages=num_pages, max_context=num_pages * page_size,
                       max_requests=max_requests, max_tokens_per_step=4096, prefill_chunk=4096, **kw)
    return Engine.from_folder(folder, cfg)


def run_portions(engine, rid, tokens, portions, want_all=True):
    """Feed `tokens` in the given portion sizes, wanting every position; returns [len, V]."""
    from serve_amd.engine.batch import Segment
    assert sum(portions) == len(tokens)
    assert engine.runner.admit(rid)
    rows, at = [], 0
    for n in portions:
        rows.append(engine.step([Segment(rid, tokens[at: at + n], list(range(n)))]))
        at += n
    engine.runner.release(rid)
    return torch.cat(rows, dim=0)


def clear_tokens(folder: str, n: int, rng, vocab: int, margin: float = 0.25, chunk: int = 3) -> List[int]:
    """`n` random tokens for which the plain model's routing decisions are all clear (the last chosen
    expert leads the first that is left out by `margin` of the logits' spread), so that a comparison in
    bfloat16 does not rest on a close call.  Built chunk by chunk: the model is causal, so a chunk that
    brings an unclear decision is drawn again without touching what came before."""
    weights, cfg = plain_weights(folder), plain_config(folder)
    if not any((l.get("mlp") or {}).get("kind") == "moe" for l in cfg["layers"]):
        return [rng.randrange(vocab) for _ in range(n)]
    tokens: List[int] = []
    while len(tokens) < n:
        for _ in range(200):
            cand = tokens + [rng.randrange(vocab) for _ in range(min(chunk, n - len(tokens)))]
            seen: list = []
            zozosun_plain.forward(cand, weights, cfg, dtype=torch.float64, margins=seen)
            if all(m >= margin for t, m in seen if t >= len(tokens)):
                tokens = cand
                break
        else:
            raise RuntimeError("no chunk of tokens with clear routing found")
    return tokens
