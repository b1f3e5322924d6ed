"""Small Timopel models for the tests, their folders with random weights, and comparisons of the
engine's logits with the plain implementation's (tests/plain/timopel_plain.py).

The models differ in every size and option:
  TA  width 64; layers: (no blending, dense), (blending begins here, experts with a shared one),
      (blends, no feed-forward), (blends, experts without a shared one, top 1); 4 heads on 2 key/value heads
      of 16 x 16, but in the first layer 2 heads on one with keys of 32 and values of 8 (layers of one model with
      cache heads of different sizes); query temperature steps every 8 / 5 / 3 positions and one layer without
  TB  width 96, 6 heads on one key/value head, keys of 24 and values of 40 (a cache head of 48), eps 1e-6,
      an embedding scale of 1, every layer blends, top 2 of 5
  TC  width 50 (no multiple of 8), as many key/value heads as heads (3), keys of 10 and values of 7, vocabulary
      101, experts of width 9 of which all are taken (top = experts = 3), nobody blends
  TD  keys of 136 (a cache head of 144: above what the matrix-core and tiled attention kernels take), values of
      20, 2 heads on one key/value head
  TE  20 heads on one key/value head (more rows a key/value head than the kernels for single tokens take), a layer
      that does not blend between two that do, top 2 of 9 experts
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch

from serve_amd.config.timopel import (ClampedMoeConfig, GatedDenseConfig, QueryTemperature, SinkAttentionConfig,
                                      TimopelConfig, TimopelLayerConfig)
from serve_amd.weights.loader import write_random_model
from tests.plain import timopel_plain

L = TimopelLayerConfig


def _att(heads, kv_heads, dim, vdim, scale, temp=None, v_mix=False):
    return SinkAttentionConfig(heads, kv_heads, dim, vdim, scale, None if temp is None else QueryTemperature(*temp), v_mix)


TA = TimopelConfig(vocab=150, width=64, eps=1e-5, residual_mult=0.4, embedding_scale=2.0, layers=(
    L(_att(2, 1, 32, 8, 0.3, (0.4, 8)), GatedDenseConfig(96)),
    L(_att(4, 2, 16, 16, 0.45, (0.7, 5), v_mix=True), ClampedMoeConfig(6, 2, 1.7, 24, 1.0, 40, 0.7)),
    L(_att(4, 2, 16, 16, 0.45, None, v_mix=True), None),
    L(_att(4, 2, 16, 16, 0.45, (0.2, 3), v_mix=True), ClampedMoeConfig(4, 1, 0.8, 32, 2.5)),
))

TB = TimopelConfig(vocab=211, width=96, eps=1e-6, residual_mult=0.7, embedding_scale=1.0, layers=(
    L(_att(6, 1, 24, 40, 0.3, (0.5, 7), v_mix=True), ClampedMoeConfig(5, 2, 1.0, 40, 1.5, 24, 3.0)),
    L(_att(6, 1, 24, 40, 0.3, (0.5, 7), v_mix=True), GatedDenseConfig(120)),
))

TC = TimopelConfig(vocab=101, width=50, eps=1e-5, residual_mult=1.0, embedding_scale=0.5, layers=(
    L(_att(3, 3, 10, 7, 0.5, (1.0, 2)), ClampedMoeConfig(3, 3, 3.0, 9, 0.9, 5, 0.9)),
    L(_att(3, 3, 10, 7, 0.5, (0.3, 11)), GatedDenseConfig(30)),
    L(_att(3, 3, 10, 7, 0.5, None), None),
))

TD = TimopelConfig(vocab=120, width=64, eps=1e-5, residual_mult=0.3, embedding_scale=4.0, layers=(
    L(_att(2, 1, 136, 20, 0.15, (0.3, 16), v_mix=True), GatedDenseConfig(64)),
    L(_att(2, 1, 136, 20, 0.15, (0.3, 16), v_mix=True), None),
))

TE = TimopelConfig(vocab=130, width=80, eps=1e-5, residual_mult=0.3, embedding_scale=1.5, layers=(
    L(_att(20, 1, 32, 32, 0.2, (0.3, 4), v_mix=True), ClampedMoeConfig(9, 2, 1.0, 16, 1.2, 24, 1.2)),
    L(_att(20, 1, 32, 32, 0.2, (0.3, 4), v_mix=False), GatedDenseConfig(48)),
    L(_att(20, 1, 32, 32, 0.2, (0.3, 4), v_mix=True), None),
))

MODELS = {"TA": (TA, 3), "TB": (TB, 4), "TC": (TC, 5), "TD": (TD, 6), "TE": (TE, 7)}

# the embedding at a scale at which the logits (the table is the output matrix too) are of order one, and sinks
# that weigh as much as dozens of keys in some heads
BASE = {r"^embed$": 12.0, r"\.sink$": 2.5}

# per row of logits: root mean square of the difference over that of the row.  float32: a few ulp of the
# largest intermediate; bfloat16: 8 bits of mantissa at every product's input, through sharp softmaxes and
# models 50 to 96 wide (a lost sink, a temperature step that is one position off or values that are
# not blended move rows by several times this, see the tests; the routers' choices are kept clear, `clear_tokens`)
TOLERANCE = {"float32": 2e-4, "bfloat16": 0.08}


def make_folder(tmp_path, name: str, config: Optional[TimopelConfig] = None, seed=None, scales=None) -> str:
    cfg, s = MODELS.get(name, (config, seed))
    folder = os.path.join(str(tmp_path), f"timopel_{name}")
    if not os.path.isdir(folder):
        write_random_model(folder, cfg if config is None else config, s if seed is None else seed,
                           scales=dict(BASE, **(scales or {})))
    return folder


def plain_weights(folder: str) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file
    return load_file(os.path.join(folder, "model.safetensors"))


def plain_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def plain_logits(folder: str, tokens: List[int], config: Optional[dict] = None,
                 weights: Optional[Dict[str, torch.Tensor]] = None) -> torch.Tensor:
    return timopel_plain.forward(tokens, weights or plain_weights(folder), config or plain_config(folder),
                                 dtype=torch.float64)


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


_CLEAR: Dict[tuple, List[int]] = {}


def clear_tokens(folder: str, n: int, seed: int, vocab: int, margin: float = 0.07, chunk: int = 4) -> List[int]:
    """`n` random tokens for which every routing decision of the plain model is clear (the last chosen expert
    leads the first that is left out by `margin` of the logits' spread), so that a comparison in bfloat16 does
    not rest on a close call: one flipped choice moves its own row, and through that token's keys and values
    in the layers behind, rows after it.  Built chunk by chunk: the model is causal, so a chunk that brings an
    unclear decision is drawn again without touching what came before."""
    import random
    key = (os.path.basename(folder), n, seed, vocab)
    if key in _CLEAR:
        return _CLEAR[key]
    rng = random.Random(seed)
    weights, cfg = plain_weights(folder), plain_config(folder)
    if not any((l.get("mlp") or {}).get("kind") == "moe" for l in cfg["layers"]):
        _CLEAR[key] = [rng.randrange(vocab) for _ in range(n)]
        return _CLEAR[key]
    tokens: List[int] = []
    while len(tokens) < n:
        for _ in range(300):
            cand = tokens + [rng.randrange(vocab) for _ in range(min(chunk, n - len(tokens)))]
            seen: list = []
            timopel_plain.forward(cand, weights, cfg, dtype=torch.float64, margins=seen)
            if all(m >= margin for t, m in seen if t >= len(tokens)):
                tokens = cand
                break
        else:
            raise RuntimeError("no chunk of tokens with clear routing found")
    _CLEAR[key] = tokens
    return tokens


def assert_matches_plain(got: torch.Tensor, folder: str, tokens: List[int], dtype: str, what: str = "", rows=None) -> None:
    """`got`: the engine's logits for all of `tokens`, or for the places `rows` among them.  float32: every row.
    bfloat16 (with tokens whose routing is clear, `clear_tokens`): of twenty rows and more, one in fifty (and one)
    may be off; a fault of a page, a slot, a batch or a mechanism moves rows by the dozen."""
    want = plain_logits(folder, tokens)
    if rows is not None:
        want = want[rows]
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    got = got.detach().cpu()
    if dtype == "bfloat16" and len(want) >= 20:
        order = row_distance(got, want).argsort(descending=True)[len(want) // 50 + 1:]
        got, want = got[order], want[order]
    assert_rows_close(got, want, dtype, what)


def engine_for(folder: str, dtype: str, num_pages=64, page_size=8, max_requests=4, **kw):
    from serve_amd.config.engine import EngineConfig
    from serve_amd.engine.engine import Engine
    cfg = EngineConfig(dtype=dtype, page_size=page_size, num_pages=num_pages, max_context=num_pages * page_size,
                       max_requests=max_requests, max_tokens_per_step=4096, prefill_chunk=4096, **kw)
    return Engine.from_folder(folder, cfg)


def run_portions(engine, rid, tokens, portions):
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
