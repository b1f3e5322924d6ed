"""Zozosun without a GPU: configuration, model description, tensor names, the random-weights writer,
the cache and state the model asks for, and the plain implementation's own consistency."""
from __future__ import annotations

import json
import os
import random

import pytest
import torch

from serve_amd.config.llama import ConfigError
from serve_amd.config.zozosun import ZozosunConfig
from serve_amd.models.model import Model
from serve_amd.registry import get_architecture, load_config
from tests import zozosun_models as zm
from tests.plain import zozosun_plain as zp


@pytest.mark.parametrize("name", list(zm.MODELS))
def test_config_round_trip_and_folder(tmp_path, name):
    cfg = zm.MODELS[name][0]
    assert ZozosunConfig.from_hf_dict(json.loads(json.dumps(cfg.to_hf_dict()))) == cfg
    folder = zm.make_folder(tmp_path, name)
    arch, read = load_config(folder)             # config.json names its architecture as a string
    assert arch.name == "Zozosun" and read == cfg
    model = Model(arch.build_spec(read))
    from safetensors import safe_open
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        names = set(f.keys())
    assert names == {r.checkpoint_name for r in model.weight_requests()}
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.ls1"} <= names


def test_tensor_names_of_each_kind_of_layer():
    model = Model(get_architecture("Zozosun").build_spec(zm.ZA))
    names = {r.checkpoint_name: tuple(r.shape) for r in model.weight_requests()}
    assert names["l0.mix.q.conv"] == (2 * 16, 3) and names["l0.mix.v"] == (4 * 24, 64) and names["l0.mix.A_log"] == (4,)
    assert names["l0.mix.norm"] == (24,) and names["l0.mlp.up"] == (96, 64) and names["l0.mlp.down"] == (64, 96)
    assert names["l1.mix.q"] == (3 * (16 + 8), 64) and names["l1.mix.dkv"] == (40 + 8, 64) and names["l1.mix.dkv.norm"] == (40,)
    assert names["l1.mix.uk"] == (3 * 16, 40) and names["l1.mix.uv"] == (3 * 24, 40)
    assert names["l1.mlp.router"] == (6, 64) and names["l1.mlp.e5.down"] == (64, 32) and names["l1.mlp.shared.sg"] == (1, 64)
    assert "l2.mix.dkv" not in names and "l2.norm2" not in names and "l2.mlp.up" not in names     # reads layer 1's cache; no feed-forward
    assert "l3.mlp.shared.gate" not in names and names["l3.mlp.e4.gate"] == (24, 64)


def test_cache_and_state_the_model_asks_for():
    model = Model(get_architecture("Zozosun").build_spec(zm.ZA))
    order = [(e.layer, e.cache, e.writes_cache) for e in model.spec.run_order]
    assert order == [(0, 0, True), (1, 1, True), (2, 1, False), (3, 2, True)]
    caches, states = model.cache_requests(), model.state_requests()
    assert caches[0] is None and caches[2] is None and states[1] is None
    # rows of kv_rank + rot_dim, padded to 16; kept for the longer of the two windows that read them
    assert [t.shape for t in caches[1].tensors] == [(1, 48), (1, 48)] and caches[1].window == 33
    assert states[0].shape == (4 * 16 * 24 + 2 * (2 * 2 * 16 + 4 * 24),) and states[0].dtype == torch.float32
    assert states[2].shape == (2 * 40 * 16 + 1 * (2 * 2 * 40 + 2 * 16),)
    only_delta = Model(get_architecture("Zozosun").build_spec(zm.ZD))
    assert all(c is None for c in only_delta.cache_requests()) and only_delta.graph_safe()


def test_config_errors_name_the_key():
    good = zm.ZA.to_hf_dict()
    for change, text in (
            (lambda d: d["layers"][2]["mixer"].update(kv_from=0), "kv_from"),
            (lambda d: d["layers"][2]["mixer"].update(kv_rank=24), "kv_rank"),
            (lambda d: d["layers"][1]["mixer"]["rot"].update(dims=4), "rot.dims"),
            (lambda d: d["layers"][0].update(type="conv"), "type"),
            (lambda d: d["layers"][3]["mlp"]["router"].update(top=9), "top"),
            (lambda d: d["layers"][0]["mixer"].pop("conv"), "conv"),
            (lambda d: d["layers"][0]["mlp"].update(kind="glu"), "kind"),
            (lambda d: d.pop("width"), "width")):
        bad = json.loads(json.dumps(good))
        change(bad)
        with pytest.raises(ConfigError, match=text):
            ZozosunConfig.from_hf_dict(bad)


def test_step_cost_counts_the_chosen_experts_only():
    model = Model(get_architecture("Zozosun").build_spec(zm.ZA))
    ffn = model.layers[1].ffn
    one = ffn.step_cost(1)
    many = ffn.step_cost(100)
    per_expert = 3 * 32 * 64
    assert one.weight_elements == 6 * 64 + 2 * per_expert + 3 * 48 * 64 + 64
    assert many.weight_elements == 6 * 64 + 6 * per_expert + 3 * 48 * 64 + 64
    assert many.flops == pytest.approx(100 * one.flops)


# -- the plain implementation against itself ------------------------------------------------------
def test_plain_recurrence_equals_its_closed_form_for_one_token():
    q, k, v = torch.randn(1, 6, dtype=torch.float64), torch.randn(1, 6, dtype=torch.float64), torch.randn(1, 4, dtype=torch.float64)
    out = zp.delta_recurrence(q, k, v, torch.tensor([0.7], dtype=torch.float64), torch.tensor([0.3], dtype=torch.float64))
    assert torch.allclose(out[0], 0.7 * v[0] * (k[0] @ q[0]))        # S = k (beta v)^T from a zero state


def test_plain_convolution_and_rotation():
    x = torch.arange(12, dtype=torch.float64).view(6, 2)
    w = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]], dtype=torch.float64)
    y = zp.short_conv(x, w)
    assert y[0].tolist() == [0.0, 1.0] and y[1].tolist() == [200.0, 3.0] and y[3].tolist() == [2 + 40 + 600, 7.0]
    v = torch.randn(5, 3, 8, dtype=torch.float64)
    r = zp.rotate(v, torch.arange(5), 100.0)
    assert torch.allclose(r.norm(dim=-1), v.norm(dim=-1)) and torch.allclose(r[0], v[0])
    # a score between two rotated vectors depends on the distance of their positions only
    a, b = torch.randn(1, 8, dtype=torch.float64), torch.randn(1, 8, dtype=torch.float64)
    s1 = zp.rotate(a, torch.tensor([7]), 50.0) @ zp.rotate(b, torch.tensor([3]), 50.0).t()
    s2 = zp.rotate(a, torch.tensor([104]), 50.0) @ zp.rotate(b, torch.tensor([100]), 50.0).t()
    assert torch.allclose(s1, s2)


@pytest.mark.parametrize("name", ["ZA", "ZB"])
def test_plain_model_is_causal_and_windows_forget(tmp_path, name):
    folder = zm.make_folder(tmp_path, name, sharp=True)
    rng = random.Random(2)
    vocab = zm.MODELS[name][0].vocab
    tokens = [rng.randrange(vocab) for _ in range(30)]
    full = zm.plain_logits(folder, tokens)
    assert torch.allclose(zm.plain_logits(folder, tokens[:17]), full[:17], atol=1e-9)
    changed = list(tokens)
    changed[0] = (tokens[0] + 1) % vocab
    assert not torch.allclose(zm.plain_logits(folder, changed)[-1], full[-1], atol=1e-6)   # the delta rule's state remembers
