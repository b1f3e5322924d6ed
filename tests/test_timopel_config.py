"""Timopel without a GPU: the configuration and its round trip, the tensors the model asks for, which
layer plays which part in the blending of values, the cache it needs, and the plain implementation
against closed forms."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from serve_amd.config.llama import ConfigError
from serve_amd.config.timopel import TimopelConfig
from serve_amd.models.model import Model
from serve_amd.models.timopel import build_timopel_spec
from tests import timopel_models as tm
from tests.plain import timopel_plain as tp


@pytest.mark.parametrize("name", sorted(tm.MODELS))
def test_config_round_trip(name):
    cfg = tm.MODELS[name][0]
    d = cfg.to_hf_dict()
    assert d["architecture"] == "Timopel"
    assert TimopelConfig.from_hf_dict(copy.deepcopy(d)) == cfg
    assert TimopelConfig.from_hf_dict(d).to_hf_dict() == d


def test_config_errors():
    d = tm.TA.to_hf_dict()
    for path, value in ((("layers", 0, "type"), "delta"), (("layers", 1, "mlp", "kind"), "glu"),
                        (("layers", 0, "mixer", "kv_heads"), 3), (("layers", 1, "mlp", "router", "top"), 7),
                        (("layers", 0, "mixer", "q_temp", "every"), 0), (("layers", 1, "mlp", "expert", "limit"), 0.0)):
        bad = copy.deepcopy(d)
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError):
            TimopelConfig.from_hf_dict(bad)
    for key in ("residual_mult", "embedding", "norm", "vocab"):
        bad = copy.deepcopy(d)
        del bad[key]
        with pytest.raises(ConfigError):
            TimopelConfig.from_hf_dict(bad)
    bad = copy.deepcopy(d)
    bad["layers"][3]["mixer"]["vdim"] = 32          # blends with values of another shape
    with pytest.raises(ConfigError):
        TimopelConfig.from_hf_dict(bad)


def test_optional_keys_have_defaults():
    d = tm.TC.to_hf_dict()
    for layer in d["layers"]:
        layer["mixer"].pop("v_mix")
        layer["mixer"].pop("q_temp", None)
    cfg = TimopelConfig.from_hf_dict(d)
    assert all(not l.mixer.v_mix and l.mixer.q_temp is None for l in cfg.layers)


def test_tensor_names_and_shapes():
    model = Model(build_timopel_spec(tm.TA))
    req = {r.checkpoint_name: tuple(r.shape) for r in model.weight_requests() if not r.alias_only}
    assert req["embed"] == (150, 64) and req["final.norm"] == (64,)
    assert req["l0.mix.q"] == (64, 64) and req["l0.mix.k"] == (32, 64) and req["l0.mix.v"] == (8, 64)
    assert req["l0.mix.q.norm"] == (32,) and req["l0.mix.k.norm"] == (32,) and req["l0.mix.sink"] == (2,)
    assert req["l0.mix.o"] == (64, 16)
    assert req["l1.mix.q"] == (64, 64) and req["l1.mix.v"] == (32, 64) and req["l1.mix.sink"] == (4,) and req["l1.mix.o"] == (64, 64)
    assert "l0.mix.vmix" not in req and req["l1.mix.vmix"] == () and req["l3.mix.vmix"] == ()
    assert req["l0.mlp.gate"] == (96, 64) and req["l0.mlp.down"] == (64, 96)
    assert req["l1.mlp.router"] == (6, 64) and req["l1.mlp.e5.up"] == (24, 64) and req["l1.mlp.shared.down"] == (64, 40)
    assert not any(k.startswith("l2.mlp") or k.startswith("l2.norm2") for k in req)
    assert "l3.mlp.shared.gate" not in req and req["l3.mlp.e3.down"] == (64, 32)
    for i in range(4):
        assert req[f"l{i}.norm1"] == (64,) and req[f"l{i}.norm1b"] == (64,)
    # the head is the embedding table: no tensor of its own
    assert [r.checkpoint_name for r in model.weight_requests() if r.alias_only] == ["embed"]


def test_who_blends_with_whom_and_what_is_cached():
    model = Model(build_timopel_spec(tm.TA))
    assert [l.mixer.v_blend for l in model.layers] == ["none", "source", "blend", "blend"]
    assert [l.mixer.q_temp_every for l in model.layers] == [8, 5, 0, 3]
    assert [l.ffn is None for l in model.layers] == [False, False, True, False]
    assert model.graph_safe()
    # keys of 24 and values of 40 share cache heads of 48; keys of 136 heads of 144
    for cfg, size, kv in ((tm.TB, 48, 1), (tm.TD, 144, 1), (tm.TC, 16, 3)):
        reqs = Model(build_timopel_spec(cfg)).cache_requests()
        assert all(r.window is None and [t.shape for t in r.tensors] == [(kv, size), (kv, size)] for r in reqs)
    reqs = Model(build_timopel_spec(tm.TA)).cache_requests()         # layers with cache heads of different sizes
    assert [[t.shape for t in r.tensors] for r in reqs] == [[(1, 32), (1, 32)]] + [[(2, 16), (2, 16)]] * 3
    assert all(s is None for s in model.state_requests())


# ---------------------------------------------------------------------------------------------
# the plain implementation against closed forms
# ---------------------------------------------------------------------------------------------
def test_plain_sink_softmax():
    s = torch.tensor([[0.3, -1.0, 2.0]], dtype=torch.float64)
    none = tp.sink_softmax(s, torch.tensor([-math.inf], dtype=torch.float64))
    assert torch.allclose(none, torch.softmax(s, -1))
    p = tp.sink_softmax(s, torch.tensor([1.5], dtype=torch.float64))
    denom = s.exp().sum() + math.exp(1.5)
    assert torch.allclose(p, s.exp() / denom) and p.sum().item() < 1.0
    # one key: e^s / (e^s + e^sink), also when the sink is by far the larger
    one = tp.sink_softmax(torch.tensor([[0.0]], dtype=torch.float64), torch.tensor([30.0], dtype=torch.float64))
    assert math.isclose(one.item(), 1.0 / (1.0 + math.exp(30.0)), rel_tol=1e-12)
    # a key that is not seen takes no weight
    masked = tp.sink_softmax(torch.tensor([[0.5, -math.inf]], dtype=torch.float64), torch.tensor([0.5], dtype=torch.float64))
    assert torch.allclose(masked, torch.tensor([[0.5, 0.0]], dtype=torch.float64))


def test_plain_query_temperature_steps():
    t = tp.query_temperature(torch.arange(20), 0.5, 8)
    assert torch.all(t[:7] == 1.0)                       # p + 1 < 8
    assert math.isclose(t[7].item(), 1.0 + 0.5 * math.log(2.0)) and t[14] == t[7]
    assert math.isclose(t[15].item(), 1.0 + 0.5 * math.log(3.0))
    assert torch.all(tp.query_temperature(torch.arange(5), 0.0, 1) == 1.0)


def test_plain_route_and_gate():
    z = torch.tensor([[0.1, 2.0, -0.5, 2.0, 1.0]], dtype=torch.float64)
    ids, w = tp.route(z, 3, 2.5)
    assert ids.tolist() == [[1, 3, 4]]                   # a tie goes to the lower index
    chosen = torch.softmax(z[0, [1, 3, 4]], -1)
    assert torch.allclose(w[0], 2.5 * chosen) and math.isclose(w.sum().item(), 2.5)
    g = torch.tensor([-3.0, 0.5, 9.0], dtype=torch.float64)
    u = torch.tensor([-9.0, 0.25, 9.0], dtype=torch.float64)
    a = tp.clamped_swish_gate(g, u, 2.0)
    sig = lambda x: 1.0 / (1.0 + math.exp(-1.702 * x))   # noqa: E731
    assert torch.allclose(a, torch.tensor([-3.0 * sig(-3.0) * (-2.0 + 1.0), 0.5 * sig(0.5) * 1.25, 2.0 * sig(2.0) * 3.0],
                                          dtype=torch.float64))


def test_plain_model_is_causal_and_mechanisms_show(tmp_path):
    """The logits of a prefix do not depend on what follows; the scalar of the layer whose values the others
    blend with is not read; and dropping the sinks, moving a temperature step by one position or not blending
    moves the logits by far more than the tolerance the engine is held to."""
    folder = tm.make_folder(tmp_path, "TA")
    W, cfg = tm.plain_weights(folder), tm.plain_config(folder)
    rng = torch.Generator().manual_seed(1)
    tokens = torch.randint(0, 150, (40,), generator=rng).tolist()
    full = tp.forward(tokens, W, cfg)
    assert torch.allclose(tp.forward(tokens[:17], W, cfg), full[:17], atol=1e-12)
    other = dict(W)
    other["l1.mix.vmix"] = torch.tensor(0.9)
    assert torch.equal(tp.forward(tokens, other, cfg), full)
    loose = 2 * tm.TOLERANCE["bfloat16"]

    def moved(weights=None, config=None):
        return tm.row_distance(tp.forward(tokens, weights or W, config or cfg), full)
    no_sink = {k: (torch.full_like(v, -1e4) if k.endswith(".sink") else v) for k, v in W.items()}
    d = moved(no_sink)
    assert (d[:8] > loose).all() and (d > loose).float().mean() > 0.5
    unblended = {k: (torch.zeros_like(v) if k.endswith(".vmix") else v) for k, v in W.items()}
    assert (moved(unblended) > loose).float().mean() > 0.8
    late = copy.deepcopy(cfg)
    late["layers"][1]["mixer"]["q_temp"]["every"] += 1
    d = moved(config=late)
    # (one position in five has another temperature in one layer of four: the float32 comparison is the one that tells)
    assert d[:4].max() == 0.0 and (d[4:] > 20 * tm.TOLERANCE["float32"]).float().mean() > 0.8


def test_random_model_from_the_command_line(tmp_path):
    """`random-model` writes a folder for the named shape, and again from that folder's config.json: the same
    tensors (a pure function of seed and tensor name), which the plain model can run."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = str(tmp_path / "a"), str(tmp_path / "b")
    run = lambda *args: subprocess.run([sys.executable, "-m", "serve_amd", "random-model", *args], cwd=root,   # noqa: E731
                                       capture_output=True, text=True, timeout=300)
    p = run("--shape", "timopel-tiny", "--out", a, "--seed", "5")
    assert p.returncode == 0, p.stderr[-2000:]
    p = run("--config", os.path.join(a, "config.json"), "--out", b, "--seed", "5")
    assert p.returncode == 0, p.stderr[-2000:]
    wa, wb = tm.plain_weights(a), tm.plain_weights(b)
    assert sorted(wa) == sorted(wb) and all(torch.equal(wa[k], wb[k]) for k in wa)
    logits = tp.forward([1, 2, 3, 4, 5], wa, tm.plain_config(a))
    assert logits.shape == (5, 512) and torch.isfinite(logits).all()


def test_checkpoint_tensors_that_nothing_reads_are_tolerated():
    """A blending scalar in a layer that does not blend and second-half norms in a layer without feed-forward are
    ignored; the first blending layer's scalar may be missing; anything else that is unexpected or missing is an error."""
    from serve_amd.weights.loader import WeightError, check_against, random_reader
    model = Model(build_timopel_spec(tm.TA))
    reader = random_reader(model, 1)
    reader._t["l0.mix.vmix"] = torch.tensor(0.5)
    reader._t["l2.norm2"] = torch.ones(64)
    reader._t["l2.norm2b"] = torch.ones(64)
    del reader._t["l1.mix.vmix"]
    check_against(model, reader)
    reader._t["l2.mlp.gate"] = torch.ones(4, 64)
    del reader._t["l3.mix.vmix"]
    with pytest.raises(WeightError) as e:
        check_against(model, reader)
    assert e.value.unexpected == ["l2.mlp.gate"] and e.value.missing == ["l3.mix.vmix"]
