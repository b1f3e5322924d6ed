"""The Zozosun decoder through the engine against the plain implementation, float32 and bfloat16:
whole prompts; prompt then token by token; portions down to two tokens; unequal requests in one
batch against each alone, with pages and state slots that are freed and used again; keys just inside
and just outside a window, at page borders and far back, in prompts and in decoding; first tokens;
long decoding; greedy generation through the scheduler (graphs and steps launched ahead included)."""
from __future__ import annotations

import copy
import random

import pytest
import torch

from tests import zozosun_models as zm

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
NAMES = ["ZA", "ZB", "ZD", "ZL", "ZO"]


def tokens_for(folder, dtype, n, seed, vocab):
    rng = random.Random(seed)
    # bfloat16 must not rest on a close call of a router; float32 takes whatever comes
    return zm.clear_tokens(folder, n, rng, vocab) if dtype == "bfloat16" else [rng.randrange(vocab) for _ in range(n)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sharp", [False, True])
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts_and_first_tokens(tmp_path, name, sharp, dtype):
    folder = zm.make_folder(tmp_path, name, sharp)
    engine = zm.engine_for(folder, dtype)
    vocab = zm.MODELS[name][0].vocab
    for n in (1, 2, 3, 5, 61):          # shorter than the convolution's taps, than a page, than the windows; longer
        tokens = tokens_for(folder, dtype, n, 100 + n, vocab)
        got = zm.run_portions(engine, f"r{n}", tokens, [n])
        zm.assert_matches_plain(got, folder, tokens, dtype, f"{name} whole {n}")
    engine.runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_token_by_token(tmp_path, name, dtype):
    folder = zm.make_folder(tmp_path, name, sharp=True)
    engine = zm.engine_for(folder, dtype)
    vocab = zm.MODELS[name][0].vocab
    tokens = tokens_for(folder, dtype, 84, 7, vocab)
    got = zm.run_portions(engine, "r", tokens, [84 - 45] + [1] * 45)     # the windows pass over decoded tokens
    zm.assert_matches_plain(got, folder, tokens, dtype, f"{name} prompt + 45 single tokens")
    got = zm.run_portions(engine, "s", tokens[:30], [1] * 30)             # from the very first token on
    zm.assert_matches_plain(got, folder, tokens, dtype, f"{name} token by token from the start", rows=slice(0, 30))
    if dtype == "float32":
        whole = zm.run_portions(engine, "w", tokens, [84])
        assert zm.row_distance(got, whole[:30]).max().item() <= 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(tmp_path, name, dtype):
    folder = zm.make_folder(tmp_path, name, sharp=True)
    engine = zm.engine_for(folder, dtype)
    vocab = zm.MODELS[name][0].vocab
    tokens = tokens_for(folder, dtype, 73, 8, vocab)
    for portions in ([7, 2, 16, 3, 2, 9, 2, 11, 5, 4, 1, 1, 2, 8], [2] * 10 + [53], [1, 3, 69], [40, 33]):
        got = zm.run_portions(engine, "r", tokens, portions)
        zm.assert_matches_plain(got, folder, tokens, dtype, f"{name} portions {portions}")


def mixed_trace(rng, reqs, max_live=4):
    """Up to `max_live` live requests; portions of some beside single tokens of others; staggered."""
    fed = {k: 0 for k in reqs}
    order, live, steps, nxt = list(reqs), [], [], 0
    while nxt < len(order) or live:
        while len(live) < max_live and nxt < len(order) and (not live or rng.random() < 0.6):
            live.append(order[nxt])
            nxt += 1
        entries, ended = [], []
        for k in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue                         # left out of this step, goes on later
            n = min(len(reqs[k]) - fed[k], rng.choice([1, 1, 1, 2, 3, 5, 8, 13]))
            entries.append((k, reqs[k][fed[k]: fed[k] + n]))
            fed[k] += n
            if fed[k] == len(reqs[k]):
                ended.append(k)
                live.remove(k)
        if entries:
            steps.append((entries, ended))
    return steps


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_requests_together_with_pages_and_slots_used_again(tmp_path, name, dtype):
    from serve_amd.engine.batch import Segment
    folder = zm.make_folder(tmp_path, name, sharp=True)
    page_size = 4
    lengths = [23, 41, 9, 30, 17, 2, 36, 1, 40, 28, 33, 5]
    # four live requests of at most 41 tokens: pool and slots are far fewer than the requests need together
    engine = zm.engine_for(folder, dtype, num_pages=4 * 11 + 1, page_size=page_size, max_requests=4)
    vocab = zm.MODELS[name][0].vocab
    reqs = {f"q{i}": tokens_for(folder, dtype, n, 300 + i, vocab) for i, n in enumerate(lengths)}
    steps = mixed_trace(random.Random(13), reqs)
    rows = {k: [] for k in reqs}
    slots_seen = {}
    for entries, ended in steps:
        segs = []
        for k, toks in entries:
            if k not in engine.runner.cache:
                assert engine.runner.admit(k)
                slots_seen.setdefault(engine.runner.cache.slot_of(k), []).append(k)
            segs.append(Segment(k, toks, list(range(len(toks)))))
        logits = engine.step(segs)
        at = 0
        for k, toks in entries:
            rows[k].append(logits[at: at + len(toks)])
            at += len(toks)
        for k in ended:
            engine.runner.release(k)
        engine.runner.cache.check_invariants()
    assert any(len(v) > 1 for v in slots_seen.values()), "no state slot was used twice"
    pairs = [zm.kept_rows(torch.cat(rows[k]), folder, toks, dtype, f"{name} request {k} in the mix") for k, toks in reqs.items()]
    if dtype == "float32":
        for (got, want), k in zip(pairs, reqs):
            zm.assert_rows_close(got, want, dtype, f"{name} request {k} in the mix")
    zm.assert_close_but_few(torch.cat([g.cpu() for g, _ in pairs]), torch.cat([w for _, w in pairs]), dtype,
                            f"{name}: all requests of the mix")


def _with_windows(config: dict, shift: int) -> dict:
    c = copy.deepcopy(config)
    for layer in c["layers"]:
        if layer["type"] == "latent_attention" and layer["mixer"].get("mask"):
            layer["mixer"]["mask"]["size"] += shift
    return c


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["ZA", "ZB", "ZL"])
def test_window_edges_show_in_the_logits_and_are_right(tmp_path, name, dtype):
    """With sharp attention a window that is one token too long or too short moves the logits by far more than
    the tolerance (the plain model says so); the engine agrees with the right window, for tokens of a prompt, of
    portions that end and begin around the edge, and for single tokens."""
    folder = zm.make_folder(tmp_path, name, sharp=True)
    cfg = zm.plain_config(folder)
    vocab = zm.MODELS[name][0].vocab
    tokens = tokens_for(folder, dtype, 70, 21, vocab)
    want = zm.plain_logits(folder, tokens)
    longest = max(l["mixer"]["mask"]["size"] for l in cfg["layers"] if l["mixer"].get("mask"))
    # (short windows move every row a lot; a window of 33 keys moves them by less than bfloat16's tolerance,
    # and there the float32 run is the one that would tell)
    shows = (name, dtype) in (("ZA", "float32"), ("ZB", "float32"), ("ZB", "bfloat16"))
    for shift in (-1, 1) if shows else ():
        other = zm.plain_logits(folder, tokens, _with_windows(cfg, shift))
        moved = zm.row_distance(other, want)
        assert (moved[longest:] > 2 * zm.TOLERANCE[dtype]).float().mean().item() > 0.5, f"a window off by {shift} would not show"
    engine = zm.engine_for(folder, dtype, page_size=4)
    windows = sorted({l["mixer"]["mask"]["size"] for l in cfg["layers"] if l["mixer"].get("mask")})
    for portions in ([70], [windows[0] - 1, 1, 1, 1] + [70 - windows[0] - 2], [windows[-1], 2, 2] + [1] * (66 - windows[-1]),
                     [3] + [1] * 67):
        got = zm.run_portions(engine, "r", tokens, portions)
        zm.assert_matches_plain(got, folder, tokens, dtype, f"{name} windows {windows}, portions {portions[:5]}...")


def far_key_model(tmp_path):
    """One latent-attention layer that sees every key, and an embedding table made so that one score
    stands out: the row of token 1 is solved for, so that the one head's query of token 1, taken into the latent
    space, points along the latent of token 0.  A sequence that ends in token 1 and holds token 0 once,
    far back, then reads that one key with nearly all of its weight."""
    from safetensors.torch import save_file
    from serve_amd.config.zozosun import ZozosunConfig, ZozosunLayerConfig
    from tests.plain import zozosun_plain as zp
    import os
    cfg = ZozosunConfig(vocab=90, width=64, eps=1e-5, layers=(
        ZozosunLayerConfig(zm._latent(1, 16, 8, 16, 48, None, scale=0.6), None),))
    folder = zm.make_folder(tmp_path, "far", config=cfg, seed=11)
    W = zm.plain_weights(folder)
    m = zm.plain_config(folder)["layers"][0]["mixer"]
    Wd = {k: v.double() for k, v in W.items()}
    c0, _ = zp.latent_and_rotated_key(Wd["embed"][0:1], Wd, "l0.mix.", m, 1e-5)
    dn, dr, R = m["dim"], m["rot_dim"], m["kv_rank"]
    A = Wd["l0.mix.uk"][:dn].t() @ Wd["l0.mix.q"][:dn]                 # token's row -> its query in the latent space
    target = 50.0 / m["scale"] * c0[0] / c0[0].pow(2).sum()              # a score of 50 against token 0's latent
    W["embed"][1] = (torch.linalg.pinv(A) @ target).to(W["embed"].dtype)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return folder


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_among_hundreds(tmp_path, dtype):
    folder = far_key_model(tmp_path)
    rng = random.Random(5)
    n = 420
    for far in (3, 37, 203):                  # in the first page, further on, and the last key of a page (page size 4)
        with_key = [rng.randrange(2, 90) for _ in range(n - 1)] + [1]
        with_key[far] = 0
        without = list(with_key)
        without[far] = 2
        want = zm.plain_logits(folder, with_key)[-1:]
        # losing that one key would move the last row by far more than the tolerance
        assert zm.row_distance(zm.plain_logits(folder, without)[-1:], want).item() > 2 * zm.TOLERANCE[dtype]
        engine = zm.engine_for(folder, dtype, num_pages=120, page_size=4)
        got = zm.run_portions(engine, "r", with_key, [n - 3, 1, 1, 1])[-1:]
        zm.assert_rows_close(got, want, dtype, f"key {far} of {n}, read by a token decoded alone")
        got = zm.run_portions(engine, "r", with_key, [200, 220])[-1:]
        zm.assert_rows_close(got, want, dtype, f"key {far} of {n}, read from a portion")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["ZA", "ZD"])
def test_long_decoding_keeps_the_state(tmp_path, name, dtype):
    folder = zm.make_folder(tmp_path, name)
    engine = zm.engine_for(folder, dtype, num_pages=80)
    vocab = zm.MODELS[name][0].vocab
    tokens = tokens_for(folder, dtype, 260, 31, vocab)
    got = zm.run_portions(engine, "r", tokens, [4] + [1] * 256)
    zm.assert_matches_plain(got, folder, tokens, dtype, f"{name} 256 single tokens")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["ZA", "ZB"])
def test_greedy_generation_through_the_scheduler(tmp_path, name, dtype):
    """`generate` (scheduler, mixed steps, graphs, steps launched ahead of the host) picks the tokens the
    plain model picks, as long as the plain model's choice is clear."""
    from serve_amd.engine.engine import Request
    folder = zm.make_folder(tmp_path, name)
    engine = zm.engine_for(folder, dtype, num_pages=128, page_size=8, max_requests=3)
    vocab = zm.MODELS[name][0].vocab
    prompts = [tokens_for(folder, dtype, n, 50 + n, vocab) for n in (5, 19, 1, 33, 8)]
    new = 12
    reqs = [Request(torch.tensor(p), len(p), new) for p in prompts]
    out = engine.generate(reqs, temperature=0.0, return_logits="all")
    for p, o in zip(prompts, out):
        assert o.error is None and len(o.generated_tokens) == new
        seq = list(p)
        for i, tok in enumerate(o.generated_tokens.tolist()):
            row = zm.plain_logits(folder, seq)[-1]
            top2 = row.topk(2).values
            if (top2[0] - top2[1]).item() < (1e-3 if dtype == "float32" else 0.15):
                break                            # the plain model's own choice is a close call: stop comparing
            assert tok == int(row.argmax()), f"{name}: token {i} after a prompt of {len(p)}"
            if dtype == "float32":
                zm.assert_rows_close(o.logits[i: i + 1], row[None], dtype, f"{name} logits of generated token {i}")
            seq.append(tok)
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.free_slots() == 3


# ---------------------------------------------------------------------------------------------
# the kernels alone
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("experts,top", [(5, 1), (16, 2), (70, 3), (130, 8)])
def test_route_picks_the_largest_and_weights_them_among_themselves(experts, top):
    from serve_amd import ops
    torch.manual_seed(experts)
    T = 37
    logits = torch.randn(T, experts + 1, device="cuda")          # one more column rides along, as the shared gate does
    ids = torch.empty(T, top, dtype=torch.int32, device="cuda")
    w = torch.empty(T, top, dtype=torch.float32, device="cuda")
    ops.moe_route(logits, experts, top, ids, w)
    vals, want = logits[:, :experts].double().topk(top, dim=-1)
    assert torch.equal(ids.long(), want)
    assert torch.allclose(w.double(), torch.softmax(vals, -1), atol=1e-6)


def test_experts_route_by_themselves_for_few_tokens():
    from serve_amd import ops
    torch.manual_seed(9)
    T, d, F, E, top = 13, 64, 32, 9, 3
    h = torch.randn(T, d, device="cuda").bfloat16()
    wg, wu = (torch.randn(E, F, d, device="cuda") * 0.2).bfloat16(), (torch.randn(E, F, d, device="cuda") * 0.2).bfloat16()
    wd = (torch.randn(E, d, F, device="cuda") * 0.2).bfloat16()
    logits = torch.randn(T, E + 1, device="cuda")
    ids_a, w_a = torch.empty(T, top, dtype=torch.int32, device="cuda"), torch.empty(T, top, device="cuda")
    ops.moe_route(logits, E, top, ids_a, w_a)
    yk_a = torch.empty(T * top, d, device="cuda")
    ops.moe_experts(h, ids_a, wg, wu, wd, yk_a)
    ids_b, w_b = torch.full((T, top), -1, dtype=torch.int32, device="cuda"), torch.zeros(T, top, device="cuda")
    yk_b = torch.empty(T * top, d, device="cuda")
    ops.moe_experts(h, ids_b, wg, wu, wd, yk_b, logits, w_b)
    assert torch.equal(ids_a, ids_b) and torch.equal(w_a, w_b) and torch.equal(yk_a, yk_b)


@pytest.mark.parametrize("T,d,F", [(45, 72, 40), (45, 75, 42), (400, 64, 48)])   # few rows; sizes the matrix cores do not take; many rows
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_experts_against_one_by_one(dtype, T, d, F):
    from serve_amd import ops
    torch.manual_seed(3)
    E, top = 7, 3
    h = torch.randn(T, d, device="cuda").to(dtype)
    wg, wu = (torch.randn(E, F, d, device="cuda") * 0.2).to(dtype), (torch.randn(E, F, d, device="cuda") * 0.2).to(dtype)
    wd = (torch.randn(E, d, F, device="cuda") * 0.2).to(dtype)
    ids = torch.stack([torch.randperm(E, device="cuda")[:top] for _ in range(T)]).int().contiguous()
    ids[5: T - 5] = ids[4]                               # many rows for few experts: more than one tile of rows
    yk = torch.empty(T * top, d, dtype=torch.float32, device="cuda")
    ops.moe_experts(h, ids, wg, wu, wd, yk)
    hd = h.double()
    for t in list(range(0, T, 7)) + [4, 5, T - 6, T - 5, T - 1]:
        for k in range(top):
            e = int(ids[t, k])
            a = torch.nn.functional.silu(hd[t] @ wg[e].double().t()) * (hd[t] @ wu[e].double().t())
            if dtype == torch.bfloat16:
                a = a.to(dtype).double()
            want = a @ wd[e].double().t()
            assert torch.allclose(yk[t * top + k].double(), want, atol=2e-4 if dtype == torch.float32 else 2e-2, rtol=1e-3)


@pytest.mark.parametrize("T", [1, 9, 64, 65, 200])          # a workgroup per (token, head) up to 64 tokens, tiles of tokens above
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_per_head_products(dtype, T):
    from serve_amd import ops
    torch.manual_seed(T)
    H, K, N, stride_in, stride_out = 5, 37, 70, 5 * 48, 5 * 80      # heads' inputs and outputs lie inside wider rows
    x = torch.randn(T, stride_in, device="cuda").to(dtype)
    w = (torch.randn(H, K, N, device="cuda") * 0.3).to(dtype)
    out = torch.full((T, stride_out), 7.0, device="cuda").to(dtype)
    ops.head_linear(x, stride_in, 48, w, out, stride_out, 80, T)
    want = torch.einsum("thk,hkn->thn", x.view(T, H, 48)[:, :, :K].double(), w.double())
    got = out.view(T, H, 80)
    tol = dict(atol=1e-4 if dtype == torch.float32 else 5e-2, rtol=1e-2)
    assert torch.allclose(got[:, :, :N].double(), want, **tol)
    assert (got[:, :, N:] == 7.0).all(), "a place behind a head's outputs was written"
    # with a tail: the 6 inputs behind the K are rotated by position and put behind the N outputs, then 2 zeros
    from tests.plain import zozosun_plain as zp
    positions = torch.arange(3, 3 + T, dtype=torch.int32, device="cuda")
    base = 50.0
    inv_freq = torch.tensor([base ** (-2.0 * i / 6) for i in range(3)], dtype=torch.float32, device="cuda")
    ops.head_linear(x, stride_in, 48, w, out, stride_out, 80, T, positions, inv_freq, 6, 8)
    got = out.view(T, H, 80)
    assert torch.allclose(got[:, :, :N].double(), want, **tol)
    turned = zp.rotate(x.view(T, H, 48)[:, :, K: K + 6].double().cpu(), positions.cpu().long(), base)
    assert torch.allclose(got[:, :, N: N + 6].double().cpu(), turned, **tol)
    assert (got[:, :, N + 6: N + 8] == 0).all() and (got[:, :, N + 8:] == 7.0).all()


@pytest.mark.parametrize("longest", [1, 64])      # which shape of the recurrence kernel runs: single tokens, prompt portions
@pytest.mark.parametrize("dk,dv,heads,kv_heads,taps", [(16, 24, 4, 2, 3), (72, 80, 2, 1, 4), (200, 8, 1, 1, 1), (33, 130, 3, 3, 2)])
def test_delta_rule_kernels_in_two_steps(dk, dv, heads, kv_heads, taps, longest):
    """The kernels over two steps of two segments (one of them a single token) against the plain
    recurrence over the whole sequences: the state and the convolution's last inputs carry over."""
    from types import SimpleNamespace
    from serve_amd import ops
    from tests.plain import zozosun_plain as zp
    torch.manual_seed(dk)
    H, Hk = heads, kv_heads
    C = 2 * Hk * dk + H * dv
    lens = [[9, 1], [1, 6]]                              # request 0: 9 then 1 tokens; request 1: 1 then 6
    total = [sum(x) for x in zip(*lens)]
    z = [torch.randn(n, C + H * dv, dtype=torch.float64) for n in total]
    ba = [torch.randn(n, 2 * H, dtype=torch.float64) for n in total]
    conv_w = torch.randn(C, taps, dtype=torch.float64) * 0.6
    A_log, dt_bias, norm_w = -torch.rand(H, dtype=torch.float64) * 3, -torch.rand(H, dtype=torch.float64) * 2, 1 + 0.1 * torch.randn(dv, dtype=torch.float64)
    eps = 1e-5
    want = []
    for r in range(2):
        conv = zp.silu(zp.short_conv(z[r][:, :C], conv_w))
        q = zp.unit_vectors(conv[:, :Hk * dk].view(-1, Hk, dk)) * dk ** -0.5
        k = zp.unit_vectors(conv[:, Hk * dk: 2 * Hk * dk].view(-1, Hk, dk))
        v = conv[:, 2 * Hk * dk:].view(-1, H, dv)
        beta = torch.sigmoid(ba[r][:, :H])
        g = torch.exp(-torch.exp(A_log) * zp.softplus(ba[r][:, H:] + dt_bias))
        gate = zp.silu(z[r][:, C:]).view(-1, H, dv)
        out = torch.stack([zp.rms(zp.delta_recurrence(q[:, i // (H // Hk)], k[:, i // (H // Hk)], v[:, i], beta[:, i], g[:, i]), eps)
                           * norm_w * gate[:, i] for i in range(H)], dim=1)
        want.append(out.reshape(-1, H * dv))
    state = torch.zeros(3, H * dk * dv + (taps - 1) * C + 5, dtype=torch.float32, device="cuda")
    f = lambda t: t.float().cuda().contiguous()   # noqa: E731
    at = [0, 0]
    got = [[], []]
    for step in range(2):
        n = [lens[step][0], lens[step][1]]
        zs = torch.cat([z[r][at[r]: at[r] + n[r]] for r in range(2)])
        bs = torch.cat([ba[r][at[r]: at[r] + n[r]] for r in range(2)])
        T = zs.shape[0]
        ctx = SimpleNamespace(num_tokens=T, num_segments=2, max_q_len=longest,
                              seg_of_token=torch.tensor([0] * n[0] + [1] * n[1], dtype=torch.int32, device="cuda"),
                              cu_q=torch.tensor([0, n[0], T], dtype=torch.int32, device="cuda"),
                              state_slots=torch.tensor([2, 0], dtype=torch.int32, device="cuda"))
        y = torch.empty(T, H * dv, dtype=torch.float32, device="cuda")
        ops.delta_rule(f(zs), f(conv_w), f(bs), f(A_log), f(dt_bias), f(norm_w), state, ctx, y, eps, H, Hk, dk, dv, taps)
        got[0].append(y[: n[0]].cpu())
        got[1].append(y[n[0]:].cpu())
        at = [at[0] + n[0], at[1] + n[1]]
    for r in range(2):
        g_ = torch.cat(got[r]).double()
        assert torch.allclose(g_, want[r], atol=3e-4, rtol=1e-3), f"request {r}: max diff {(g_ - want[r]).abs().max().item():.3g}"
    assert state[1].abs().max().item() == 0.0, "a slot that no segment named was written"


# ---------------------------------------------------------------------------------------------
# the trace runner as a user runs it
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_traces_through_the_program(tmp_path, dtype):
    """`bin/trace_run` as a child process on a model folder: whole prompts, prompt then single tokens, portions, and
    a mix of four live requests (the program has four state slots, and pages for 256 tokens), against the plain model."""
    import json
    import os
    import subprocess
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    name = "ZA"
    folder = zm.make_folder(tmp_path, name, sharp=True)
    vocab = zm.MODELS[name][0].vocab
    reqs, steps = {}, []

    def feed(key, n, portions, seed):
        reqs[key] = tokens_for(folder, dtype, n, seed, vocab)
        at = 0
        for j, m in enumerate(portions):
            steps.append(([(key, reqs[key][at: at + m])], [key] if j == len(portions) - 1 else []))
            at += m
        assert at == n
    feed("whole", 50, [50], 1)
    feed("tail", 70, [30] + [1] * 40, 2)
    feed("cut", 61, [7, 2, 16, 3, 2, 9, 2, 11, 5, 4], 3)
    mixed = {f"m{i}": tokens_for(folder, dtype, n, 40 + i, vocab) for i, n in enumerate([23, 41, 9, 30, 17, 2, 36, 12, 40])}
    reqs.update(mixed)
    steps.extend(mixed_trace(random.Random(5), mixed))
    lines = [json.dumps({"step": i, "entries": [{"id": k, "tokens": t, "want": list(range(len(t)))} for k, t in entries],
                         "end": ended}) for i, (entries, ended) in enumerate(steps)]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                           "--max-tokens", "256"], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(steps))]
    rows = {k: [] for k in reqs}
    for i, (entries, _) in enumerate(steps):
        arr = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(sum(len(t) for _, t in entries), vocab))
        at = 0
        for k, t in entries:
            rows[k].append(arr[at: at + len(t)])
            at += len(t)
    assert sum(len(t) for t in reqs.values()) > 256          # pages went from request to request
    pairs = [zm.kept_rows(torch.cat(rows[k]), folder, t, dtype, f"trace request {k}") for k, t in reqs.items()]
    zm.assert_close_but_few(torch.cat([g for g, _ in pairs]), torch.cat([w for _, w in pairs]), dtype, "all requests of the traces")
