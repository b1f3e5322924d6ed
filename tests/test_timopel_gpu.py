"""The Timopel decoder through the engine against the plain implementation, float32 and bfloat16:
whole prompts and first tokens; prompt then token by token; portions down to two tokens; unequal requests
in one batch against each alone, with pages and slots that are freed and used again; a far key among
hundreds, at page borders, in prompts and in decoding; positions just before and at a temperature step; a
sink that outweighs the keys; long decoding; greedy generation through the scheduler; the trace runner as a
program; and the kernels alone."""
from __future__ import annotations

import math
import random

import pytest
import torch

from tests import timopel_models as tm
from tests.plain import timopel_plain as tp

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
NAMES = ["TA", "TB", "TC", "TD", "TE"]


def tokens_for(n, seed, vocab, folder=None, dtype="float32"):
    """Random tokens; for a comparison in bfloat16 of a model with routers (`folder` given), tokens whose routing
    decisions are all clear in the plain model, so that the comparison does not rest on a close call."""
    if folder is not None and dtype == "bfloat16":
        return tm.clear_tokens(folder, n, seed, vocab)
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts_and_first_tokens(tmp_path, name, dtype):
    folder = tm.make_folder(tmp_path, name)
    engine = tm.engine_for(folder, dtype)
    vocab = tm.MODELS[name][0].vocab
    for n in (1, 2, 3, 5, 61):
        tokens = tokens_for(n, 100 + n, vocab, folder, dtype)
        got = tm.run_portions(engine, f"r{n}", tokens, [n])
        tm.assert_matches_plain(got, folder, tokens, dtype, f"{name} whole {n}")
    engine.runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_token_by_token(tmp_path, name, dtype):
    folder = tm.make_folder(tmp_path, name)
    engine = tm.engine_for(folder, dtype)
    vocab = tm.MODELS[name][0].vocab
    tokens = tokens_for(84, 7, vocab, folder, dtype)
    got = tm.run_portions(engine, "r", tokens, [84 - 45] + [1] * 45)     # temperature steps pass under decoded tokens
    tm.assert_matches_plain(got, folder, tokens, dtype, f"{name} prompt + 45 single tokens")
    got = tm.run_portions(engine, "s", tokens[:30], [1] * 30)             # from the very first token on
    tm.assert_matches_plain(got, folder, tokens, dtype, f"{name} token by token from the start", rows=slice(0, 30))
    if dtype == "float32":
        whole = tm.run_portions(engine, "w", tokens, [84])
        assert tm.row_distance(got, whole[:30]).max().item() <= 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(tmp_path, name, dtype):
    folder = tm.make_folder(tmp_path, name)
    engine = tm.engine_for(folder, dtype)
    vocab = tm.MODELS[name][0].vocab
    tokens = tokens_for(73, 8, vocab, folder, dtype)
    for portions in ([7, 2, 16, 3, 2, 9, 2, 11, 5, 4, 1, 1, 2, 8], [2] * 10 + [53], [1, 3, 69], [40, 33]):
        got = tm.run_portions(engine, "r", tokens, portions)
        tm.assert_matches_plain(got, folder, tokens, dtype, f"{name} portions {portions}")


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
    folder = tm.make_folder(tmp_path, name)
    lengths = [23, 41, 9, 30, 17, 2, 36, 1, 40, 28, 33, 5]
    # four live requests of at most 41 tokens: pool and slots are far fewer than the requests need together
    engine = tm.engine_for(folder, dtype, num_pages=4 * 11 + 1, page_size=4, max_requests=4)
    vocab = tm.MODELS[name][0].vocab
    reqs = {f"q{i}": tokens_for(n, 300 + i, vocab, folder, dtype) for i, n in enumerate(lengths)}
    steps = mixed_trace(random.Random(13), reqs)
    rows = {k: [] for k in reqs}
    slots_seen, pages_seen = {}, {}
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
            for page in engine.runner.cache.block_table(k, 0):
                pages_seen.setdefault(page, set()).add(k)
        for k in ended:
            engine.runner.release(k)
        engine.runner.cache.check_invariants()
    assert any(len(v) > 1 for v in slots_seen.values()), "no slot was used twice"
    assert any(len(v) > 1 for v in pages_seen.values()), "no page went from one request to another"
    for k, toks in reqs.items():
        tm.assert_matches_plain(torch.cat(rows[k]), folder, toks, dtype, f"{name} request {k} in the mix")


def one_layer_model(tmp_path, name, heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, temp=None, seed=11, vocab=90):
    from serve_amd.config.timopel import TimopelConfig, TimopelLayerConfig
    cfg = TimopelConfig(vocab=vocab, width=64, eps=1e-5, residual_mult=1.0, embedding_scale=1.0, layers=(
        TimopelLayerConfig(tm._att(heads, kv_heads, dim, vdim, scale, temp), None),))
    return tm.make_folder(tmp_path, name, config=cfg, seed=seed)


def far_key_model(tmp_path):
    """One attention layer and an embedding table made so that one score stands out: the row of token 1 is set
    so that, behind the layer's first norm and its query matrix, the queries of both heads point along the
    normed key of token 0.  A sequence that ends in token 1 and holds token 0 once, far back, then reads that
    one key with nearly all of its weight (its score is about 16 times the scale, the others' are spread by 4 times
    the scale around zero)."""
    import os
    from safetensors.torch import save_file
    folder = one_layer_model(tmp_path, "far", scale=2.5)
    W = {k: v.double() for k, v in tm.plain_weights(folder).items()}
    h0 = tp.rms_norm(W["embed"][0:1], W["l0.norm1"], 1e-5)
    k0 = tp.rms_norm((h0 @ W["l0.mix.k"].T).view(1, 1, 16), W["l0.mix.k.norm"], 1e-5)[0, 0]
    # h1 with W_q h1 = [k0 | k0] (per head), then the table's row as the normed stream's pre-image
    want_q = torch.cat([k0 / W["l0.mix.q.norm"]] * 2)
    h1 = torch.linalg.pinv(W["l0.mix.q"]) @ want_q
    row = h1 / W["l0.norm1"]
    out = tm.plain_weights(folder)
    out["embed"][1] = (row / row.pow(2).mean().sqrt()).to(out["embed"].dtype)
    save_file({k: v.contiguous() for k, v in out.items()}, os.path.join(folder, "model.safetensors"))
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
        want = tm.plain_logits(folder, with_key)[-1:]
        # losing that one key would move the last row by far more than the tolerance
        assert tm.row_distance(tm.plain_logits(folder, without)[-1:], want).item() > 2 * tm.TOLERANCE["bfloat16"]
        engine = tm.engine_for(folder, dtype, num_pages=120, page_size=4)
        got = tm.run_portions(engine, "r", with_key, [n - 3, 1, 1, 1])[-1:]
        tm.assert_rows_close(got, want, dtype, f"key {far} of {n}, read by a token decoded alone")
        got = tm.run_portions(engine, "r", with_key, [200, 220])[-1:]
        tm.assert_rows_close(got, want, dtype, f"key {far} of {n}, read from a portion")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_sink_that_outweighs_the_keys(tmp_path, dtype):
    """Sinks of +8 and -6 in the two heads of one layer: the first head's output nearly vanishes, the second
    head's does not feel its sink; without the sinks the logits are far away (the plain model says so)."""
    import os
    from safetensors.torch import save_file
    folder = one_layer_model(tmp_path, "sink", scale=0.3, temp=(0.1, 4))
    W = tm.plain_weights(folder)
    W["l0.mix.sink"] = torch.tensor([8.0, -6.0]).to(W["l0.mix.sink"].dtype)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    tokens = tokens_for(150, 3, 90)
    want = tm.plain_logits(folder, tokens)
    none = dict(W)
    none["l0.mix.sink"] = torch.tensor([-1e4, -1e4])
    moved = tm.row_distance(tm.plain_logits(folder, tokens, weights=none), want) > 2 * tm.TOLERANCE["bfloat16"]
    assert moved[:20].all() and moved.float().mean() > 0.8
    engine = tm.engine_for(folder, dtype, num_pages=80, page_size=4)
    for portions in ([150], [100] + [1] * 50, [3, 2, 60, 85]):
        tm.assert_rows_close(tm.run_portions(engine, "r", tokens, portions), want, dtype, f"sinks, portions {portions[:4]}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_temperature_steps_in_prompts_and_in_decoding(tmp_path, dtype):
    """A strong temperature (coef 3) that steps every 6 positions: portions that end just before, at and just
    behind a step, and single tokens across steps.  A step that came one position late would show."""
    import copy
    folder = one_layer_model(tmp_path, "temp", scale=0.5, temp=(3.0, 6), seed=12)
    tokens = tokens_for(40, 9, 90)
    want = tm.plain_logits(folder, tokens)
    late = copy.deepcopy(tm.plain_config(folder))
    late["layers"][0]["mixer"]["q_temp"]["every"] = 7
    moved = tm.row_distance(tm.plain_logits(folder, tokens, late), want)
    # (positions 5 and 11 are the first whose count of steps differs between the two)
    assert moved[:5].max().item() == 0.0 and moved[5] > 2 * tm.TOLERANCE["bfloat16"] and moved[11] > 100 * tm.TOLERANCE["float32"]
    engine = tm.engine_for(folder, dtype, page_size=4)
    for portions in ([40], [4, 1, 1, 1, 4, 1, 1, 1, 26], [5, 6, 6, 7] + [1] * 16, [1] * 40):
        tm.assert_rows_close(tm.run_portions(engine, "r", tokens, portions), want, dtype, f"temperature, portions {portions[:5]}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["TA", "TB"])
def test_long_decoding(tmp_path, name, dtype):
    folder = tm.make_folder(tmp_path, name)
    engine = tm.engine_for(folder, dtype, num_pages=80)
    vocab = tm.MODELS[name][0].vocab
    tokens = tokens_for(260, 31, vocab, folder, dtype)
    got = tm.run_portions(engine, "r", tokens, [4] + [1] * 256)
    tm.assert_matches_plain(got, folder, tokens, dtype, f"{name} 256 single tokens")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["TA", "TB"])
def test_greedy_generation_through_the_scheduler(tmp_path, name, dtype):
    """`generate` (scheduler, mixed steps, graphs, steps launched ahead of the host) picks the tokens the
    plain model picks, as long as the plain model's choice is clear."""
    from serve_amd.engine.engine import Request
    folder = tm.make_folder(tmp_path, name)
    engine = tm.engine_for(folder, dtype, num_pages=128, page_size=8, max_requests=3)
    vocab = tm.MODELS[name][0].vocab
    prompts = [tokens_for(n, 50 + n, vocab, folder, dtype) for n in (5, 19, 1, 33, 8)]
    new = 12
    reqs = [Request(torch.tensor(p), len(p), new) for p in prompts]
    out = engine.generate(reqs, temperature=0.0, return_logits="all")
    compared = 0
    for p, o in zip(prompts, out):
        assert o.error is None and len(o.generated_tokens) == new
        seq = list(p)
        for i, tok in enumerate(o.generated_tokens.tolist()):
            row = tm.plain_logits(folder, seq)[-1]
            top2 = row.topk(2).values
            if (top2[0] - top2[1]).item() < (1e-3 if dtype == "float32" else 0.15):
                break                            # the plain model's own choice is a close call: stop comparing
            assert tok == int(row.argmax()), f"{name}: token {i} after a prompt of {len(p)}"
            if dtype == "float32":
                tm.assert_rows_close(o.logits[i: i + 1], row[None], dtype, f"{name} logits of generated token {i}")
            seq.append(tok)
            compared += 1
    assert compared >= new
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.free_slots() == 3
    # without the logits the scheduler samples on the device and replays decode steps from graphs: the same tokens
    again = engine.generate([Request(torch.tensor(p), len(p), new) for p in prompts], temperature=0.0)
    if dtype == "float32":
        assert [o.generated_tokens.tolist() for o in again] == [o.generated_tokens.tolist() for o in out]


# ---------------------------------------------------------------------------------------------
# the kernels alone
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pad", [5, 8])      # rows that do not keep 16-byte alignment (the general kernel), and rows that do
@pytest.mark.parametrize("H,G,D,Dv,Dp", [(4, 2, 16, 16, 16), (6, 1, 24, 40, 48), (3, 3, 10, 7, 16), (2, 1, 136, 24, 144),
                                         (5, 5, 128, 64, 128)])
def test_qk_norm_kv_write(dtype, H, G, D, Dv, Dp, pad):
    from serve_amd import ops
    torch.manual_seed(D)
    T, page, P = 11, 4, 9
    width = H * D + G * (D + Dv)
    wide = torch.randn(T, width + pad, device="cuda").to(dtype)             # rows inside wider rows
    qkv = wide[:, :width]
    first = torch.randn(T, G * Dv + pad, device="cuda").to(dtype)[:, : G * Dv]
    wq, wk = torch.rand(D, device="cuda") + 0.5, torch.rand(D, device="cuda") + 0.5
    positions = torch.tensor([0, 1, 2, 3, 4, 5, 6, 7, 30, 31, 32], dtype=torch.int32, device="cuda")
    slots = torch.tensor([5, 6, 7, 8, 20, 21, 22, 23, -1, 1, 35], dtype=torch.int32, device="cuda")
    k_pages = torch.full((P, G, page, Dp), 7.0, device="cuda").to(dtype)
    v_pages = torch.full((P, G, Dp, page), 7.0, device="cuda").to(dtype)
    q = torch.full((T, H * Dp), 7.0, device="cuda").to(dtype)
    eps, coef, every, lam = 1e-5, 0.6, 4, 0.3
    ops.qk_norm_kv_write(qkv, q, positions, slots, k_pages, v_pages, wq, wk, eps, H, G, D, Dv, coef, every, first, lam)
    x = qkv.double().cpu()
    temp = tp.query_temperature(positions.cpu().long(), coef, every)
    want_q = tp.rms_norm(x[:, : H * D].view(T, H, D), wq.double().cpu(), eps) * temp[:, None, None]
    want_k = tp.rms_norm(x[:, H * D: (H + G) * D].view(T, G, D), wk.double().cpu(), eps)
    want_v = (1 - lam) * x[:, (H + G) * D:].view(T, G, Dv) + lam * first.double().cpu().view(T, G, Dv)
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
    got_q = q.double().cpu().view(T, H, Dp)
    assert torch.allclose(got_q[:, :, :D], want_q, **tol) and (got_q[:, :, D:] == 0).all()
    kp, vp = k_pages.double().cpu(), v_pages.double().cpu()
    written = set()
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        pg, off = divmod(s, page)
        written.add((pg, off))
        assert torch.allclose(kp[pg, :, off, :D], want_k[t], **tol) and (kp[pg, :, off, D:] == 0).all()
        assert torch.allclose(vp[pg, :, :Dv, off], want_v[t], **tol) and (vp[pg, :, Dv:, off] == 0).all()
    for pg in range(P):
        for off in range(page):
            if (pg, off) not in written:
                assert (kp[pg, :, off] == 7.0).all() and (vp[pg, :, :, off] == 7.0).all(), "a slot that no token named was written"
    # queries alone (no slots), no temperature, no blending
    q2 = torch.empty_like(q)
    ops.qk_norm_kv_write(qkv, q2, positions, None, None, None, wq, wk, eps, H, G, D, Dv)
    assert torch.allclose(q2.double().cpu().view(T, H, Dp)[:, :, :D], want_q / temp[:, None, None], **tol)


def _attention_case(dtype, H, G, D, page, lens, ctxs, seed=0):
    """Random pages and block tables for segments of `lens` tokens that end contexts of `ctxs` tokens."""
    from serve_amd.ops import AttentionStep
    torch.manual_seed(seed)
    B, T = len(lens), sum(lens)
    per = [-(-c // page) for c in ctxs]
    P = sum(per) + 3
    order = torch.randperm(P - 1)[: sum(per)] + 1          # (page 0 stays unused)
    bt = torch.zeros(B, max(per), dtype=torch.int32)
    at = 0
    for b in range(B):
        bt[b, : per[b]] = order[at: at + per[b]].int()
        at += per[b]
    k_pages = torch.randn(P, G, page, D)
    v_pages = torch.randn(P, G, D, page)
    q = torch.randn(T, H * D)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    seg = [b for b, n in enumerate(lens) for _ in range(n)]
    dev = lambda t, dt=None: (t.to(dt) if dt else t).cuda().contiguous()   # noqa: E731
    step = AttentionStep(num_segments=B, num_tokens=T, cu_q=dev(torch.tensor(cu, dtype=torch.int32)),
                         ctx_len=dev(torch.tensor(ctxs, dtype=torch.int32)), seg_of_token=dev(torch.tensor(seg, dtype=torch.int32)),
                         q_lens=list(lens), ctx_lens=list(ctxs), max_q_len=max(lens), max_ctx_len=max(ctxs),
                         decode_only=all(n == 1 for n in lens))
    q, k_pages, v_pages = q.to(dtype), k_pages.to(dtype), v_pages.to(dtype)       # (the reference reads the rounded values)
    return step, dev(q), dev(k_pages), dev(v_pages), dev(bt), (q.double(), k_pages.double(), v_pages.double(), bt, cu)


def _attention_reference(host, lens, ctxs, H, G, D, page, scale, sinks):
    q, kp, vp, bt, cu = host
    out = torch.zeros(q.shape[0], H, D, dtype=torch.float64)
    for b, (n, c) in enumerate(zip(lens, ctxs)):
        pages = bt[b, : -(-c // page)].long()
        for h in range(H):
            g = h // (H // G)
            keys = kp[pages, g].reshape(-1, D)[:c]
            vals = vp[pages, g].permute(0, 2, 1).reshape(-1, D)[:c]
            for j in range(n):
                pos = c - n + j
                s = (keys[: pos + 1] @ q[cu[b] + j].view(H, D)[h]) * scale
                sink = torch.tensor(-math.inf if sinks is None else float(sinks[h]), dtype=torch.float64)
                out[cu[b] + j, h] = tp.sink_softmax(s[None], sink[None])[0] @ vals[: pos + 1]
    return out.view(q.shape[0], H * D)


ATTENTION_CASES = [
    # (heads, kv heads, head size, page size, portion lengths, contexts)
    (4, 2, 32, 8, [1, 1, 1], [5, 300, 64]),                    # single tokens, short contexts: keys cut inside a workgroup
    (8, 1, 64, 16, [1] * 5, [1500, 900, 2200, 33, 700]),       # single tokens over long contexts: keys cut over the grid
    (6, 3, 48, 4, [40, 7, 130], [40, 90, 130]),                # prompt portions, whole prompts among them
    (2, 1, 16, 16, [20], [2100]),                              # a short portion of a long context: its keys cut over the grid
    (4, 1, 128, 8, [1, 1, 1, 1, 33, 2], [9, 70, 200, 64, 33, 58]),   # single tokens first, then portions: two launches
    (3, 3, 144, 4, [1, 9], [37, 9]),                           # a head size only the general kernel takes
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", range(len(ATTENTION_CASES)))
def test_attention_kernels_with_sinks(dtype, case):
    """Every family of attention kernels with a sink in each head's softmax, against the plain softmax with one
    more term in its denominator; sinks far below the scores change nothing; no sinks: the kernels as before."""
    from serve_amd import ops
    H, G, D, page, lens, ctxs = ATTENTION_CASES[case]
    step, q, k_pages, v_pages, bt, host = _attention_case(dtype, H, G, D, page, lens, ctxs, seed=case)
    scale = 0.5 / math.sqrt(D)
    sinks = torch.linspace(-2.0, 3.0, H)
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    for s in (sinks, None, torch.full((H,), -80.0)):
        out = torch.empty(q.shape[0], H * D, dtype=dtype, device="cuda")
        ops.paged_attention(q, H * D, out, k_pages, v_pages, bt, step, H, scale, None,
                            None if s is None else s.float().cuda())
        want = _attention_reference(host, lens, ctxs, H, G, D, page, scale, None if s is None or s[0] < -50 else s)
        got = out.double().cpu()
        assert torch.allclose(got, want, **tol), f"sinks {None if s is None else s.tolist()}: max diff {(got - want).abs().max():.3g}"


@pytest.mark.parametrize("experts,top", [(5, 1), (16, 2), (70, 3), (130, 8), (4, 4)])
def test_route_over_all_experts(experts, top):
    from serve_amd import ops
    torch.manual_seed(experts)
    T = 37
    logits = (torch.randn(T, experts + 1, device="cuda") * 3).contiguous()
    ids = torch.empty(T, top, dtype=torch.int32, device="cuda")
    w = torch.empty(T, top, dtype=torch.float32, device="cuda")
    ops.moe_route(logits, experts, top, ids, w, over_all=True, scale=2.5)
    want_ids, want_w = tp.route(logits[:, :experts].double().cpu(), top, 2.5)
    assert torch.equal(ids.long().cpu(), want_ids)
    assert torch.allclose(w.double().cpu(), want_w, atol=1e-6, rtol=1e-5)
    # the experts' call routes by itself for few tokens: the same ids and weights
    d, F = 32, 16
    h = torch.randn(9, d, device="cuda")
    wg, wu, wd = torch.randn(experts, F, d, device="cuda"), torch.randn(experts, F, d, device="cuda"), torch.randn(experts, d, F, device="cuda")
    ids2, w2 = torch.empty(9, top, dtype=torch.int32, device="cuda"), torch.empty(9, top, device="cuda")
    ops.moe_experts(h, ids2, wg, wu, wd, torch.empty(9 * top, d, device="cuda"), logits[:9].contiguous(), w2,
                    over_all=True, scale=2.5, gate="clamped_swish", limit=1.0)
    assert torch.equal(ids2, ids[:9]) and torch.equal(w2, w[:9])


@pytest.mark.parametrize("T,d,F", [(45, 72, 40), (45, 75, 42), (400, 64, 48)])   # few rows; sizes the matrix cores do not take; many rows
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_experts_with_clamped_gates(dtype, T, d, F):
    from serve_amd import ops
    torch.manual_seed(3)
    E, top, limit = 7, 3, 0.8
    h = torch.randn(T, d, device="cuda").to(dtype)
    wg, wu = (torch.randn(E, F, d, device="cuda") * 0.2).to(dtype), (torch.randn(E, F, d, device="cuda") * 0.2).to(dtype)
    wd = (torch.randn(E, d, F, device="cuda") * 0.2).to(dtype)
    ids = torch.stack([torch.randperm(E, device="cuda")[:top] for _ in range(T)]).int().contiguous()
    yk = torch.empty(T * top, d, dtype=torch.float32, device="cuda")
    ops.moe_experts(h, ids, wg, wu, wd, yk, gate="clamped_swish", limit=limit)
    hd = h.double().cpu()
    clipped = 0
    for t in list(range(0, T, 7)) + [T - 1]:
        for k in range(top):
            e = int(ids[t, k])
            g, u = hd[t] @ wg[e].double().cpu().t(), hd[t] @ wu[e].double().cpu().t()
            clipped += int((g > limit).sum() + (u.abs() > limit).sum())
            a = tp.clamped_swish_gate(g, u, limit)
            if dtype == torch.bfloat16:
                a = a.to(dtype).double()
            want = a @ wd[e].double().cpu().t()
            assert torch.allclose(yk[t * top + k].double().cpu(), want, atol=2e-4 if dtype == torch.float32 else 2e-2, rtol=1e-3)
    assert clipped > 20, "the limit was hardly reached: the test shows nothing"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind,limit", [("silu", 0.0), ("gelu_tanh", 0.0), ("clamped_swish", 0.7)])
def test_gates(dtype, kind, limit):
    from serve_amd import ops
    torch.manual_seed(1)
    for T, I in ((5, 24), (3, 37)):                  # whole groups of eight, and not
        gu = (torch.randn(T, 2 * I, device="cuda") * 2).to(dtype)
        out = torch.empty(T, I, device="cuda", dtype=dtype)
        ops.gate_mul(gu, out, kind, limit)
        g, u = gu.double().cpu()[:, :I], gu.double().cpu()[:, I:]
        want = {"silu": lambda: g * torch.sigmoid(g) * u, "gelu_tanh": lambda: tp.gelu_tanh(g) * u,
                "clamped_swish": lambda: tp.clamped_swish_gate(g, u, limit)}[kind]()
        assert torch.allclose(out.double().cpu(), want, atol=1e-5 if dtype == torch.float32 else 3e-2, rtol=1e-5 if dtype == torch.float32 else 1e-2)


def test_scaled_embedding_rows():
    from serve_amd import ops
    torch.manual_seed(2)
    for d, dt in ((64, torch.bfloat16), (50, torch.bfloat16), (50, torch.float32)):
        table = torch.randn(20, d, device="cuda").to(dt)
        ids = torch.tensor([3, 19, 0, 3], dtype=torch.int32, device="cuda")
        x = torch.empty(4, d, dtype=torch.float32, device="cuda")
        ops.embed(table, ids, x, scale=2.75)
        assert torch.equal(x, table[ids.long()].float() * 2.75)


# ---------------------------------------------------------------------------------------------
# the trace runner as a user runs it
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_traces_through_the_program(tmp_path, dtype):
    """`bin/trace_run` as a child process on a model folder: whole prompts, prompt then single tokens, portions, and
    a mix of four live requests (pages for 256 tokens, so pages go from request to request), against the plain model."""
    import json
    import os
    import subprocess
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    name = "TA"
    folder = tm.make_folder(tmp_path, name)
    vocab = tm.MODELS[name][0].vocab
    reqs, steps = {}, []

    def feed(key, n, portions, seed):
        reqs[key] = tokens_for(n, seed, vocab, folder, dtype)
        at = 0
        for j, m in enumerate(portions):
            steps.append(([(key, reqs[key][at: at + m])], [key] if j == len(portions) - 1 else []))
            at += m
        assert at == n
    feed("whole", 50, [50], 1)
    feed("tail", 70, [30] + [1] * 40, 2)
    feed("cut", 61, [7, 2, 16, 3, 2, 9, 2, 11, 5, 4], 3)
    mixed = {f"m{i}": tokens_for(n, 40 + i, vocab, folder, dtype) for i, n in enumerate([23, 41, 9, 30, 17, 2, 36, 12, 40])}
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
    for k, t in reqs.items():
        tm.assert_matches_plain(torch.cat(rows[k]), folder, t, dtype, f"trace request {k}")


def test_generate_from_the_command_line():
    """`python -m serve_amd generate` with the named shape: as many token lists as prompts, of the asked length."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-m", "serve_amd", "generate", "--shape", "timopel-tiny", "--random-prompts", "3:20",
                           "--max-new-tokens", "6", "--temperature", "0"], cwd=root, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 3 and all(len(l) == 6 and all(0 <= t < 512 for t in l) for l in lines)


@pytest.mark.parametrize("dtype", DTYPES)
def test_steps_with_prompt_portions_replayed_from_graphs(tmp_path, dtype):
    """Six slots and portions of eight tokens: steps of a few decoding requests in front of prompt portions come
    again and again, are padded with inert segments (no pages, no slot: nothing of them is stored) and replayed from
    graphs; the greedy tokens are those of the same schedule launched kernel by kernel, and the plain model's where
    its choice is clear."""
    from serve_amd.engine.engine import Request
    name = "TA"
    folder = tm.make_folder(tmp_path, name)
    vocab = tm.MODELS[name][0].vocab
    rng = random.Random(46)
    count = 30
    prompts = [tokens_for(rng.randrange(9, 30), 700 + i, vocab, folder, dtype) for i in range(count)]
    new = [rng.randrange(4, 12) for _ in range(count)]
    kw = dict(num_pages=64, page_size=8, max_requests=6)
    outs = []
    for mixed in (True, False):
        from serve_amd.config.engine import EngineConfig
        from serve_amd.engine.engine import Engine
        engine = Engine.from_folder(folder, EngineConfig(dtype=dtype, max_context=256, max_tokens_per_step=24, prefill_chunk=8,
                                                         graph_mixed_steps=mixed, **kw))
        out = engine.generate([Request(torch.tensor(p), len(p), n) for p, n in zip(prompts, new)], temperature=0.0)
        assert all(r.error is None and len(r.generated_tokens) == n for r, n in zip(out, new))
        graphs = [k for k, e in engine.runner._graphs.items() if k[0] == "mixed" and e.graph is not None and e.launches > 2]
        assert bool(graphs) == mixed, f"mixed graphs {mixed}: replayed shapes {graphs}"
        engine.runner.cache.check_invariants()
        outs.append([r.generated_tokens.tolist() for r in out])
    if dtype == "float32":
        assert outs[0] == outs[1]
    compared = 0
    for p, got in zip(prompts, outs[0]):
        seq = list(p)
        for tok in got:
            row = tm.plain_logits(folder, seq)[-1]
            top2 = row.topk(2).values
            if (top2[0] - top2[1]).item() < (1e-3 if dtype == "float32" else 0.15):
                break
            assert tok == int(row.argmax())
            seq.append(tok)
            compared += 1
    assert compared > 3 * count


@pytest.mark.parametrize("gate,limit", [("silu", 0.0), ("clamped_swish", 0.8)])
@pytest.mark.parametrize("T,d,F,E,top", [(700, 128, 192, 5, 2), (300, 64, 64, 9, 4), (2048, 256, 128, 6, 1)])
def test_experts_of_many_rows_with_both_operands_through_lds(T, d, F, E, top, gate, limit):
    """More than 1,024 (token, k) rows in bf16 with widths that are multiples of 64 and the gates' and ups' matrices in
    one tensor: tiles of 128 grouped rows; experts with no row, with a few, and with several tiles of rows."""
    from serve_amd import ops
    torch.manual_seed(T + E)
    h = torch.randn(T, d, device="cuda").bfloat16()
    wgu = (torch.randn(2, E, F, d, device="cuda") * 0.1).bfloat16()
    wd = (torch.randn(E, d, F, device="cuda") * 0.1).bfloat16()
    assert T * top > ops.MOE_WIDE_MIN_ROWS and ops.moe_wide_available(h, wgu[0], wgu[1], wd)
    ids = torch.stack([torch.randperm(E, device="cuda")[:top] for _ in range(T)]).int().contiguous()
    if top < E:
        ids[ids == E - 1] = 0 if top == 1 else ids[ids == E - 1]          # (top 1: the last expert gets no row at all)
    ids[: T // 2, 0] = ids[0, 0]                                          # one expert with many tiles of rows
    if top > 1:
        ids[: T // 2, 1:] = ids[0, 1:]
    yk = torch.full((T * top, d), float("nan"), dtype=torch.float32, device="cuda")
    ops.moe_experts(h, ids, wgu[0], wgu[1], wd, yk, gate=gate, limit=limit)
    assert torch.isfinite(yk).all(), "a row was not written"
    # the same through the kernels for few rows, slice by slice
    ref = torch.empty_like(yk)
    for t0 in range(0, T, 200):
        n = min(200, T - t0)
        ops.moe_experts(h[t0: t0 + n].contiguous(), ids[t0: t0 + n].contiguous(), wgu[0], wgu[1], wd,
                        ref[t0 * top: (t0 + n) * top], gate=gate, limit=limit)
    assert torch.allclose(yk, ref, atol=2e-2, rtol=2e-2), f"max diff {(yk - ref).abs().max().item():.3g}"
    hd = h.double().cpu()
    for t in (0, 1, T // 2 - 1, T // 2, T - 1):
        for k in range(top):
            e = int(ids[t, k])
            g, u = hd[t] @ wgu[0, e].double().cpu().t(), hd[t] @ wgu[1, e].double().cpu().t()
            a = (tp.clamped_swish_gate(g, u, limit) if gate == "clamped_swish" else g * torch.sigmoid(g) * u).bfloat16().double()
            want = a @ wd[e].double().cpu().t()
            assert torch.allclose(yk[t * top + k].double().cpu(), want, atol=2e-2, rtol=1e-2)
