"""Karopel through the engine against the plain float64 implementation (plain_karopel.py): every mechanism alone at
the level of its kernels or as a one-layer model, then whole models of made-up sizes in every way of cutting and
batching, 32-bit and bfloat16, and greedy generation through the engine's own entry point."""
import json
import math
import random

import pytest
import torch

import plain_karopel as plain

pytestmark = pytest.mark.gpu
F = torch.float64

BANDS = dict(factor=4.0, low=1.0, high=3.0, original=24)


def attention(heads, kv_heads, dim, vdim, size, keep_first, dims=None, base=10000.0, scaling=None, scale=None):
    rot = dict(base=base, dims=dim if dims is None else dims, scaling=scaling)
    return dict(type="attention", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale or dim ** -0.5,
                                             mask=dict(size=size, keep_first=keep_first), rot=rot))


def parallel(lh, lg, ld, size, rh, rg, rd, rv, conv, ls, rs, scale=None):
    return dict(type="parallel", mixer=dict(
        left=dict(heads=lh, kv_heads=lg, dim=ld, vdim=ld, scale=scale or ld ** -0.5, mask=dict(size=size)),
        right=dict(heads=rh, kv_heads=rg, dim=rd, vdim=rv, conv=conv), left_scale=ls, right_scale=rs))


def with_mlp(layer, ff):
    return dict(layer, mlp=None if ff is None else dict(kind="dense", ff=ff))


def model(vocab, width, layers, loop=None, mult=0.5, logit_scale=1.0, eps=1e-6):
    return dict(architecture="Karopel", vocab=vocab, width=width, residual_mult=mult, logit_scale=logit_scale,
                norm=dict(eps=eps), loop=loop, layers=layers)


A1 = attention(4, 2, 16, 24, size=10, keep_first=3, dims=8, scaling=BANDS)           # values wider than keys, half rotated
P1 = parallel(4, 1, 16, 7, 4, 2, 16, 8, 3, 0.7, 0.45)
A2 = attention(3, 3, 40, 40, size=33, keep_first=0, base=300.0)                      # nothing kept, no scaling, odd head count
P2 = parallel(2, 2, 24, 40, 3, 3, 40, 48, 2, 1.0, 1.0)                               # scales of one, two taps
A3 = attention(8, 1, 32, 16, size=5, keep_first=7, scaling=dict(factor=6.0, low=0.5, high=2.0, original=16))   # keeps more than it sees
P3 = parallel(6, 3, 8, 3, 2, 1, 64, 32, 4, 0.25, 2.0)
A4 = attention(4, 2, 32, 32, size=24, keep_first=5, dims=16, scaling=BANDS)          # sizes the matrix-core kernel takes
P4 = parallel(2, 1, 64, 9, 2, 1, 32, 32, 4, 0.7, 0.4)
A5 = attention(2, 1, 20, 28, size=11, keep_first=2, dims=10)                         # head sizes that are no multiples of 8
P5 = parallel(3, 3, 12, 6, 2, 2, 20, 10, 3, 0.8, 0.9)

CONFIGS = {
    # layers 1 and 2 run three times; a layer without feed-forward; pages of 4
    "C1": (model(96, 64, [with_mlp(P1, 48), with_mlp(A1, 80), with_mlp(A1, None), with_mlp(P1, 56)],
                 loop=dict(start=1, stop=3, times=3)), 4, 11),
    # no loop, logits scaled, another eps
    "C2": (model(131, 72, [with_mlp(A2, 64), with_mlp(P2, 40), with_mlp(A2, 88)], mult=1.0, logit_scale=1.7, eps=1e-3), 8, 12),
    # the whole model is one pass run twice, starting with a parallel layer; one tap would be no convolution: four
    "C3": (model(80, 48, [with_mlp(P3, 32), with_mlp(A3, 64)], loop=dict(start=0, stop=2, times=2), mult=0.35, logit_scale=0.5), 16, 13),
    # bfloat16: both attentions on the matrix cores (heads of 32 and 64, pages of 8), the parallel layer looped
    "C4": (model(120, 64, [with_mlp(A4, 96), with_mlp(P4, 64), with_mlp(A4, None)], loop=dict(start=1, stop=2, times=2),
                 mult=0.4, logit_scale=1.3), 8, 14),
    "C5": (model(77, 40, [with_mlp(A5, 56), with_mlp(P5, 24)], mult=0.6), 4, 15),
}
# one mechanism a model
ONE = {
    "attention": (model(64, 32, [with_mlp(A1, None)]), 4, 21),
    "left": (model(64, 32, [with_mlp(parallel(4, 2, 16, 6, 2, 1, 8, 8, 2, 1.0, 0.0), None)]), 4, 22),
    "right": (model(64, 32, [with_mlp(parallel(2, 1, 8, 6, 4, 2, 16, 24, 4, 0.0, 1.0), None)]), 4, 23),
    "feed_forward": (model(64, 32, [with_mlp(parallel(2, 1, 8, 6, 2, 1, 8, 8, 2, 0.0, 0.0), 72)]), 4, 24),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    from dinfer_amd.weights.safetensors_io import write_safetensors
    out = {}
    for name, (cfg, page, seed) in {**CONFIGS, **ONE}.items():
        d = tmp_path_factory.mktemp(f"karopel_{name}")
        w = plain.random_weights(cfg, seed)
        (d / "config.json").write_text(json.dumps(cfg))
        write_safetensors(d / "model.safetensors", w, metadata={"format": "pt"})
        out[name] = (d, cfg, plain.as_float64(w), page)
    return out


def make_runner(models, name, dtype, max_tokens=512, num_blocks=160, max_seqs=4, max_len=512, graph=False):
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.runner import ModelRunner
    d, _, _, page = models[name]
    opt = EngineOptions(dtype=dtype, max_model_len=max_len, max_num_seqs=max_seqs, max_num_batched_tokens=max_tokens,
                        block_size=page, num_blocks=num_blocks, max_logits_rows=max_tokens,
                        decode_exempt_from_budget=False, hip_graph=graph)
    return ModelRunner.from_dir(d, opt)


def tokens_for(cfg, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(cfg["vocab"]) for _ in range(n)]


def check_logits(got, want, dtype, what):
    got = got.double().cpu()
    scale = want.std(dim=-1, keepdim=True)
    err = ((got - want).abs() / scale).max().item()
    rms = ((got - want).pow(2).mean(dim=-1, keepdim=True).sqrt() / scale).max().item()
    if dtype == "float32":
        assert err < 5e-4, f"{what}: 32-bit logits off by {err:.2e} row-sigmas"
    else:
        # roundings to 8 bits through these narrow models add up to a few hundredths of a row's spread; a key too
        # many, a sink left out or a lost state is several times that
        assert err < 0.25 and rms < 0.07, f"{what}: bf16 logits off by {err:.3f} (rms {rms:.4f}) row-sigmas"


def replay(runner, steps):
    """steps: [(entries, ends)], entries [(id, tokens, want)] -> {(id, position): logits row}."""
    from dinfer_amd.engine.batch import Entry
    computed, rows = {}, {}
    for entries, ends in steps:
        es = []
        for rid, toks, want in entries:
            start = computed.get(rid, 0)
            assert runner.reserve(rid, start, len(toks)), f"out of pages for {rid}"
            es.append(Entry(rid, toks, start, want))
        if es:
            logits = runner.step(es).double().cpu()
            i = 0
            for e in es:
                for w in e.want:
                    rows[(e.req_id, e.start + w)] = logits[i]
                    i += 1
                computed[e.req_id] = e.start + len(e.tokens)
                runner.advance(e.req_id, computed[e.req_id])
        for rid in ends:
            runner.finish(rid)
            del computed[rid]
        runner.cache.check()
    return rows


def compare_rows(rows, cfg, w, toks, dtype, what):
    assert rows
    for rid in {k[0] for k in rows}:
        want, _ = plain.forward(toks[rid.split("#")[0]], w, cfg)
        pos = sorted(p for (r, p) in rows if r == rid)
        check_logits(torch.stack([rows[(rid, p)] for p in pos]), want[pos], dtype, f"{what} request {rid}")


def cut(ids, sizes):
    out, i, k = [], 0, 0
    while i < len(ids):
        out.append(ids[i:i + sizes[k % len(sizes)]])
        i += len(out[-1])
        k += 1
    return out


DTYPES = ["float32", "bfloat16"]
NAMES = list(CONFIGS)


# ---- one mechanism a model ------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(ONE))
def test_one_mechanism(models, name, dtype):
    """A model of one layer that is one mechanism (the other half of a parallel layer scaled by zero): a whole prompt,
    the same in portions of two and three, and token by token."""
    _, cfg, w, _ = models[name]
    ids = tokens_for(cfg, 45, 3)
    r = make_runner(models, name, dtype)
    for what, parts in (("whole", [ids]), ("portions", cut(ids, [2, 3])), ("single tokens", [[t] for t in ids])):
        steps = [([("x", p, list(range(len(p))))], []) for p in parts]
        steps[-1] = (steps[-1][0], ["x"])
        compare_rows(replay(r, steps), cfg, w, {"x": ids}, dtype, f"{name} alone, {what}")


# ---- whole models ---------------------------------------------------------------------------------------------
def test_which_attention_kernel_serves_which_model(models):
    """bfloat16 with heads and pages the matrix-core kernel takes: that kernel, and values that are the keys are kept
    in value pages as well; everything else: the plain kernel, keys only."""
    for name, dtype, mfma in (("C4", "bfloat16", True), ("C4", "float32", False), ("C1", "bfloat16", False)):
        r = make_runner(models, name, dtype)
        mixers = [b.mixer for b in r.model.blocks]
        plain_ones = [m for m in mixers if hasattr(m, "mfma_ext")]
        joined = [m for mx in mixers if hasattr(mx, "members") for _, m, _, _ in mx.members if hasattr(m, "mfma_ext")]
        assert plain_ones and joined and all(m.mfma_ext == mfma for m in plain_ones + joined)
        assert all(m.stores_values == mfma for m in joined)
        views = [v for v, b in zip(r.cache_views, [r.model.blocks[e.layer] for e in r.model.run]) if hasattr(b.mixer, "members")]
        assert views and all(("left.v" in v.tensors) == mfma for v in views)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts(models, name, dtype):
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, dtype)
    for n, seed in ((1, 1), (2, 2), (19, 3), (150, 4)):
        ids = tokens_for(cfg, n, seed)
        rows = replay(r, [([("x", ids, list(range(n)))], ["x"])])
        compare_rows(rows, cfg, w, {"x": ids}, dtype, f"{name} whole prompt of {n}")


@pytest.mark.parametrize("name", NAMES)
def test_residual_stream_after_every_layer_run(models, name):
    from dinfer_amd.engine.batch import Entry
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, "float32")
    ids = tokens_for(cfg, 37, 9)
    _, want = plain.forward(ids, w, cfg)
    seen = []
    for block in r.model.blocks:
        inner = block.forward

        def spy(hidden, pending, batch, cache, _inner=inner, **kw):
            out = _inner(hidden, pending, batch, cache, **kw)
            seen.append(hidden[:batch.num_tokens].double().cpu())
            return out
        block.forward = spy
    assert r.reserve("x", 0, len(ids))
    r.step([Entry("x", ids, 0, [0])])
    assert len(seen) == len(want) == len(plain.run_order(cfg))
    for i, (g, x) in enumerate(zip(seen, want)):
        assert (g - x).abs().max().item() < 2e-4 * max(1.0, x.abs().max().item()), f"{name}: the stream after layer run {i} differs"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_long_decoding(models, name, dtype):
    """Decoding far beyond every window of the model, across many pages, from eager steps."""
    _, cfg, w, page = models[name]
    r = make_runner(models, name, dtype)
    ids = tokens_for(cfg, 3 * page + 120, 5)
    first = 3 * page - 1                      # the first decoded token opens a new page
    steps = [([("x", ids[:first], [first - 1])], [])]
    steps += [([("x", [ids[p]], [0])], []) for p in range(first, len(ids))]
    compare_rows(replay(r, steps), cfg, w, {"x": ids}, dtype, f"{name} decode after prompt")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_token_by_token_from_the_first(models, name, dtype):
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, dtype)
    ids = tokens_for(cfg, 60, 6)
    compare_rows(replay(r, [([("x", [t], [0])], []) for t in ids]), cfg, w, {"x": ids}, dtype, f"{name} one token a step")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("sizes", [[2], [7, 16, 2, 5, 3, 33, 2, 8, 1], [64, 3, 31]])
def test_portions(models, name, dtype, sizes):
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, dtype)
    ids = tokens_for(cfg, 131 if sizes != [2] else 48, 7)
    steps = [([("x", part, list(range(len(part))))], []) for part in cut(ids, sizes)]
    compare_rows(replay(r, steps), cfg, w, {"x": ids}, dtype, f"{name} portions of {sizes}")


def test_cuts_leave_the_same_bits_in_32bit(models):
    """32-bit: whole, in portions and token by token, a position's logits are equal to the last bit or two."""
    _, cfg, w, _ = models["C1"]
    ids = tokens_for(cfg, 70, 8)
    got = []
    for parts in ([ids], cut(ids, [5, 2, 11, 1]), [[t] for t in ids]):
        r = make_runner(models, "C1", "float32")
        rows = replay(r, [([("x", p, list(range(len(p))))], []) for p in parts])
        got.append(torch.stack([rows[("x", p)] for p in range(len(ids))]))
    for other in got[1:]:
        assert (other - got[0]).abs().max().item() < 2e-5 * got[0].abs().max().item()


def mixed_schedule(cfg, seed):
    """Four live requests at most: portions of some beside single tokens of others, requests that pause, finish and are
    followed by new ones in their pages and slots."""
    rng = random.Random(seed)
    lens = {"a": 90, "b": 33, "c": 57, "d": 21, "e": 70, "f": 12, "a#2": 90}
    toks = {k: tokens_for(cfg, n, sum(map(ord, k.split("#")[0]))) for k, n in lens.items()}
    order, live, at, steps = list(lens), [], {}, []
    while order or live:
        while order and len(live) < 4:
            k = order.pop(0)
            live.append(k)
            at[k] = 0
        entries, ends = [], []
        for k in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue                                      # left out of this step
            left = lens[k] - at[k]
            n = min(left, rng.choice([1, 1, 1, 2, 3, 9, 17, 40]))
            entries.append((k, toks[k][at[k]:at[k] + n], sorted(rng.sample(range(n), min(n, 3)))))
            at[k] += n
            if at[k] == lens[k]:
                ends.append(k)
                live.remove(k)
        if entries:
            steps.append((entries, ends))
    return toks, steps


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_reused_pages_and_slots(models, name, dtype):
    _, cfg, w, page = models[name]
    toks, steps = mixed_schedule(cfg, 3)
    # fewer pages than all requests together need, and as many state slots as live requests: both are used again
    r = make_runner(models, name, dtype, num_blocks=(90 + 70 + 57 + 33) // page + 12, max_len=96)
    rows = replay(r, steps)
    compare_rows(rows, cfg, w, toks, dtype, f"{name} mixed")
    if dtype == "float32":      # each request alone gives the same rows
        alone = replay(make_runner(models, name, dtype), [([("b", toks["b"], list(range(33)))], ["b"])])
        for (rid, p), row in rows.items():
            if rid == "b":
                assert (row - alone[("b", p)]).abs().max().item() < 1e-4 * row.abs().max().item()


def test_pages_behind_the_window_are_given_back_but_the_kept_ones(models):
    """A long request in a model whose every layer has a window holds a few pages at any time: those of its windows
    and, where a layer keeps its first tokens, theirs."""
    _, cfg, w, page = models["C3"]      # windows 5 and 3, keeps 7, pages of 16
    r = make_runner(models, "C3", "float32", num_blocks=40, max_len=400)
    ids = tokens_for(cfg, 300, 4)
    steps = [([("x", p, [len(p) - 1])], []) for p in cut(ids, [9, 1, 1, 30, 2])]
    rows = replay(r, steps)
    compare_rows(rows, cfg, w, {"x": ids}, "float32", "C3 long request")
    assert len(r.group_specs) == 2
    for g, spec in enumerate(r.group_specs):
        table = r.cache.block_table("x", g)
        held = [i for i, pg in enumerate(table) if pg >= 0]
        assert r.cache.num_free(g) == 40 - len(held)
        last = (len(ids) - 1) // page
        assert held == ([0] if spec.keep_first else []) + list(range((len(ids) - spec.window + 1) // page, last + 1))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["C1", "C3"])
def test_decode_steps_from_graphs(models, name, dtype):
    """Steps of single rows replay captured graphs (batch sizes 1 to 3, requests of unequal length, padded rows that
    use the spare state slot)."""
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, dtype, graph=True)
    assert r._graphs_allowed
    ids = {k: tokens_for(cfg, n, s) for k, n, s in (("a", 60, 1), ("b", 45, 2), ("c", 70, 3))}
    steps = [([("a", ids["a"][:30], [29]), ("b", ids["b"][:5], [4])], []), ([("c", ids["c"][:41], [40])], [])]
    at = {"a": 30, "b": 5, "c": 41}
    while any(at[k] < len(ids[k]) for k in ids):
        es, ends = [], []
        for k in ids:
            if at[k] < len(ids[k]):
                es.append((k, [ids[k][at[k]]], [0]))
                at[k] += 1
                if at[k] == len(ids[k]):
                    ends.append(k)
        steps.append((es, ends))
    compare_rows(replay(r, steps), cfg, w, ids, dtype, f"{name} graph decode")
    assert r._graphs, "no decode graph was captured"


@pytest.mark.parametrize("name", ["C1", "C2"])
def test_greedy_generation_through_the_engine(models, name):
    from dinfer_amd import Engine, SamplingParams
    d, cfg, w, page = models[name]
    eng = Engine(str(d), dtype="float32", max_model_len=256, max_num_seqs=3, block_size=page, num_blocks=120,
                 max_num_batched_tokens=64)
    prompts = [tokens_for(cfg, n, s) for n, s in ((5, 1), (70, 2), (23, 3), (1, 4))]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for tok in out:
            logits = plain.forward(ids, w, cfg)[0][-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() > 1e-3 * logits.std().item():     # a clear choice
                assert tok == int(logits.argmax()), f"{name}: greedy token differs after {len(ids)} tokens"
            ids.append(tok)


def test_bfloat16_generation_is_the_same_from_graphs(models):
    from dinfer_amd import Engine, SamplingParams
    d, cfg, _, page = models["C1"]
    prompts = [tokens_for(cfg, 40, s) for s in range(1, 9)] + [tokens_for(cfg, n, 20 + n) for n in (9, 3)]
    outs = []
    for graphs in (True, False):
        eng = Engine(str(d), dtype="bfloat16", max_model_len=128, max_num_seqs=2, block_size=page, num_blocks=96,
                     max_num_batched_tokens=16, hip_graph=graphs, gemm_tuning="heuristic")
        outs.append(eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0)))
        if graphs:
            assert eng.runner._graphs
    assert outs[0] == outs[1]


# ---- kernels alone --------------------------------------------------------------------------------------------
def paged(rows, page, order):
    """rows [G, n, d] of one request -> (pages [blocks, G, page, d] with the request's pages in `order`, block table)."""
    G, n, d = rows.shape
    nb = -(-n // page)
    pages = torch.full((max(order) + 1, G, page, d), 7.0, dtype=rows.dtype)     # what no key owns holds junk, not zeros
    for i in range(nb):
        part = rows[:, i * page:(i + 1) * page]
        pages[order[i], :, :part.shape[1]] = part
    return pages, torch.tensor([order[:nb]], dtype=torch.int32)


ATTN_CASES = [
    # (heads, kv heads, dim, vdim, page, keys, window, keep_first, sink, slope_exp, values are keys)
    (4, 2, 16, 24, 4, 150, 20, 5, True, 0.0, False),
    (4, 2, 16, 16, 8, 150, 20, 0, False, 8.0, True),
    (3, 3, 40, 8, 16, 200, 0, 0, True, 0.0, False),      # no window
    (8, 1, 32, 32, 4, 90, 7, 12, True, 8.0, False),       # keeps more than the window holds
    (2, 1, 20, 12, 4, 70, 9, 2, True, 0.0, False),        # a head size that is no multiple of 8
    (4, 2, 36, 36, 8, 70, 9, 0, False, 8.0, True),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", ATTN_CASES)
def test_attention_with_options_alone(case, dtype):
    """The kernel on a made-up cache in shuffled pages. Each query is a key of its request times a factor, so that
    one score stands out: far back, the oldest key the window still holds and the one before it, the last kept
    first key and the one after it, keys at a page's last and first place, and the query's own."""
    from dinfer_amd.kernels import ops
    H, G, D, V, page, n, window, keep, sink, slope_exp, vk = case
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(n + D)
    k = torch.randn(G, n, D, generator=g).to(dt)
    v = k if vk else torch.randn(G, n, V, generator=g).to(dt)
    sinks = (torch.randn(H, generator=g) * 2).float() if sink else None
    p = n - 1                                      # the queries' position: all rows are the request's last token
    wlo = max(0, p - window + 1) if window else 0
    targets = sorted({0, 1, wlo, max(wlo - 1, 0), max(keep - 1, 0), min(keep, p), p, p - 1,
                      (p // page) * page, max((p // page) * page - 1, 0), wlo // page * page, n // 2} - {-1})
    order = list(range(-(-n // page) + 3))
    random.Random(n).shuffle(order)
    kp, table = paged(k, page, order)
    vp, _ = paged(v, page, order)
    scale = 0.9 / D ** 0.5
    for target in targets:
        # T rows, each a request of its own over the same pages would need T tables: one row a launch instead
        q = torch.randn(H, D, generator=g)
        for h in range(H):
            q[h] += 6.0 * k[h // (H // G), target].float() / k[h // (H // G), target].float().norm() * D ** 0.25
        q = q.to(dt)
        out = torch.zeros(1, H * V, dtype=dt, device="cuda")
        k_cache = ops.k_cache_pack(kp).cuda()
        v_cache = None if vk else vp.permute(0, 1, 3, 2).contiguous().cuda()
        ops.attn_paged_ext(q.view(1, H * D).cuda(), out, k_cache, v_cache, table.cuda(),
                           torch.tensor([0, 1], dtype=torch.int32, device="cuda"),
                           torch.tensor([n], dtype=torch.int32, device="cuda"), 1, 1, scale=scale, window=window, heads=H,
                           kv_heads=G, head_dim=D, page_size=page, v_dim=V, keep_first=keep,
                           sinks=sinks.cuda() if sink else None, slope_exp=slope_exp, out_scale=0.5)
        j = torch.arange(n)
        mask = ((j <= p) & ((p - j < window) | (j < keep))) if window else (j <= p)
        want = torch.zeros(H, V, dtype=F)
        for h in range(H):
            s = (k[h // (H // G)].double() @ q[h].double()) * scale
            if slope_exp:
                s = s - 2.0 ** (-slope_exp * (h + 1) / H) * (p - j).double()
            pr = plain.softmax_rows(s[None], mask[None], sinks[h].item() if sink else None)
            want[h] = 0.5 * pr[0] @ v[h // (H // G)].double()
        tol = 2e-5 if dtype == "float32" else 2e-2
        err = (out.double().cpu().view(H, V) - want).abs().max().item()
        assert err < tol * max(1.0, want.abs().max().item()), f"{case} target {target}: off by {err:.2e}"


FLASH_CASES = [
    # (heads, kv heads, dim, page, window, keep_first, sink, slope_exp, [(keys, rows of this step)])
    (4, 2, 32, 8, 20, 5, True, 0.0, [(150, 37), (90, 1), (3, 3)]),
    (4, 2, 64, 16, 40, 0, False, 8.0, [(200, 64), (41, 1)]),
    (8, 1, 128, 16, 70, 12, True, 8.0, [(300, 100), (300, 1), (75, 2), (12, 12)]),
    (3, 3, 48, 8, 0, 0, True, 0.0, [(100, 17), (64, 1)]),
    (16, 4, 128, 16, 33, 40, True, 0.0, [(520, 130), (71, 1)]),     # keeps more than it sees; rows of three tiles
]


@pytest.mark.parametrize("kernel", ["flash", "plain"])
@pytest.mark.parametrize("case", FLASH_CASES)
def test_attention_with_options_on_the_matrix_cores(case, kernel):
    """A step of prompt portions and single rows of several requests, pages shuffled among them: the matrix-core flash
    kernel with options, and the plain kernel on the same bfloat16 caches, against float64. A row in eight is made to
    look hard at one key: the oldest its window holds, the one before it, the last kept first key or the one after."""
    from dinfer_amd.kernels import ops
    H, G, D, page, window, keep, sink, slope_exp, reqs = case
    g = torch.Generator().manual_seed(D + page)
    sinks = (torch.randn(H, generator=g) * 2).float() if sink else None
    scale = 0.9 / D ** 0.5
    nb = sum(-(-n // page) for n, _ in reqs)
    ids = list(range(nb + 2))
    random.Random(D).shuffle(ids)
    kp = torch.full((nb + 2, G, page, D), 7.0, dtype=torch.bfloat16)
    vp = torch.full((nb + 2, G, page, D), 7.0, dtype=torch.bfloat16)
    table = torch.full((len(reqs), max(-(-n // page) for n, _ in reqs)), -1, dtype=torch.int32)
    qs, want, at = [], [], 0
    for b, (n, rows) in enumerate(reqs):
        k = torch.randn(G, n, D, generator=g).to(torch.bfloat16)
        v = torch.randn(G, n, D, generator=g).to(torch.bfloat16)
        for i in range(-(-n // page)):
            table[b, i] = ids[at]
            kp[ids[at], :, :min(page, n - i * page)] = k[:, i * page:(i + 1) * page]
            vp[ids[at], :, :min(page, n - i * page)] = v[:, i * page:(i + 1) * page]
            at += 1
        for r in range(rows):
            p = n - rows + r
            q = torch.randn(H, D, generator=g)
            if r % 8 == 0:
                wlo = max(0, p - window + 1) if window else 0
                target = [wlo, max(wlo - 1, 0), max(keep - 1, 0), min(keep, p)][(r // 8) % 4]
                for h in range(H):
                    kk = k[h // (H // G), target].float()
                    q[h] += 5.0 * kk / kk.norm() * D ** 0.25
            q = q.to(torch.bfloat16)
            qs.append(q.view(H * D))
            j = torch.arange(n)
            mask = ((j <= p) & ((p - j < window) | (j < keep))) if window else (j <= p)
            o = torch.zeros(H, D, dtype=F)
            for h in range(H):
                sc = (k[h // (H // G)].double() @ q[h].double()) * scale
                if slope_exp:
                    sc = sc - 2.0 ** (-slope_exp * (h + 1) / H) * (p - j).double()
                o[h] = 0.5 * plain.softmax_rows(sc[None], mask[None], sinks[h].item() if sink else None)[0] @ v[h // (H // G)].double()
            want.append(o.view(H * D))
    q = torch.stack(qs).cuda()
    T = q.shape[0]
    out = torch.zeros(T, H * D, dtype=torch.bfloat16, device="cuda")
    cu = torch.tensor([0] + list(torch.tensor([r for _, r in reqs]).cumsum(0)), dtype=torch.int32, device="cuda")
    sl = torch.tensor([n for n, _ in reqs], dtype=torch.int32, device="cuda")
    k_cache, v_cache = ops.k_cache_pack(kp).cuda(), vp.permute(0, 1, 3, 2).contiguous().cuda()
    opts = dict(scale=scale, window=window, heads=H, kv_heads=G, head_dim=D, page_size=page, keep_first=keep,
                sinks=sinks.cuda() if sink else None, slope_exp=slope_exp, out_scale=0.5)
    if kernel == "flash":
        assert ops.attn_mfma_supports(D, page, H, G)
        ops.attn_flash_ext(q, out, k_cache, v_cache, table.cuda(), cu, sl, len(reqs), max(r for _, r in reqs), **opts)
    else:
        ops.attn_paged_ext(q, out, k_cache, v_cache, table.cuda(), cu, sl, len(reqs), T, **opts)
    want = torch.stack(want)
    err = (out.double().cpu() - want).abs().max(dim=1).values
    worst = int(err.argmax())
    assert err.max().item() < 2e-2 * max(1.0, want.abs().max().item()), f"{case}: row {worst} off by {err.max().item():.2e}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("wide_loads", [False, True])
@pytest.mark.parametrize("sizes", [(2, 1, 8, 8, 2), (4, 2, 16, 24, 4), (3, 3, 40, 48, 3), (2, 1, 64, 32, 1), (2, 2, 128, 136, 4),
                                   (6, 3, 32, 8, 5)])
def test_delta_rule_kernels_alone(sizes, dtype, wide_loads):
    """Two requests of unequal length in one step, then each continued by portions and single rows, against the plain
    recurrence over the whole sequences; slots are not the requests' order, and one starts in a slot that holds junk.
    wide_loads: the transposed taps are given too, so sizes that fit it run the kernel that takes 8 channels a lane."""
    from dinfer_amd.kernels import ops
    H, G, D, V, K = sizes
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(D + V)
    C = 2 * G * D + H * V
    cols = C + H * V + 2 * H
    lens = [37, 9]
    seqs = [torch.randn(n, cols, generator=g).to(dt) for n in lens]
    taps = torch.randn(C, K, generator=g).to(torch.bfloat16).float() * 0.6
    a_log, dt_bias = torch.randn(H, generator=g) * 0.5, torch.randn(H, generator=g) * 0.5
    w_norm = 1 + 0.1 * torch.randn(V, generator=g)
    slots = [3, 1]
    state = torch.full((5, H, V, D), 9.0, device="cuda")                    # junk: a first step must not read it
    conv = torch.full((5, C, K - 1), 9.0, dtype=dt, device="cuda")
    work = torch.zeros(64, ops.delta_work_columns(G, H, D, V), device="cuda")
    o = torch.zeros(64, H * V, device="cuda")
    got = [[], []]
    schedule = [[(0, 5), (1, 2)], [(0, 1), (1, 1)], [(1, 6)], [(0, 17)], [(0, 2), (1, 0)], [(0, 12)]]
    at = [0, 0]
    for step in schedule:
        step = [(r, n) for r, n in step if n]
        rows = torch.cat([seqs[r][at[r]:at[r] + n] for r, n in step]).cuda()
        T = rows.shape[0]
        cu = torch.tensor([0] + list(torch.tensor([n for _, n in step]).cumsum(0)), dtype=torch.int32, device="cuda")
        sl = torch.tensor([at[r] + n for r, n in step], dtype=torch.int32, device="cuda")
        ss = torch.tensor([slots[r] for r, _ in step], dtype=torch.int32, device="cuda")
        common = dict(state_slots=ss, cu_seqlens=cu, seq_lens=sl, num_reqs=len(step))
        ops.delta_prep(rows, T, qkv_off=0, b_off=C + H * V, a_off=C + H * V + H, taps=taps.cuda(), a_log=a_log.cuda(),
                       dt_bias=dt_bias.cuda(), conv_state=conv, work=work, qk_heads=G, heads=H, dim=D, vdim=V, eps=1e-6,
                       q_scale=D ** -0.5, taps_t=taps.t().contiguous().cuda() if wide_loads else None, **common)
        ops.delta_conv_update(rows, qkv_off=0, conv_state=conv, **common)
        ops.delta_recurrence(work, state, o, qk_heads=G, heads=H, dim=D, vdim=V, **common)
        out = torch.zeros(T, H * V, dtype=dt, device="cuda")
        ops.delta_out(o, rows, C, w_norm.cuda(), out, T, heads=H, vdim=V, eps=1e-5)
        t = 0
        for r, n in step:
            got[r].append(out[t:t + n].double().cpu())
            t += n
            at[r] += n
    for r in range(2):
        x = seqs[r].double()
        n = at[r]
        q = plain.silu(plain.short_convolution(x[:n, :G * D], taps[:G * D].double())).view(n, G, D)
        k = plain.silu(plain.short_convolution(x[:n, G * D:2 * G * D], taps[G * D:2 * G * D].double())).view(n, G, D)
        v = plain.silu(plain.short_convolution(x[:n, 2 * G * D:C], taps[2 * G * D:].double())).view(n, H, V)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        gate = plain.silu(x[:n, C:C + H * V]).view(n, H, V)
        beta = torch.sigmoid(x[:n, C + H * V:C + H * V + H])
        dec = torch.exp(-torch.exp(a_log.double()) * plain.softplus(x[:n, C + H * V + H:] + dt_bias.double()))
        want = torch.zeros(n, H, V, dtype=F)
        for h in range(H):
            S = torch.zeros(D, V, dtype=F)
            for t in range(n):
                S = dec[t, h] * S
                u = beta[t, h] * (v[t, h] - S.T @ k[t, h // (H // G)])
                S = S + torch.outer(k[t, h // (H // G)], u)
                want[t, h] = S.T @ q[t, h // (H // G)]
        want = (plain.norm_plain(want, w_norm.double(), 1e-5) * gate).reshape(n, H * V)
        err = (torch.cat(got[r]) - want).abs().max().item()
        assert err < (1e-4 if dtype == "float32" else 3e-2) * max(1.0, want.abs().max().item()), f"request {r}: off by {err:.2e}"


@pytest.mark.parametrize("width", [8, 10, 72, 320, 4096, 5000, 9000])
@pytest.mark.parametrize("types", [("float32", "float32", "float32"), ("bfloat16", "float32", "bfloat16")])
def test_stream_norm_kernel(width, types):
    """stream += mult * norm(branch) * (1 + wb); out = norm(stream) * (1 + w), with and without each half, on listed rows."""
    from dinfer_amd.kernels import ops
    bt, st, ot = (getattr(torch, t) for t in types)
    g = torch.Generator().manual_seed(width)
    branch = torch.randn(9, width, generator=g).to(bt)
    stream = torch.randn(9, width, generator=g).to(st)
    wb, w = torch.randn(width, generator=g) * 0.2, torch.randn(width, generator=g) * 0.2
    rows = torch.tensor([7, 0, 3], dtype=torch.int32)
    for use_branch, use_out, use_rows in ((True, True, False), (True, False, False), (False, True, True), (True, True, True)):
        s = stream.clone().cuda()
        out = torch.zeros(9, width, dtype=ot, device="cuda") if use_out else None
        n = 3 if use_rows else 9
        ops.rmsnorm_stream(s, n, branch=branch.cuda() if use_branch else None, branch_weight=wb.cuda() if use_branch else None,
                           branch_eps=1e-6, branch_offset=1.0, mult=0.3, out=out, weight=w.cuda() if use_out else None,
                           eps=1e-5, offset=1.0, rows=rows.cuda() if use_rows else None)
        idx = rows.long() if use_rows else torch.arange(9)
        x = stream.double()
        if use_branch:
            x = x.clone()
            x[idx] = x[idx] + 0.3 * plain.norm_around_zero(branch.double()[idx], wb.double(), 1e-6)
            x = x.to(st).double()
        assert (s.double().cpu() - x).abs().max().item() < 1e-5 * (1 if st == torch.float32 else 1e3)
        if use_out:
            want = plain.norm_around_zero(x[idx], w.double(), 1e-5)
            assert (out[:n].double().cpu() - want).abs().max().item() < (1e-5 if ot == torch.float32 else 4e-2)


@pytest.mark.parametrize("dims", [8, 6, 16])
def test_rotation_by_wavelength_bands(dims):
    """The table against angles from the plain frequencies, and the kernel's rotation of pairs (2i, 2i+1) on the first
    `dims` entries of a head of 16."""
    from dinfer_amd.kernels import ops
    from dinfer_amd.parts.position import Rotary
    rot = dict(base=900.0, dims=dims, scaling=BANDS)
    table = Rotary(16, 900.0, 64, dims, "interleaved", dict(kind="wavelength_bands", **BANDS)).host_table(64)
    f = plain.rotary_frequencies(rot)
    ang = torch.arange(64, dtype=F)[:, None] * f[None, :]
    assert (table.double() - torch.cat([ang.cos(), ang.sin()], 1)).abs().max().item() < 1e-6
    assert f[0] == 1.0 and f[-1] < 900.0 ** (-(dims - 2) / dims) * 0.99          # the fastest kept, the slowest slowed
    x = torch.randn(5, 3 * 16)
    pos = torch.tensor([0, 1, 17, 40, 63], dtype=torch.int32)
    buf = x.clone().cuda()
    ops.qkv_post(buf, 5, heads=1, kv_heads=1, head_dim=16, q_off=0, k_off=16, v_off=32, q_gain=None, k_gain=None, eps=0.0,
                 gain_offset=0.0, positions=pos.cuda(), cos_sin=table.cuda(), rotary_dim=dims, rope_style=1, k_cache=None,
                 v_cache=None, slot_mapping=None, page_size=4)
    want = plain.rotate_pairs(x[:, :32].double().view(5, 2, 16), pos, rot).view(5, 32)
    assert (buf[:, :32].double().cpu() - want).abs().max().item() < 1e-5
    assert torch.equal(buf[:, 32:].cpu(), x[:, 32:])


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_program(models, tmp_path, dtype):
    """bin/trace_run as a user runs it: a subprocess fed JSON lines; five requests through a pool made for three, so
    pages and state slots are used again; logits read from the files it writes."""
    import subprocess
    import sys
    from pathlib import Path
    import numpy as np
    d, cfg, w, page = models["C4"]
    V = cfg["vocab"]
    seqs = {k: tokens_for(cfg, n, sum(map(ord, k))) for k, n in (("a", 50), ("b", 90), ("c", 33), ("d", 64), ("e", 20))}
    plan = [[("a", 30), ("b", 7)], [("a", 20), ("b", 2), ("c", 33)], [("b", 50)], [("b", 1), ("d", 40)],
            [("b", 1), ("d", 2), ("e", 19)], [("b", 29), ("d", 22), ("e", 1)]]
    steps, fed, expect = [], {k: 0 for k in seqs}, {}
    for i, st in enumerate(plan):
        entries, ends = [], []
        for k, n in st:
            wants = sorted({0, n - 1})
            entries.append({"id": k, "tokens": seqs[k][fed[k]:fed[k] + n], "want": wants})
            expect.setdefault(i, []).extend((k, fed[k] + j) for j in wants)
            fed[k] += n
            if fed[k] == len(seqs[k]):
                ends.append(k)
        steps.append({"step": i, "entries": entries, "end": ends})
    root = Path(__file__).resolve().parent.parent
    p = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(d), "--dtype", dtype, "--out",
                        str(tmp_path), "--max-tokens", "256", "--block-size", str(page)],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(plan))]
    want = {k: plain.forward(v, w, cfg)[0] for k, v in seqs.items()}
    for i, places in expect.items():
        got = torch.from_numpy(np.fromfile(tmp_path / f"{i}.f32", dtype="<f4").reshape(len(places), V))
        check_logits(got, torch.stack([want[k][pos] for k, pos in places]), dtype, f"replayed step {i}")
