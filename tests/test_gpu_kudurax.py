"""Kudurax through the engine against the plain float64 implementation (plain_kudurax.py): every mechanism alone
at the level of its kernels, then whole models of made-up sizes in every way of cutting and batching, 32-bit and
bfloat16, and greedy generation through the engine's own entry point."""
import json
import math
import random

import pytest
import torch

import plain_kudurax as plain

pytestmark = pytest.mark.gpu
F = torch.float64


# ---- configurations -------------------------------------------------------------------------------------------
def mixer(heads, dim, rot_dim, vdim, rank, scale, base=10000.0, dims=None, scaling=None, kv_from=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=rank, scale=scale,
             rot=dict(base=base, dims=rot_dim if dims is None else dims))
    if scaling is not None:
        m["rot"]["scaling"] = scaling
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, ff, shared=None):
    f = dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=ff))
    if shared:
        f["shared"] = dict(ff=shared)
    return f


def layer(m, f):
    return dict(type="latent_attention", mixer=m, mlp=f)


YARN = dict(factor=4.0, original=64, fast=8.0, slow=1.0)
M1 = dict(heads=4, dim=16, rot_dim=8, vdim=24, rank=32, scale=0.2, scaling=YARN)
M2 = dict(heads=3, dim=12, rot_dim=6, vdim=10, rank=40, scale=0.31, dims=4, base=500.0)
M3a = dict(heads=16, dim=8, rot_dim=16, vdim=8, rank=64, scale=0.25, base=30000.0, scaling=dict(factor=16.0, original=32, fast=4.0, slow=2.0))
M3b = dict(heads=2, dim=8, rot_dim=8, vdim=16, rank=48, scale=0.4)

CONFIGS = {
    # sizes the matrix-core kernels take; a routed layer on another layer's cache, a layer without feed-forward
    "K1": (dict(architecture="Kudurax", vocab=200, width=64, embedding=dict(scale=5.5), norm=dict(eps=1e-5), layers=[
        layer(mixer(**M1), dense(96)), layer(mixer(**M1, kv_from=0), moe(6, 2, 32, shared=40)),
        layer(mixer(**M1), moe(4, 3, 24)), layer(mixer(**M1, kv_from=2), None)]), 8, 5),
    # sizes no matrix-core kernel takes (odd heads, a latent of 40, pages of 4), fewer rotated dims than the rotated
    # part has, no scaling, one expert of five a token
    "K2": (dict(architecture="Kudurax", vocab=131, width=72, embedding=dict(scale=1.0), norm=dict(eps=1e-3), layers=[
        layer(mixer(**M2), moe(5, 1, 20, shared=24)), layer(mixer(**M2, kv_from=0), dense(40)),
        layer(mixer(**M2, kv_from=0), moe(3, 3, 16))]), 4, 6),
    # a whole tile of heads a token; layers of unequal latent sizes (two page groups); every expert chosen
    "K3": (dict(architecture="Kudurax", vocab=97, width=48, embedding=dict(scale=2.0), norm=dict(eps=1e-6), layers=[
        layer(mixer(**M3a), moe(4, 4, 16, shared=16)), layer(mixer(**M3b), dense(64)),
        layer(mixer(**M3a, kv_from=0), dense(32)), layer(mixer(**M3b, kv_from=1), moe(8, 2, 8))]), 16, 7),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    from dinfer_amd.weights.safetensors_io import write_safetensors
    out = {}
    for name, (cfg, page, seed) in CONFIGS.items():
        d = tmp_path_factory.mktemp(f"kudurax_{name}")
        w = plain.random_weights(cfg, seed)
        (d / "config.json").write_text(json.dumps(cfg))
        write_safetensors(d / "model.safetensors", w, metadata={"format": "pt"})
        out[name] = (d, cfg, w, page)
    return out


def make_runner(models, name, dtype, max_tokens=512, num_blocks=128, max_seqs=4, max_len=512, graph=False):
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
        assert err < 3e-4, f"{what}: 32-bit logits off by {err:.2e} row-sigmas"
    else:
        # roundings to 8 bits through these narrow models add up to 0.01 to 0.035 of a row's spread; a key too many,
        # a gate left out or a wrong expert is several times that
        assert err < 0.2 and rms < 0.06, f"{what}: bf16 logits off by {err:.3f} (rms {rms:.4f}) row-sigmas"


def step_choices(runner, tokens):
    """What the routed layers chose in the step that has just run: {layer: [tokens, top]} in the step's token order."""
    torch.cuda.synchronize()
    out = {}
    for i, block in enumerate(runner.model.blocks):
        ff = block.ff
        if ff is not None and hasattr(ff, "idx"):
            out[i] = ff.idx[:tokens * ff.top].view(tokens, ff.top).cpu().long().clone()
    return out


class Rows(dict):
    """{(id, position): logits row}, and .choices {id: {layer: [positions, top]}}: the experts the engine used."""

    def __init__(self):
        super().__init__()
        self.choices = {}


def replay(runner, steps):
    """steps: [(entries, ends)], entries [(id, tokens, want)] -> Rows."""
    from dinfer_amd.engine.batch import Entry
    computed, rows = {}, Rows()
    for entries, ends in steps:
        es = []
        for rid, toks, want in entries:
            start = computed.get(rid, 0)
            assert runner.reserve(rid, start, len(toks)), f"out of pages for {rid}"
            es.append(Entry(rid, toks, start, want))
        if es:
            logits = runner.step(es).double().cpu()
            chosen, t = step_choices(runner, sum(len(e.tokens) for e in es)), 0
            for e in es:
                mine = rows.choices.setdefault(e.req_id, {})
                for layer_no, c in chosen.items():
                    mine[layer_no] = torch.cat([mine.get(layer_no, c[:0]), c[t:t + len(e.tokens)]])
                t += len(e.tokens)
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
    """Every replayed row against the plain model run on the request's whole sequence. 32-bit: the engine must have
    chosen the plain model's experts. bfloat16: the plain model is told the engine's experts (each of which must be a
    close call, see plain.routed_ff), so that a rounding that tips a choice does not hide everything behind it."""
    assert rows
    for rid in {k[0] for k in rows}:
        ids = toks[rid.split("#")[0]]
        chosen = {l: c for l, c in rows.choices.get(rid, {}).items() if c.shape[0] == len(ids)}
        assert len(chosen) == len(rows.choices.get(rid, {})), "the test must feed a request to its end"
        want = plain.forward(cfg, w, ids, choices=chosen if dtype == "bfloat16" else None)
        if dtype == "float32" and chosen:
            free = {}
            plain_choices(cfg, w, ids, free)
            for l, c in chosen.items():
                assert torch.equal(c, free[l]), f"{what} request {rid}: layer {l} chose other experts than the plain model"
        pos = sorted(p for (r, p) in rows if r == rid)
        check_logits(torch.stack([rows[(rid, p)] for p in pos]), want[pos], dtype, f"{what} request {rid}")


def plain_choices(cfg, w, ids, out):
    """The plain model's own expert choices per routed layer, by running it with a spy on its routing."""
    inner = plain.routed_ff

    def spy(h, wts, p, mlp, forced=None):
        z = h @ wts[p + "router"].double().T
        out[int(p[1:p.index(".")])] = torch.argsort(-z, dim=-1, stable=True)[:, :mlp["router"]["top"]]
        return inner(h, wts, p, mlp, forced)
    plain.routed_ff = spy
    try:
        plain.forward(cfg, w, ids)
    finally:
        plain.routed_ff = inner


def cut(ids, sizes):
    out, i, k = [], 0, 0
    while i < len(ids):
        out.append(ids[i:i + sizes[k % len(sizes)]])
        i += len(out[-1])
        k += 1
    return out


DTYPES = ["float32", "bfloat16"]
NAMES = ["K1", "K2", "K3"]


# ---- whole models ---------------------------------------------------------------------------------------------
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
def test_residual_stream_after_every_layer(models, name):
    """32-bit, layer by layer: the stream after block i (its pending branch added) against the plain layer outputs."""
    from dinfer_amd.engine.batch import Entry
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, "float32")
    ids = tokens_for(cfg, 37, 9)
    want = []
    plain.forward(cfg, w, ids, layers_out=want)
    seen = []
    model = r.model
    for i, block in enumerate(model.blocks):
        inner = block.forward

        def spy(hidden, pending, batch, cache, _inner=inner, **kw):
            out = _inner(hidden, pending, batch, cache, **kw)
            seen.append((hidden[:batch.num_tokens].double() + out[:batch.num_tokens].double()).cpu())
            return out
        block.forward = spy
    assert r.reserve("x", 0, len(ids))
    r.step([Entry("x", ids, 0, [0])])
    assert len(seen) == len(want)
    for i, (g, x) in enumerate(zip(seen, want)):
        assert (g - x).abs().max().item() < 2e-4 * max(1.0, x.abs().max().item()), f"{name}: the stream after layer {i} differs"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_long_decoding(models, name, dtype):
    _, cfg, w, page = models[name]
    r = make_runner(models, name, dtype)
    ids = tokens_for(cfg, 3 * page + 90, 5)
    first = 3 * page - 1                      # the first decoded token opens a new page
    steps = [([("x", ids[:first], [first - 1])], [])]
    steps += [([("x", [ids[p]], [0])], []) for p in range(first, len(ids))]
    compare_rows(replay(r, steps), cfg, w, {"x": ids}, dtype, f"{name} decode after prompt")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_token_by_token_from_the_first(models, name, dtype):
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, dtype)
    ids = tokens_for(cfg, 40, 6)
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
    # fewer pages than all requests together need
    r = make_runner(models, name, dtype, num_blocks=(90 + 70 + 57 + 33) // page + 12, max_len=96)
    rows = replay(r, steps)
    compare_rows(rows, cfg, w, toks, dtype, f"{name} mixed")
    # each request alone gives the same rows (32-bit: to rounding of the last bit or two)
    if dtype == "float32":
        alone = replay(make_runner(models, name, dtype), [([("b", toks["b"], list(range(33)))], ["b"])])
        for (rid, p), row in rows.items():
            if rid == "b":
                assert (row - alone[("b", p)]).abs().max().item() < 1e-4 * row.abs().max().item()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["K1", "K3"])
def test_decode_steps_from_graphs(models, name, dtype):
    """Steps of single rows replay captured graphs (batch sizes 1 to 4, requests of unequal length, padded rows)."""
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


@pytest.mark.parametrize("name", ["K1", "K2"])
def test_greedy_generation_through_the_engine(models, name):
    from dinfer_amd import Engine, SamplingParams
    d, cfg, w, page = models[name]
    eng = Engine(str(d), dtype="float32", max_model_len=256, max_num_seqs=3, block_size=page, num_blocks=96,
                 max_num_batched_tokens=64)
    prompts = [tokens_for(cfg, n, s) for n, s in ((5, 1), (70, 2), (23, 3), (1, 4))]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for tok in out:
            logits = plain.forward(cfg, w, ids)[-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() > 1e-3 * logits.std().item():     # a clear choice
                assert tok == int(logits.argmax()), f"{name}: greedy token differs after {len(ids)} tokens"
            ids.append(tok)


@pytest.mark.parametrize("name", ["K1", "K3"])
def test_bfloat16_generation_is_the_same_from_graphs(models, name):
    """Greedy generation in bfloat16 through the engine, steps replayed from graphs (single rows and prompt portions whose
    counts come up again) against the same engine launching every step eagerly: the same tokens, and graphs were used."""
    from dinfer_amd import Engine, SamplingParams
    d, cfg, _, page = models[name]
    prompts = [tokens_for(cfg, 40, s) for s in range(1, 11)] + [tokens_for(cfg, n, 20 + n) for n in (9, 3)]
    outs = []
    for graphs in (True, False):
        eng = Engine(str(d), dtype="bfloat16", max_model_len=128, max_num_seqs=2, block_size=page, num_blocks=64,
                     max_num_batched_tokens=16, hip_graph=graphs, gemm_tuning="heuristic")
        outs.append(eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0)))
        if graphs:
            assert eng.runner._graphs and eng.runner.portion_replays > 0
    assert outs[0] == outs[1]


def test_config_round_trip_and_refusals(models):
    from dinfer_amd.config import ConfigError, load_config
    d, cfg, _, _ = models["K1"]
    arch, typed = load_config(d)
    assert arch.name == "Kudurax" and typed.to_dict() == cfg
    bad = json.loads(json.dumps(cfg))
    bad["layers"][1]["mixer"]["kv_from"] = 1
    with pytest.raises(ConfigError):
        arch.config_class.from_dict(bad)        # layer 1 cannot read its own cache
    bad["layers"][1]["mixer"]["kv_from"] = 0
    bad["layers"][1]["mixer"]["kv_rank"] = 16
    with pytest.raises(ConfigError):
        arch.config_class.from_dict(bad)        # the borrowed cache has another latent size


# ---- mechanisms alone -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("width", [48, 200, 1024])
def test_layer_norm_kernel(width):
    from dinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(width)
    x = torch.randn(9, width, generator=g) * 3 + 1.5
    res = torch.randn(9, width, generator=g)
    w, b = 1 + 0.3 * torch.randn(width, generator=g), torch.randn(width, generator=g)
    want = plain.layer_norm(x.double(), w.double(), b.double(), 1e-5)
    out = torch.empty(9, width, device="cuda")
    ops.layernorm(x.cuda(), w.cuda(), b.cuda(), out, 1e-5, 9)
    assert (out.double().cpu() - want).abs().max() < 1e-5
    # a bfloat16 branch added into a float stream; only rows 7 and 2 are normed
    xb = x.to(torch.bfloat16)
    stream = res.clone().cuda()
    rows = torch.tensor([7, 2], dtype=torch.int32, device="cuda")
    outb = torch.empty(2, width, device="cuda", dtype=torch.bfloat16)
    ops.layernorm(xb.cuda(), w.cuda(), b.cuda(), outb, 1e-5, 2, residual=stream, rows=rows)
    summed = xb.double() + res.double()
    assert (stream.double().cpu()[[7, 2]] - summed[[7, 2]]).abs().max() < 1e-6
    assert torch.equal(stream.cpu()[[0, 1, 3]], res[[0, 1, 3]])
    want2 = plain.layer_norm(summed[[7, 2]], w.double(), b.double(), 1e-5)
    assert (outb.double().cpu() - want2).abs().max() < 0.02 * want2.abs().max()


@pytest.mark.parametrize("scaling", [None, dict(factor=8.0, original=128, fast=16.0, slow=1.0),
                                     dict(factor=2.5, original=40, fast=2.0, slow=0.5)])
def test_rotation_table(scaling):
    from dinfer_amd.parts.position import Rotary
    dims = 12
    rot = Rotary(head_dim=16, theta=3000.0, max_positions=400, rotary_dim=dims, style="interleaved", scaling=scaling)
    table = rot.host_table(400).double()
    x = torch.randn(400, 3, 16, dtype=F)
    want = plain.rotate_interleaved(x, torch.arange(400), dims, 3000.0, scaling)
    c, s = table[:, None, :dims // 2], table[:, None, dims // 2:]
    got = x.clone()
    got[..., 0:dims:2] = x[..., 0:dims:2] * c - x[..., 1:dims:2] * s
    got[..., 1:dims:2] = x[..., 1:dims:2] * c + x[..., 0:dims:2] * s
    assert (got - want).abs().max() < 1e-5
    if scaling:     # slow pairs are slowed by the factor, fast ones are not, and both cos and sin grow
        f, m = plain.rotary_frequencies(dims, 3000.0, scaling)
        f0, _ = plain.rotary_frequencies(dims, 3000.0, None)
        assert m > 1 and f[0] == f0[0] and abs(f[-1] * scaling["factor"] / f0[-1] - 1) < 1e-12


def latent_case(seqs, q_lens, H, R, dr, page, seed, dtype, far=None):
    """A made-up cache and step: returns what the kernels take and, per request, (q rows, key rows, start)."""
    g = torch.Generator().manual_seed(seed)
    DK = R + dr
    n_pages = sum(-(-s // page) for s in seqs) + 3
    order = torch.randperm(n_pages, generator=g).tolist()        # pages in no order
    cache = torch.randn(n_pages, page, DK, generator=g)
    bt = torch.full((len(seqs), max(-(-s // page) for s in seqs)), -1, dtype=torch.int32)
    keys = []
    for b, s in enumerate(seqs):
        for j in range(-(-s // page)):
            bt[b, j] = order.pop()
        rows = torch.stack([cache[bt[b, j // page], j % page] for j in range(s)])
        keys.append(rows)
    T = sum(q_lens)
    qa = torch.randn(T, H * DK, generator=g) * 0.3
    if far is not None:      # one query made to look at one key: (request, row of the step, head, key)
        b, i, h, j = far
        t = sum(q_lens[:b]) + i
        qa[t, h * DK:(h + 1) * DK] = keys[b][j] * 3.0
    cu = torch.tensor([sum(q_lens[:i]) for i in range(len(q_lens) + 1)], dtype=torch.int32)
    return dict(qa=qa.to(dtype), cache=cache.to(dtype), bt=bt, cu=cu, seq=torch.tensor(seqs, dtype=torch.int32),
                keys=keys)


def latent_plain(case, q_lens, seqs, H, R, dr, scale, window=0):
    qa, DK = case["qa"].double(), R + dr
    out, t = [], 0
    for b, (n, s) in enumerate(zip(q_lens, seqs)):
        k = case["cache"].double()[case["bt"][b].long().clamp(min=0)].reshape(-1, DK)[:s]
        q = qa[t:t + n].view(n, H, DK)
        pos = torch.arange(s - n, s)
        sc = torch.einsum("nhd,sd->nhs", q, k) * scale
        j = torch.arange(s)
        hidden = (j[None, :] > pos[:, None]) | ((j[None, :] <= pos[:, None] - window) if window else False)
        a = torch.softmax(sc.masked_fill(hidden[:, None, :], float("-inf")), dim=-1)
        out.append(torch.einsum("nhs,sd->nhd", a, k[:, :R]).reshape(n, H * R))
        t += n
    return torch.cat(out)


LATENT_CASES = [
    # seqs, q_lens, H, R, dr, page, window, far
    ([300], [300], 4, 32, 8, 8, 0, (0, 299, 2, 3)),                 # a whole prompt; its last row looks at key 3
    ([777, 40, 129], [1, 1, 1], 8, 64, 16, 16, 0, (0, 0, 5, 15)),   # single rows; a key at a page's last place
    ([777, 40, 129], [1, 1, 1], 8, 64, 16, 16, 0, (0, 0, 5, 16)),   # ... and at the next page's first
    ([500, 64, 33], [37, 1, 33], 16, 128, 32, 8, 0, (0, 36, 9, 0)), # a portion behind a history, a single row, a prompt
    ([200, 90], [64, 2], 3, 48, 8, 8, 50, (0, 10, 1, 200 - 64 + 10 - 49)),   # a window: the oldest key a row still sees
    ([200, 90], [64, 2], 3, 48, 8, 8, 50, (0, 10, 1, 200 - 64 + 10 - 50)),   # ... and the first it does not
    ([150, 70], [150, 3], 2, 512, 128, 16, 0, (0, 149, 1, 5)),     # the widest rows the matrix-core kernels take (no room in LDS)
    ([260], [100], 5, 80, 24, 24, 0, (0, 99, 4, 160)),             # pages that are no power of two
]


@pytest.mark.parametrize("case_no", range(len(LATENT_CASES)))
@pytest.mark.parametrize("kernel", ["plain32", "plain16", "mfma", "mfma_split"])
def test_latent_attention_kernels(case_no, kernel):
    from dinfer_amd.kernels import ops
    seqs, q_lens, H, R, dr, page, window, far = LATENT_CASES[case_no]
    if kernel == "mfma_split" and any(n != 1 for n in q_lens):
        pytest.skip("parts are cut for steps of single rows")
    dtype = torch.float32 if kernel == "plain32" else torch.bfloat16
    case = latent_case(seqs, q_lens, H, R, dr, page, 100 + case_no, dtype, far)
    scale = 0.7 / math.sqrt(R + dr)
    want = latent_plain(case, q_lens, seqs, H, R, dr, scale, window)
    dev = {k: v.cuda() for k, v in case.items() if k != "keys"}
    T, B = sum(q_lens), len(seqs)
    out = torch.zeros(T, H * R, dtype=dtype, device="cuda")
    geo = dict(scale=scale, window=window, heads=H, rank=R, rot_dim=dr, page_size=page)
    if kernel.startswith("plain"):
        ops.latent_attn_ref(dev["qa"], out, dev["cache"], dev["bt"], dev["cu"], dev["seq"], B, T, **geo)
    else:
        assert ops.latent_mfma_supports(R, dr, page)
        cache_t = dev["cache"][:, :, :R].transpose(1, 2).contiguous()
        splits = 5 if kernel == "mfma_split" else 1
        part = torch.zeros(T * H * splits * (R + 4), dtype=torch.float32, device="cuda")
        ops.latent_attn_mfma(dev["qa"], out, dev["cache"], cache_t, dev["bt"], dev["cu"], dev["seq"], B, T, splits, part, **geo)
    got = out.double().cpu()
    tol = 2e-5 if dtype == torch.float32 else 0.03
    assert (got - want).abs().max().item() < tol * max(1.0, want.abs().max().item()), f"{kernel} case {case_no}"
    # the row that was made to look at one key: seen, it dominates; just outside the window, it is gone
    b, i, h, j = far
    t = sum(q_lens[:b]) + i
    p = seqs[b] - q_lens[b] + i
    seen = j <= p and (not window or j > p - window)
    close = (got[t, h * R:(h + 1) * R] - case["keys"][b][j][:R].double()).abs().max().item()
    assert (close < 0.1) == seen


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(5, 16, 32, 24, 40), (3, 12, 40, 10, 37), (16, 64, 128, 64, 200)])
def test_products_per_head(sizes, dtype):
    from dinfer_amd.kernels import ops
    H, K, N, stride_extra, T = sizes
    g = torch.Generator().manual_seed(H)
    a = (torch.randn(T, H * (K + stride_extra) + 8, generator=g)).to(dtype)
    w = (torch.randn(H, N, K, generator=g) / math.sqrt(K)).to(dtype)
    gate = torch.randn(T, H + 3, generator=g).to(dtype)
    out = torch.zeros(T, H * N, dtype=dtype, device="cuda")
    ops.heads_nt(a.cuda(), 8, K + stride_extra, w.cuda(), out, 0, N, T, gate=gate.cuda(), gate_off=3)
    want = torch.stack([a.double()[:, 8 + h * (K + stride_extra):8 + h * (K + stride_extra) + K] @ w[h].double().T
                        * torch.sigmoid(gate.double()[:, 3 + h])[:, None] for h in range(H)], dim=1).reshape(T, H * N)
    tol = 1e-5 if dtype == torch.float32 else 0.02
    assert (out.double().cpu() - want).abs().max().item() < tol * want.abs().max().item()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(6, 2, 64, 32, 40, 70), (5, 1, 72, 20, 24, 33), (4, 4, 48, 16, None, 200), (1, 1, 32, 8, 8, 3)])
def test_routed_feed_forward_alone(sizes, dtype):
    """The part itself (route, sort, the experts' products, sum) against the plain rule; one token's logits are
    made equal on purpose: among equals the lowest expert wins."""
    from types import SimpleNamespace
    from dinfer_amd.parts import FEED_FORWARDS, BuildContext
    E, top, W, ff, shared, T = sizes
    cfg = dict(width=W, vocab=8, layers=[layer(mixer(1, 8, 8, 8, 16, 1.0), moe(E, top, ff, shared))])
    w = {k[len("l0.mlp."):]: v for k, v in plain.random_weights(cfg, E * 10 + top).items() if k.startswith("l0.mlp.")}
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, W, generator=g).to(dtype)
    if E > 2:
        w["router"][2] = w["router"][1]           # experts 1 and 2 always tie
    part = FEED_FORWARDS.get("moe")(hidden=W, experts=E, top=top, intermediate=ff, shared_intermediate=shared)
    part.load(lambda name, compute=False: w[name].to(dtype).cuda())
    ctx = BuildContext(torch.device("cuda"), dtype, 256, 256, 16)
    part.bind(ctx)
    out = part.forward(x.cuda(), SimpleNamespace(num_tokens=T))[:T].double().cpu()
    wp = {"p." + k: v for k, v in w.items()}
    mlp = dict(router=dict(experts=E, top=top), shared=dict(ff=shared) if shared else None)
    z = x.double() @ w["router"].double().T
    want = plain.routed_ff(x.double(), wp, "p.", mlp)
    tol = 1e-5 if dtype == torch.float32 else 0.03
    assert (out - want).abs().max().item() < tol * want.abs().max().item()
    # the choice itself: the device's list against topk with the lowest index first among equals
    idx = part.idx[:T * top].view(T, top).cpu().long()
    order = torch.argsort(-z, dim=-1, stable=True)[:, :top]
    assert torch.equal(idx, order)
    share = part.share[:T * top].view(T, top).double().cpu()
    assert (share - torch.softmax(torch.gather(z, 1, order), -1)).abs().max() < 1e-5
    assert (share.sum(-1) - 1).abs().max() < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("act", ["relu2", "silu", "gelu_tanh"])
def test_activations_of_one_argument(act, dtype):
    from dinfer_amd.kernels import ops
    x = torch.linspace(-6, 6, 1001).repeat(3, 1).to(dtype)
    out = torch.empty_like(x, device="cuda")
    ops.act(x.cuda(), out, 3, act)
    z = x.double()
    want = {"relu2": torch.relu(z) ** 2, "silu": z * torch.sigmoid(z), "gelu_tanh": plain.gelu_tanh(z)}[act]
    tol = 1e-5 if dtype == torch.float32 else 0.01
    assert (out.double().cpu() - want).abs().max().item() < tol * want.abs().max().item()


def test_embedding_into_a_wider_stream():
    from dinfer_amd.kernels import ops
    table = torch.randn(50, 40).to(torch.bfloat16).cuda()
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device="cuda")
    out = torch.empty(4, 40, device="cuda")
    ops.embedding(ids, table, out, scale=7.25)
    assert torch.equal(out, table[ids.long()].float() * 7.25)
