"""Karopel without a GPU: the configuration and its refusals, run order and tensor names of the model description,
the caches its mixers ask for, the pages a window gives back and the ones it keeps, and the plain float64 model
(plain_karopel.py) pinned by library functions and hand-worked cases."""
import json

import pytest
import torch

import plain_karopel as plain

F = torch.float64


def attention(size=10, keep=3, dims=8, scaling=None):
    return dict(type="attention", mlp=dict(kind="dense", ff=40),
                mixer=dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.25, mask=dict(size=size, keep_first=keep),
                           rot=dict(base=1000.0, dims=dims, scaling=scaling)))


def parallel(conv=3):
    return dict(type="parallel", mlp=None,
                mixer=dict(left=dict(heads=4, kv_heads=1, dim=16, vdim=16, scale=0.25, mask=dict(size=7)),
                           right=dict(heads=4, kv_heads=2, dim=16, vdim=8, conv=conv), left_scale=0.7, right_scale=0.45))


def config(**kw):
    cfg = dict(architecture="Karopel", vocab=96, width=64, residual_mult=0.5, logit_scale=1.5, norm=dict(eps=1e-5),
               loop=dict(start=1, stop=3, times=3), layers=[parallel(), attention(), attention(), parallel()])
    cfg.update(kw)
    return cfg


def parsed(cfg):
    from dinfer_amd.config.registry import architecture_of
    arch = architecture_of(cfg)
    return arch, arch.config_class.from_dict(cfg)


def test_config_round_trip_and_refusals():
    from dinfer_amd.config.base import ConfigError
    arch, cfg = parsed(config())
    assert arch.name == "Karopel" and cfg.vocab_size == 96 and cfg.hidden_size == 64
    assert type(cfg).from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    bad = [dict(loop=dict(start=2, stop=2, times=2)), dict(loop=dict(start=0, stop=5, times=1)),
           dict(layers=[dict(attention(), type="mamba")]), dict(layers=[attention(dims=7)]), dict(layers=[attention(dims=18)]),
           dict(layers=[dict(attention(), mlp=dict(kind="moe"))]), dict(layers=[]), dict(norm=None)]
    for change in bad:
        with pytest.raises(ConfigError):
            parsed(config(**change))
    odd = parallel()
    odd["mixer"]["left"]["vdim"] = 8                 # the values are the keys
    with pytest.raises(ConfigError):
        parsed(config(layers=[odd]))
    odd = attention()
    odd["mixer"]["kv_heads"] = 3
    with pytest.raises(ConfigError):
        parsed(config(layers=[odd]))


def test_run_order_and_tensor_names():
    from dinfer_amd.parts.model import expected_tensors
    for cfg in (config(), config(loop=None), config(loop=dict(start=0, stop=4, times=2))):
        arch, c = parsed(cfg)
        spec = arch.build_spec(c)
        want = plain.run_order(cfg)
        assert [e.layer for e in spec.run] == [i for i, _, _ in want]
        assert [e.before is not None for e in spec.run] == [first for _, _, first in want]
        starts = [e.before.params for e in spec.run if e.before is not None]
        assert [(p["row"], p["add_embedding"]) for p in starts] == [(t, t > 0) for t in range(len(starts))]
        exp, optional = expected_tensors(spec)
        shapes = plain.tensor_shapes(cfg)
        assert not optional and {n: tuple(s.shape) for n, s in exp.items()} == shapes
        assert spec.stream_dtype == "float32"
        assert (spec.logits_post is None) == (cfg["logit_scale"] == 1.0)


def test_caches_the_mixers_ask_for():
    from dinfer_amd.parts import DecoderModel, DeltaStateSpec, JoinedSpec, KVSpec
    arch, c = parsed(config())
    needs = DecoderModel(arch.build_spec(c)).cache_needs()
    assert len(needs) == 8 and all(n is not None for n in needs)      # every pass has caches of its own
    a = needs[1]
    assert isinstance(a, KVSpec) and (a.kv_heads, a.head_dim, a.v_dim, a.window, a.keep_first, a.values) == (2, 16, 24, 10, 3, True)
    assert a.page_bytes(4, torch.bfloat16) == 2 * (16 + 24) * 4 * 2
    j = needs[0]
    assert isinstance(j, JoinedSpec) and set(j.members) == {"left", "right"}
    left, right = j.members["left"], j.members["right"]
    assert (left.window, left.values, left.keep_first) == (7, False, 0) and j.window == 7 and not j.recomputable
    assert isinstance(right, DeltaStateSpec) and (right.heads, right.dim, right.vdim, right.channels, right.taps) == (4, 16, 8, 96, 3)
    assert j.group_key() == left.group_key() and j.group_key() != a.group_key()
    assert j.page_bytes(4, torch.bfloat16) == 1 * 16 * 4 * 2                 # keys only
    assert j.slot_bytes(torch.bfloat16) == 4 * 16 * 8 * 4 + 96 * 2 * 2
    made = j.allocate(5, 4, 3, torch.float32, "cpu")
    assert set(made) == {"left.k", "right.state", "right.conv"} and made["right.state"].shape == (3, 4, 8, 16)
    made["right.state"].fill_(1.0)
    made["right.conv"].fill_(1.0)
    j.reset_slots(made, torch.tensor([1]))
    assert made["right.state"][1].abs().sum() == 0 and made["right.conv"][1].abs().sum() == 0 and made["right.state"][0].min() == 1


def test_pages_of_kept_first_keys_are_never_given_back():
    from dinfer_amd.cache import CacheManager, GroupSpec
    m = CacheManager([GroupSpec(4, 32, window=6, keep_first=5), GroupSpec(4, 32, window=6)], max_seqs=2)
    m.admit("a")
    assert m.allocate("a", 0, 41)
    m.release_passed("a", 41)              # the next token sees keys 36.. and, in group 0, keys 0..4
    t0, t1 = m.block_table("a", 0), m.block_table("a", 1)
    assert [i for i, p in enumerate(t0) if p >= 0] == [0, 1, 9, 10] and [i for i, p in enumerate(t1) if p >= 0] == [9, 10]
    m.check()
    m.free("a")
    assert m.num_free(0) == m.num_free(1) == 32


# ---- the plain model itself -----------------------------------------------------------------------------------
def test_plain_short_convolution_is_a_causal_depthwise_convolution():
    g = torch.Generator().manual_seed(1)
    x, taps = torch.randn(13, 5, generator=g, dtype=F), torch.randn(5, 4, generator=g, dtype=F)
    lib = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), taps[:, None, :], groups=5)[0].T
    assert (plain.short_convolution(x, taps) - lib).abs().max() < 1e-12
    assert (plain.short_convolution(x[:2], taps) - lib[:2]).abs().max() < 1e-12      # fewer tokens than taps


def test_plain_frequencies_hand_worked():
    rot = dict(base=10000.0, dims=8, scaling=dict(factor=4.0, low=1.0, high=4.0, original=64))
    f = plain.rotary_frequencies(rot)
    # wavelengths 2 pi, 20 pi, 200 pi, 2000 pi against 64 / 4 = 16 and 64 / 1 = 64: kept, blended, slowed, slowed
    assert f[0] == 1.0 and abs(f[2] - 0.01 / 4) < 1e-15 and abs(f[3] - 0.001 / 4) < 1e-15
    s = (64 / (20 * torch.pi) - 1.0) / 3.0
    assert abs(f[1] - ((1 - s) * 0.1 / 4 + s * 0.1)) < 1e-15
    assert (plain.rotary_frequencies(dict(base=10000.0, dims=8, scaling=None))
            - torch.tensor([1.0, 0.1, 0.01, 0.001], dtype=F)).abs().max() < 1e-15
    x = torch.randn(6, 2, 12, dtype=F)
    y = plain.rotate_pairs(x, torch.arange(6), rot)
    assert torch.equal(y[..., 8:], x[..., 8:]) and torch.equal(y[0], x[0])
    assert (y[..., :8].pow(2).sum(-1) - x[..., :8].pow(2).sum(-1)).abs().max() < 1e-12
    z = torch.view_as_complex(x[..., :8].reshape(6, 2, 4, 2).contiguous()) * torch.polar(torch.ones(6, 4, dtype=F), torch.arange(6, dtype=F)[:, None] * f)[:, None]
    assert (torch.view_as_real(z).reshape(6, 2, 8) - y[..., :8]).abs().max() < 1e-12


def test_plain_masks_and_sink():
    m = plain.visible(12, 4, 2)
    assert m[11].tolist() == [True, True] + [False] * 6 + [True] * 4
    assert m[3].tolist() == [True] * 4 + [False] * 8 and plain.visible(5, 1)[4].tolist() == [False] * 4 + [True]
    s = torch.tensor([[0.0, 1.0, 2.0]], dtype=F)
    p = plain.softmax_rows(s, torch.tensor([[True, True, True]]), sink=0.5)
    e = torch.exp(s)
    assert (p - e / (e.sum() + torch.exp(torch.tensor(0.5, dtype=F)))).abs().max() < 1e-15 and p.sum() < 1
    assert abs(plain.softmax_rows(s, torch.tensor([[True, False, True]])).sum().item() - 1) < 1e-15


def test_plain_delta_rule_recalls_what_it_stored():
    """With step size 1, no decay and orthonormal keys, the state returns each stored value for its key."""
    D, V = 6, 4
    keys = torch.linalg.qr(torch.randn(D, D, dtype=F))[0][:3]
    vals = torch.randn(3, V, dtype=F)
    S = torch.zeros(D, V, dtype=F)
    for k, v in zip(keys, vals):
        S = S + torch.outer(k, 1.0 * (v - S.T @ k))
    assert (keys @ S - vals).abs().max() < 1e-12
    S = S + torch.outer(keys[0], 1.0 * (vals[1] - S.T @ keys[0]))      # overwriting: the old value is taken off first
    assert ((keys @ S)[0] - vals[1]).abs().max() < 1e-12


def test_plain_model_in_pieces():
    """The plain recurrence carried over a cut equals the whole (which is what the engine's portions are held to)."""
    cfg = config(loop=None, layers=[parallel(conv=4)])
    w = plain.as_float64(plain.random_weights(cfg, 3))
    ids = list(range(30))
    whole, streams = plain.forward(ids, w, cfg)
    assert len(streams) == 1 and whole.shape == (30, 96)
    shorter, _ = plain.forward(ids[:17], w, cfg)
    assert (whole[:17] - shorter).abs().max() < 1e-10                   # causal: later tokens change nothing before them
