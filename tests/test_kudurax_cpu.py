"""Kudurax without a GPU: its configuration reader and refusals, the model description built from it (tensor names,
run order, borrowed caches), random-weight folders, the latent cache's geometry, and the plain implementation
pinned by library routines and hand-made cases."""
import json
import math

import pytest
import torch

import plain_kudurax as plain

F = torch.float64


def tiny(**over):
    m = dict(heads=2, dim=8, rot_dim=4, vdim=6, kv_rank=16, scale=0.3, rot=dict(base=100.0, dims=4))
    cfg = dict(architecture="Kudurax", vocab=50, width=24, embedding=dict(scale=3.0), norm=dict(eps=1e-5), layers=[
        dict(type="latent_attention", mixer=dict(m), mlp=dict(kind="dense", ff=40)),
        dict(type="latent_attention", mixer=dict(m, kv_from=0),
             mlp=dict(kind="moe", router=dict(experts=3, top=2), expert=dict(ff=8), shared=dict(ff=12))),
        dict(type="latent_attention", mixer=dict(m, rot=dict(base=100.0, dims=4, scaling=dict(factor=2.0, original=16, fast=4.0, slow=1.0))),
             mlp=None)])
    cfg.update(over)
    return cfg


def test_config_reads_every_size_and_round_trips():
    from dinfer_amd.config import architecture_of
    from dinfer_amd.config.kudurax import KuduraxConfig
    d = tiny()
    assert architecture_of(d).name == "Kudurax"
    cfg = KuduraxConfig.from_dict(d)
    assert (cfg.vocab, cfg.width, cfg.embedding_scale, cfg.norm_eps, len(cfg.layers)) == (50, 24, 3.0, 1e-5, 3)
    assert cfg.layers[1].mixer.kv_from == 0 and cfg.layers[0].mixer.kv_from is None
    assert cfg.layers[2].mlp is None and cfg.layers[1].mlp.shared_ff == 12 and cfg.layers[1].mlp.top == 2
    assert cfg.layers[2].mixer.rot_scaling.factor == 2.0 and cfg.layers[0].mixer.rot_scaling is None
    assert cfg.to_dict() == d


@pytest.mark.parametrize("spoil, names", [
    (lambda d: d.pop("vocab"), "vocab"),
    (lambda d: d["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda d: d["layers"][0].update(type="other"), "type"),
    (lambda d: d["layers"][1]["mixer"].update(kv_from=2), "kv_from"),
    (lambda d: d["layers"][1]["mixer"].update(rot_dim=8, rot=dict(base=100.0, dims=8)), "rotation"),
    (lambda d: d["layers"][1]["mlp"]["router"].update(top=4), "top"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=6), "dims"),
    (lambda d: d["layers"][0]["mlp"].update(kind="gated"), "kind"),
    (lambda d: d["norm"].update(eps="small"), "eps"),
])
def test_config_refusals_name_the_key(spoil, names):
    from dinfer_amd.config import ConfigError
    from dinfer_amd.config.kudurax import KuduraxConfig
    d = tiny()
    spoil(d)
    with pytest.raises(ConfigError, match=names):
        KuduraxConfig.from_dict(d)


def test_model_description_names_and_run_order():
    from dinfer_amd.config.kudurax import KuduraxConfig
    from dinfer_amd.models.kudurax import build_spec
    from dinfer_amd.parts.model import DecoderModel, expected_tensors
    spec = build_spec(KuduraxConfig.from_dict(tiny()))
    names, optional = expected_tensors(spec)
    assert not optional and spec.stream_dtype == "float32" and spec.embed_scale == 3.0
    want = set(plain.random_weights(tiny(), 0))
    assert set(names) == want
    assert "l1.mix.dkv" not in names and "l2.norm2" not in names and "l1.mlp.shared.sg" in names
    assert tuple(names["l1.mlp.shared.sg"].shape) == (1, 24) and tuple(names["l0.mix.uk"].shape) == (16, 16)
    model = DecoderModel(spec)
    assert [(e.layer, e.cache) for e in model.run] == [(0, 0), (1, 0), (2, 2)]


def test_random_weight_folder_fits_the_model(tmp_path):
    from dinfer_amd.config import load_config
    from dinfer_amd.config.kudurax import KuduraxConfig
    from dinfer_amd.parts.model import DecoderModel
    from dinfer_amd.weights import WeightLoader, write_random_model
    write_random_model(KuduraxConfig.from_dict(tiny()), tmp_path, seed=3)
    arch, cfg = load_config(tmp_path)
    assert arch.name == "Kudurax" and cfg.to_dict() == tiny()
    model = DecoderModel(arch.build_spec(cfg))
    loader = WeightLoader(tmp_path, torch.device("cpu"), torch.float32)
    loader.check(*model.expected_tensors())
    loader.close()


def test_latent_cache_geometry():
    from dinfer_amd.parts.spec import LatentSpec
    a, b = LatentSpec(64, 16), LatentSpec(64, 16, transposed=True)
    assert a.page_bytes(16, torch.bfloat16) == 16 * 80 * 2 and b.page_bytes(16, torch.bfloat16) == 16 * 144 * 2
    assert a.group_key() != b.group_key() != LatentSpec(64, 8, transposed=True).group_key()
    t = b.allocate(5, 8, 3, torch.float32, torch.device("cpu"))
    assert tuple(t["latent"].shape) == (5, 8, 80) and tuple(t["latent_t"].shape) == (5, 64, 8)
    assert a.recomputable and a.window is None


# ---- the plain implementation, pinned ------------------------------------------------------------------------------
def test_plain_layer_norm_and_rotation_against_library_routines():
    x = torch.randn(5, 24, dtype=F)
    w, b = torch.randn(24, dtype=F), torch.randn(24, dtype=F)
    assert torch.allclose(plain.layer_norm(x, w, b, 1e-5), torch.nn.functional.layer_norm(x, (24,), w, b, 1e-5))
    # a rotation of pairs (2i, 2i+1) is a multiplication of complex numbers
    q = torch.randn(7, 3, 8, dtype=F)
    pos = torch.arange(3, 10)
    got = plain.rotate_interleaved(q, pos, 8, 50.0, None)
    f = 50.0 ** (-torch.arange(4, dtype=F) / 4)
    turn = torch.polar(torch.ones(7, 4, dtype=F), pos.to(F)[:, None] * f)
    want = torch.view_as_real(torch.view_as_complex(q.reshape(7, 3, 4, 2)) * turn[:, None, :]).reshape(7, 3, 8)
    assert torch.allclose(got, want)
    assert torch.allclose(got.norm(dim=-1), q.norm(dim=-1))       # unscaled: lengths stay
    part = plain.rotate_interleaved(q, pos, 4, 50.0, None)
    assert torch.equal(part[..., 4:], q[..., 4:])                # entries beyond `dims` pass unchanged


def test_plain_scaled_frequencies_by_hand():
    # dims 8, base 10000, original 2048: pair i makes original * f_i / (2 pi) turns: 326, 32.6, 3.26, 0.326.
    # fast 32 -> d = 1.008 -> lo 1; slow 1 -> d = 2.51 -> hi 3: pair 0 and 1 keep their speed, pair 2 is half-way, pair 3 slowed
    sc = dict(factor=8.0, original=2048, fast=32.0, slow=1.0)
    f, m = plain.rotary_frequencies(8, 10000.0, sc)
    f0 = 10000.0 ** (-torch.arange(4, dtype=F) / 4)
    assert torch.allclose(f[:2], f0[:2]) and torch.allclose(f[3], f0[3] / 8)
    assert torch.allclose(f[2], f0[2] * (0.5 / 8 + 0.5))
    assert abs(m - (0.1 * math.log(8.0) + 1)) < 1e-15


def test_plain_routing_rules():
    cfg = tiny()
    w = plain.random_weights(cfg, 1)
    h = torch.randn(9, 24, dtype=F)
    mlp = cfg["layers"][1]["mlp"]
    # all experts chosen: the plain softmax mixture of every expert plus the gated shared one
    every = dict(mlp, router=dict(experts=3, top=3))
    z = h @ w["l1.mlp.router"].to(F).T
    mix = sum(torch.softmax(z, -1)[:, e:e + 1] * plain.gated_expert(h, w, f"l1.mlp.e{e}.") for e in range(3))
    mix = mix + torch.sigmoid(h @ w["l1.mlp.shared.sg"].to(F).T) * plain.gated_expert(h, w, "l1.mlp.shared.")
    assert torch.allclose(plain.routed_ff(h, w, "l1.mlp.", every), mix)
    # one expert chosen: its weight is 1, and among equal logits the lowest index wins
    w["l1.mlp.router"][2] = w["l1.mlp.router"][0]
    one = dict(mlp, router=dict(experts=3, top=1), shared=None)
    z = h @ w["l1.mlp.router"].to(F).T
    want = torch.stack([plain.gated_expert(h[t:t + 1], w, f"l1.mlp.e{int(z[t].argmax()) if z[t].argmax() != 2 else 0}.")[0] for t in range(9)])
    assert torch.allclose(plain.routed_ff(h, w, "l1.mlp.", one), want)


def test_plain_model_in_pieces_equals_whole():
    cfg = tiny()
    w = plain.random_weights(cfg, 2)
    ids = [int(t) for t in torch.randint(0, 50, (23,))]
    whole = plain.forward(cfg, w, ids)
    latents, rows = {}, []
    for lo, hi in ((0, 7), (7, 8), (8, 20), (20, 23)):
        rows.append(plain.forward(cfg, w, ids[lo:hi], start=lo, latents=latents))
    assert torch.allclose(torch.cat(rows), whole, atol=1e-10)
    # a later token changes nothing before it
    other = plain.forward(cfg, w, ids[:12] + [(ids[12] + 1) % 50] + ids[13:])
    assert torch.allclose(other[:12], whole[:12]) and not torch.allclose(other[12:], whole[12:])
