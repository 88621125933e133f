"""Karopel: configuration -> ModelSpec.

embed -> run list of sandwich blocks( mixer | gated silu feed-forward or none ) -> norm -> head -> logits * logit_scale.
A block: h += m * norm1b(mixer(norm1(h))); h += m * norm2b(ff(norm2(h))), root-mean-square norms whose gains are stored
around zero, a 32-bit residual stream. Mixers: `attention` (grouped-query attention, per-head q/k norm with plain
gains shared by the heads, rotation of pairs (2i, 2i+1) on the first rot.dims entries with frequencies slowed by
wavelength, a window that keeps the first tokens, a learned sink a head) or `parallel` (a windowed attention without
rotation whose values are its keys, with a slope times the distance taken off the scores, beside a gated delta rule,
the two scaled and summed). `loop`: layers start .. stop-1 appear `times` times in the run list, each appearance with a
cache of its own; each pass starts by adding `loop.step[pass]`, and every pass but the first the embeddings as well.
Tensor names: embed, loop.step, l<i>.norm{1,1b,2,2b}, l<i>.mix.{q, k, v, q.norm, k.norm, sink, o} or
l<i>.mix.left.{q, k, o} and l<i>.mix.right.{q, k, v, q.conv, k.conv, v.conv, b, a, A_log, dt_bias, g, norm, o},
l<i>.mlp.{gate, up, down}, final.norm, head.
"""
from __future__ import annotations

from ..config.karopel import AttentionConfig, KaropelConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, RunEntry, part

SLOPE_EXP = 8.0      # the distance bias of head h of H is 2^(-8 (h + 1) / H) a token


def _attention(cfg: KaropelConfig, a: AttentionConfig, plain_left: bool):
    names = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "sink": "sink"}
    if plain_left:
        return part("attention", heads=a.heads, kv_heads=a.kv_heads, head_dim=a.dim, position=part("none"), window=a.window,
                    scale=a.scale, slope_exp=SLOPE_EXP, values_are_keys=True, names=names)
    if a.rot_base is None or a.rot_dims == 0:      # no rotation, or one of no entries
        position = part("none")
    else:
        s = a.rot_scaling
        position = part("rotary", theta=a.rot_base, max_positions=cfg.MAX_POSITIONS, rotary_dim=a.rot_dims, style="interleaved",
                        scaling=None if s is None else dict(kind="wavelength_bands", factor=s.factor, low=s.low,
                                                            high=s.high, original=s.original))
    return part("attention", heads=a.heads, kv_heads=a.kv_heads, head_dim=a.dim, v_dim=a.vdim, position=position,
                qk_norm=part("rmsnorm", eps=cfg.norm_eps, weight_name=""), window=a.window, keep_first=a.keep_first,
                scale=a.scale, sink=True, names=names)


def build_spec(cfg: KaropelConfig) -> ModelSpec:
    norm = part("rmsnorm", eps=cfg.norm_eps, weight_offset=1.0, weight_name="")
    layers = []
    for i, l in enumerate(cfg.layers):
        if l.type == "attention":
            mixer = _attention(cfg, l.mixer, plain_left=False)
        else:
            p, r = l.mixer, l.mixer.right
            right = part("delta_rule", heads=r.heads, qk_heads=r.kv_heads, dim=r.dim, vdim=r.vdim, taps=r.conv,
                         norm_eps=cfg.norm_eps)
            mixer = part("joined", members=[("left", _attention(cfg, p.left, plain_left=True), p.left_scale),
                                            ("right", right, p.right_scale)])
        ff = part("none") if l.ff is None else part("gated_mlp", intermediate=l.ff, act="silu", names=("gate", "up", "down"))
        layers.append(LayerSpec(block=part("sandwich", mult=cfg.residual_mult), mixer=mixer, feed_forward=ff, norm=norm,
                                prefix=f"l{i}."))
    n, lp = len(layers), cfg.loop
    if lp is None:
        run = [RunEntry(i) for i in range(n)]
    else:
        run = [RunEntry(i) for i in range(lp.start)]
        for t in range(lp.times):
            start = part("pass_start", table="loop.step", rows=lp.times, row=t, add_embedding=t > 0)
            run += [RunEntry(i, before=start if i == lp.start else None) for i in range(lp.start, lp.stop)]
        run += [RunEntry(i) for i in range(lp.stop, n)]
    return ModelSpec(
        architecture=cfg.ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=cfg.width, max_positions=cfg.MAX_POSITIONS,
        layers=layers, run=run, final_norm=norm, final_norm_name="final.norm", embed_name="embed", head_name="head",
        tie_embeddings=False, eos_token_ids=(), stream_dtype="float32",
        logits_post=None if cfg.logit_scale == 1.0 else part("scale_softcap", scale=cfg.logit_scale))


register_architecture(KaropelConfig.ARCHITECTURE, KaropelConfig, build_spec)
