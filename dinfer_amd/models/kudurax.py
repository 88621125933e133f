"""Kudurax: configuration -> ModelSpec.

embed * scale -> N x prenorm block( latent attention with an output gate | relu^2 feed-forward, routed experts with a
shared expert, or none ) -> layer norm -> head. Layer norms with bias, a 32-bit residual stream, rotation of pairs
(2i, 2i+1) with optional YaRN scaling. Tensor names: embed, l<i>.norm1(.b), l<i>.norm2(.b), l<i>.mix.{q, dkv,
dkv.norm, uk, uv, g, o}, l<i>.mlp.{up, down} or l<i>.mlp.{router, e<j>.{gate, up, down}, shared.{gate, up, down, sg}},
final.norm(.b), head. A layer with `kv_from` runs on the cache of the layer it names (a run entry that borrows).
"""
from __future__ import annotations

from ..config.kudurax import KuduraxConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, RunEntry, part


def build_spec(cfg: KuduraxConfig) -> ModelSpec:
    norm = part("layernorm", eps=cfg.norm_eps, bias=True, weight_name="", bias_name=".b")
    layers, run = [], []
    for i, l in enumerate(cfg.layers):
        m = l.mixer
        sc = m.rot_scaling
        position = part("rotary", theta=m.rot_base, max_positions=cfg.MAX_POSITIONS, rotary_dim=m.rot_dims, style="interleaved",
                        scaling=None if sc is None else dict(factor=sc.factor, original=sc.original, fast=sc.fast, slow=sc.slow))
        mixer = part("latent_attention", heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim, rank=m.kv_rank,
                     scale=m.scale, position=position, latent_norm=part("rmsnorm", eps=cfg.norm_eps, weight_name=""),
                     gated=True, shares_cache=m.kv_from is not None)
        f = l.mlp
        if f is None:
            ff = part("none")
        elif f.kind == "dense":
            ff = part("mlp", intermediate=f.ff, act="relu2", names=("up", "down"))
        else:
            ff = part("moe", experts=f.experts, top=f.top, intermediate=f.ff, shared_intermediate=f.shared_ff, act="silu")
        layers.append(LayerSpec(block=part("prenorm", mixer_prefix="mix.", ff_prefix="mlp.", norm_in="norm1", norm_post="norm2"),
                                mixer=mixer, feed_forward=ff, norm=norm, prefix=f"l{i}."))
        run.append(RunEntry(i, m.kv_from))     # layer i is run entry i, so a layer index names the entry whose cache is read
    return ModelSpec(
        architecture=cfg.ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=cfg.width, max_positions=cfg.MAX_POSITIONS,
        layers=layers, run=run, final_norm=norm, final_norm_name="final.norm", embed_name="embed", head_name="head",
        tie_embeddings=False, eos_token_ids=(), embed_scale=cfg.embedding_scale, stream_dtype="float32")


register_architecture(KuduraxConfig.ARCHITECTURE, KuduraxConfig, build_spec)
