"""Configuration of the Kudurax architecture: a decoder of latent-attention layers, each with a dense or a routed
feed-forward (or none), layer norms with bias, a multiplied embedding and an untied head.

config.json is nested; every size and every constant that may differ between models of the design is read from it:

    architecture   "Kudurax"
    vocab, width
    embedding.scale
    norm.eps
    layers[i].type            "latent_attention"
    layers[i].mixer           heads, dim, rot_dim, vdim, kv_rank, scale, rot{base, dims, scaling{factor, original, fast,
                              slow} or null}, kv_from (optional: the layer whose cache this one reads)
    layers[i].mlp             null | {kind: "dense", ff} | {kind: "moe", router{experts, top}, expert{ff}, shared{ff} or null}
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .base import ConfigError, ModelConfig, coerce, key


def _section(d: dict, name: str, where: str) -> dict:
    v = d.get(name)
    if not isinstance(v, dict):
        raise ConfigError(f"config key {where}{name!r} must be an object, got {v!r}")
    return v


def _num(d: dict, name: str, typ: type, where: str, positive: bool = True):
    if name not in d:
        raise ConfigError(f"config.json lacks the required key {where}{name!r}")
    v = coerce(where + name, d[name], typ)
    if positive and not v > 0:
        raise ConfigError(f"config key {where}{name!r} must be positive, got {v!r}")
    return v


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_scaling: RotaryScaling | None
    kv_from: int | None


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                    # "dense" | "moe"
    ff: int                      # dense: its inner size; moe: an expert's
    experts: int = 0
    top: int = 0
    shared_ff: int | None = None


@dataclass(frozen=True)
class KuduraxLayer:
    type: str
    mixer: LatentMixerConfig
    mlp: FeedForwardConfig | None


def _mixer(m: dict, where: str) -> LatentMixerConfig:
    rot = _section(m, "rot", where)
    sc = rot.get("scaling")
    scaling = None
    if sc is not None:
        if not isinstance(sc, dict):
            raise ConfigError(f"config key {where}'rot.scaling' must be an object or null, got {sc!r}")
        scaling = RotaryScaling(*(_num(sc, k, float, where + "rot.scaling.") for k in ("factor", "original", "fast", "slow")))
    kv_from = m.get("kv_from")
    if kv_from is not None:
        kv_from = coerce(where + "kv_from", kv_from, int)
    out = LatentMixerConfig(
        heads=_num(m, "heads", int, where), dim=_num(m, "dim", int, where), rot_dim=_num(m, "rot_dim", int, where),
        vdim=_num(m, "vdim", int, where), kv_rank=_num(m, "kv_rank", int, where), scale=_num(m, "scale", float, where),
        rot_base=_num(rot, "base", float, where + "rot."), rot_dims=_num(rot, "dims", int, where + "rot."),
        rot_scaling=scaling, kv_from=kv_from)
    if out.rot_dims > out.rot_dim or out.rot_dims % 2:
        raise ConfigError(f"config key {where}'rot.dims' must be even and at most rot_dim {out.rot_dim}, got {out.rot_dims}")
    return out


def _mlp(f, where: str) -> FeedForwardConfig | None:
    if f is None:
        return None
    if not isinstance(f, dict):
        raise ConfigError(f"config key {where[:-1]!r} must be an object or null, got {f!r}")
    kind = f.get("kind")
    if kind == "dense":
        return FeedForwardConfig("dense", _num(f, "ff", int, where))
    if kind == "moe":
        router = _section(f, "router", where)
        shared = f.get("shared")
        if shared is not None and not isinstance(shared, dict):
            raise ConfigError(f"config key {where}'shared' must be an object or null, got {shared!r}")
        out = FeedForwardConfig("moe", _num(_section(f, "expert", where), "ff", int, where + "expert."),
                                experts=_num(router, "experts", int, where + "router."),
                                top=_num(router, "top", int, where + "router."),
                                shared_ff=_num(shared, "ff", int, where + "shared.") if shared is not None else None)
        if out.top > out.experts:
            raise ConfigError(f"config key {where}'router.top' {out.top} exceeds the {out.experts} experts")
        return out
    raise ConfigError(f"config key {where}'kind' must be 'dense' or 'moe', got {kind!r}")


@dataclass(frozen=True)
class KuduraxConfig(ModelConfig):
    vocab: int = key(int)
    width: int = key(int)
    embedding_scale: float = field(default=1.0)
    norm_eps: float = field(default=1e-5)
    layers: tuple = field(default=())

    ARCHITECTURE = "Kudurax"
    MAX_POSITIONS = (1 << 31) - 1     # the design sets no limit; positions are 32-bit in the batch

    @classmethod
    def extra_from_dict(cls, d: dict) -> dict:
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config key 'layers' must be a non-empty list")
        out = []
        for i, l in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(l, dict):
                raise ConfigError(f"config key 'layers[{i}]' must be an object")
            typ = l.get("type")
            if typ != "latent_attention":
                raise ConfigError(f"config key {where}'type': unknown mixer {typ!r} (known: 'latent_attention')")
            out.append(KuduraxLayer(typ, _mixer(_section(l, "mixer", where), where + "mixer."), _mlp(l.get("mlp"), where + "mlp.")))
        return {"embedding_scale": _num(_section(d, "embedding", ""), "scale", float, "embedding."),
                "norm_eps": _num(_section(d, "norm", ""), "eps", float, "norm."), "layers": tuple(out)}

    def extra_to_dict(self) -> dict:
        def mixer(m):
            rot = {"base": m.rot_base, "dims": m.rot_dims}
            if m.rot_scaling is not None:
                s = m.rot_scaling
                rot["scaling"] = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
            o = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                 "scale": m.scale, "rot": rot}
            if m.kv_from is not None:
                o["kv_from"] = m.kv_from
            return o

        def mlp(f):
            if f is None:
                return None
            if f.kind == "dense":
                return {"kind": "dense", "ff": f.ff}
            o = {"kind": "moe", "router": {"experts": f.experts, "top": f.top}, "expert": {"ff": f.ff}}
            if f.shared_ff is not None:
                o["shared"] = {"ff": f.shared_ff}
            return o

        return {"architecture": self.ARCHITECTURE, "embedding": {"scale": self.embedding_scale},
                "norm": {"eps": self.norm_eps},
                "layers": [{"type": l.type, "mixer": mixer(l.mixer), "mlp": mlp(l.mlp)} for l in self.layers]}

    def to_dict(self) -> dict:
        out = {"vocab": self.vocab, "width": self.width}
        out.update(self.extra_to_dict())
        return out

    def check(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"config keys 'vocab' and 'width' must be positive, got {self.vocab} and {self.width}")
        for i, l in enumerate(self.layers):
            j = l.mixer.kv_from
            if j is None:
                continue
            if not (0 <= j < i):
                raise ConfigError(f"layers[{i}].mixer.kv_from = {j} must name an earlier layer")
            src = self.layers[j].mixer
            if src.kv_from is not None:
                raise ConfigError(f"layers[{i}].mixer.kv_from = {j}: that layer has no down projection of its own")
            same = (src.kv_rank, src.rot_dim, src.rot_base, src.rot_dims, src.rot_scaling)
            if same != (l.mixer.kv_rank, l.mixer.rot_dim, l.mixer.rot_base, l.mixer.rot_dims, l.mixer.rot_scaling):
                raise ConfigError(f"layers[{i}] reads the cache of layer {j}: their kv_rank, rot_dim and rotation must be equal")

    # what programs that know no architecture ask a configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def max_position_embeddings(self) -> int:
        return self.MAX_POSITIONS

    @property
    def eos_token_ids(self) -> tuple:
        return ()
