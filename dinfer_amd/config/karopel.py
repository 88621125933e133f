"""Configuration of the Karopel architecture: a decoder whose layers are either windowed attention with a learned
sink and kept first tokens, or a windowed attention with a distance bias beside a gated delta rule; a norm before
and after every sublayer; a group of layers that may run several times.

config.json is nested; every size and every constant that may differ between models of the design is read from it:

    architecture    "Karopel"
    vocab, width, residual_mult, logit_scale
    norm.eps
    loop            null | {start, stop, times}: layers start .. stop-1 run `times` times in a row
    layers[i].type  "attention" | "parallel"
    layers[i].mixer attention: heads, kv_heads, dim, vdim, scale, mask{size, keep_first}, rot{base, dims, scaling{factor,
                    low, high, original} or null} or null
                    parallel:  left{heads, kv_heads, dim, vdim, scale, mask{size}}, right{heads, kv_heads, dim, vdim,
                    conv}, left_scale, right_scale
    layers[i].mlp   null | {kind: "dense", ff}
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .base import ConfigError, ModelConfig, coerce, key
from .kudurax import _num, _section


@dataclass(frozen=True)
class BandScaling:
    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    keep_first: int = 0
    rot_base: float | None = None      # None: no rotation
    rot_dims: int = 0
    rot_scaling: BandScaling | None = None


@dataclass(frozen=True)
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class ParallelConfig:
    left: AttentionConfig
    right: DeltaConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class KaropelLayer:
    type: str                    # "attention" | "parallel"
    mixer: object                # AttentionConfig | ParallelConfig
    ff: int | None               # inner size of the dense feed-forward, None for a layer without one


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


def _attention(m: dict, where: str, rotation: bool, keeps: bool) -> AttentionConfig:
    mask = _section(m, "mask", where)
    kw = {}
    if keeps and mask.get("keep_first") is not None:
        kw["keep_first"] = _num(mask, "keep_first", int, where + "mask.", positive=False)
        if kw["keep_first"] < 0:
            raise ConfigError(f"config key {where}'mask.keep_first' must not be negative, got {kw['keep_first']}")
    rot = m.get("rot") if rotation else None
    if rot is not None:
        if not isinstance(rot, dict):
            raise ConfigError(f"config key {where}'rot' must be an object or null, got {rot!r}")
        kw["rot_base"] = _num(rot, "base", float, where + "rot.")
        kw["rot_dims"] = _num(rot, "dims", int, where + "rot.", positive=False)
        if kw["rot_dims"] < 0:
            raise ConfigError(f"config key {where}'rot.dims' must not be negative, got {kw['rot_dims']}")
        sc = rot.get("scaling")
        if sc is not None:
            if not isinstance(sc, dict):
                raise ConfigError(f"config key {where}'rot.scaling' must be an object or null, got {sc!r}")
            kw["rot_scaling"] = BandScaling(*(_num(sc, k, float, where + "rot.scaling.") for k in ("factor", "low", "high", "original")))
            if not kw["rot_scaling"].high > kw["rot_scaling"].low:
                raise ConfigError(f"config key {where}'rot.scaling': 'high' must exceed 'low'")
    out = AttentionConfig(heads=_num(m, "heads", int, where), kv_heads=_num(m, "kv_heads", int, where),
                          dim=_num(m, "dim", int, where), vdim=_num(m, "vdim", int, where),
                          scale=_num(m, "scale", float, where), window=_num(mask, "size", int, where + "mask."), **kw)
    if out.heads % out.kv_heads:
        raise ConfigError(f"config key {where}'heads' {out.heads} is no multiple of 'kv_heads' {out.kv_heads}")
    if out.rot_base is not None and (out.rot_dims > out.dim or out.rot_dims % 2):
        raise ConfigError(f"config key {where}'rot.dims' must be even and at most dim {out.dim}, got {out.rot_dims}")
    return out


def _delta(m: dict, where: str) -> DeltaConfig:
    out = DeltaConfig(*(_num(m, k, int, where) for k in ("heads", "kv_heads", "dim", "vdim", "conv")))
    if out.heads % out.kv_heads:
        raise ConfigError(f"config key {where}'heads' {out.heads} is no multiple of 'kv_heads' {out.kv_heads}")
    return out


@dataclass(frozen=True)
class KaropelConfig(ModelConfig):
    vocab: int = key(int)
    width: int = key(int)
    residual_mult: float = key(float, 1.0)
    logit_scale: float = key(float, 1.0)
    norm_eps: float = field(default=1e-6)
    loop: Loop | None = field(default=None)
    layers: tuple = field(default=())

    ARCHITECTURE = "Karopel"
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
            typ, m = l.get("type"), _section(l, "mixer", where)
            if typ == "attention":
                mixer = _attention(m, where + "mixer.", rotation=True, keeps=True)
            elif typ == "parallel":
                left = _attention(_section(m, "left", where + "mixer."), where + "mixer.left.", rotation=False, keeps=False)
                if left.vdim != left.dim:
                    raise ConfigError(f"config key {where}'mixer.left.vdim': the values are the keys, so it must equal 'dim'")
                mixer = ParallelConfig(left, _delta(_section(m, "right", where + "mixer."), where + "mixer.right."),
                                       _num(m, "left_scale", float, where + "mixer.", positive=False),
                                       _num(m, "right_scale", float, where + "mixer.", positive=False))
            else:
                raise ConfigError(f"config key {where}'type': unknown mixer {typ!r} (known: 'attention', 'parallel')")
            f = l.get("mlp")
            ff = None
            if f is not None:
                if not isinstance(f, dict) or f.get("kind") != "dense":
                    raise ConfigError(f"config key {where}'mlp' must be null or an object of kind 'dense', got {f!r}")
                ff = _num(f, "ff", int, where + "mlp.")
            out.append(KaropelLayer(typ, mixer, ff))
        loop = d.get("loop")
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError(f"config key 'loop' must be an object or null, got {loop!r}")
            loop = Loop(_num(loop, "start", int, "loop.", positive=False), _num(loop, "stop", int, "loop.", positive=False),
                        _num(loop, "times", int, "loop."))
        return {"norm_eps": _num(_section(d, "norm", ""), "eps", float, "norm."), "loop": loop, "layers": tuple(out)}

    def check(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"config keys 'vocab' and 'width' must be positive, got {self.vocab} and {self.width}")
        lp = self.loop
        if lp is not None and not (0 <= lp.start < lp.stop <= len(self.layers)):
            raise ConfigError(f"config key 'loop': start {lp.start} and stop {lp.stop} must bound some of the "
                              f"{len(self.layers)} layers")

    def extra_to_dict(self) -> dict:
        def attention(a: AttentionConfig, keeps: bool, rotation: bool):
            o = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                 "mask": {"size": a.window}}
            if keeps:
                o["mask"]["keep_first"] = a.keep_first
            if rotation:
                o["rot"] = None
                if a.rot_base is not None:
                    s = a.rot_scaling
                    o["rot"] = {"base": a.rot_base, "dims": a.rot_dims,
                                "scaling": None if s is None else {"factor": s.factor, "low": s.low, "high": s.high,
                                                                   "original": s.original}}
            return o

        def mixer(l: KaropelLayer):
            if l.type == "attention":
                return attention(l.mixer, True, True)
            p, r = l.mixer, l.mixer.right
            return {"left": attention(p.left, False, False),
                    "right": {"heads": r.heads, "kv_heads": r.kv_heads, "dim": r.dim, "vdim": r.vdim, "conv": r.conv},
                    "left_scale": p.left_scale, "right_scale": p.right_scale}

        lp = self.loop
        return {"architecture": self.ARCHITECTURE, "norm": {"eps": self.norm_eps},
                "loop": None if lp is None else {"start": lp.start, "stop": lp.stop, "times": lp.times},
                "layers": [{"type": l.type, "mixer": mixer(l), "mlp": None if l.ff is None else {"kind": "dense", "ff": l.ff}}
                           for l in self.layers]}

    def to_dict(self) -> dict:
        out = {"vocab": self.vocab, "width": self.width, "residual_mult": self.residual_mult,
               "logit_scale": self.logit_scale}
        out.update(self.extra_to_dict())
        return out

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
