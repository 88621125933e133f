"""Several mixers side by side on the same input: y = sum_i scale_i * mixer_i(h).

The members' input products are one product (their weight rows stacked), and so are their output products: member
i writes scale_i times the operand of its output product into its columns of one buffer, and the members' output
weights lie side by side, so [Wo_1 | Wo_2] [s_1 a_1; s_2 a_2] = s_1 Wo_1 a_1 + s_2 Wo_2 a_2 comes out of one product
with one rounding. A member is any mixer that offers its middle part alone: `in_columns`, `out_columns`,
`weight_rows(get)`, `load_small(get)`, `out_weight(get)`, `bind_core(ctx)`, `core(in_buf, col, out_buf, out_col, batch,
cache)` and the constructor parameter `out_scale`. Their caches are joined by name (JoinedSpec); tensors are read under
`<member name>.<the member's own names>`.
"""
from __future__ import annotations

import torch

from .base import CacheView, Mixer
from .linear import Linear
from .registry import MIXERS
from .spec import JoinedSpec


@MIXERS.register("joined")
class JoinedMixers(Mixer):
    def __init__(self, hidden: int, members: list):
        """members: [(name, PartSpec of a mixer, scale)]."""
        self.hidden = hidden
        self.members = []
        col = out_col = 0
        for name, spec, scale in members:
            m = MIXERS.get(spec.kind)(hidden=hidden, **dict(spec.params, out_scale=float(scale)))
            if not hasattr(m, "core"):
                raise ValueError(f"mixer {spec.kind!r} does not offer its middle part alone and cannot be joined")
            self.members.append((name, m, col, out_col))
            col += -(-m.in_columns // 8) * 8
            out_col += -(-m.out_columns // 8) * 8
        self.proj = Linear(hidden, col)
        self.o = Linear(out_col, hidden)

    @property
    def capturable(self):
        return all(m.capturable for _, m, _, _ in self.members)

    @property
    def capturable_portions(self):
        return all(m.capturable_portions for _, m, _, _ in self.members)

    def cache_spec(self):
        return JoinedSpec({name: m.cache_spec() for name, m, _, _ in self.members})

    def tensors(self):
        return {f"{name}.{n}": s for name, m, _, _ in self.members for n, s in m.tensors().items()}

    def load(self, get):
        rows, cols = [], []
        for name, m, _, _ in self.members:
            sub = lambda n, _p=name + ".", **kw: get(_p + n, **kw)
            w = m.weight_rows(sub)
            pad = -(-w.shape[0] // 8) * 8 - w.shape[0]
            rows.append(torch.cat([w, w.new_zeros(pad, self.hidden)], dim=0) if pad else w)
            o = m.out_weight(sub)
            pad = -(-o.shape[1] // 8) * 8 - o.shape[1]
            cols.append(torch.cat([o, o.new_zeros(self.hidden, pad)], dim=1) if pad else o)
            m.load_small(sub)
        self.proj.set_weight(torch.cat(rows, dim=0))
        self.o.set_weight(torch.cat(cols, dim=1))

    def bind(self, ctx):
        ws = ctx.workspace
        self.proj_buf = ws.buffer("joined_proj", self.proj.out_features)
        self.mid_buf = ws.buffer("joined_mid", self.o.in_features)
        self.out_buf = ws.buffer("mixer_out", self.hidden)
        if any(-(-m.out_columns // 8) * 8 != m.out_columns for _, m, _, _ in self.members):
            self.mid_buf.zero_()      # padding columns meet zero weights, but must hold numbers
        for _, m, _, _ in self.members:
            m.bind_core(ctx)

    def forward(self, x, batch, cache: CacheView):
        T = batch.num_tokens
        self.proj.forward(x, self.proj_buf, T, scratch=True)
        for name, m, col, out_col in self.members:
            m.core(self.proj_buf, col, self.mid_buf, out_col, batch, cache.child(name))
        return self.o.forward(self.mid_buf, self.out_buf, T, scratch=True)
