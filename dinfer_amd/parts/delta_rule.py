"""Gated delta rule: a recurrent mixer with one float32 matrix S [dim, vdim] a head and request as its state.

With h the mixer's input, H heads, G query/key heads (head i reads query/key head i // (H / G)):

    q', k' = Wq h, Wk h  (G x dim)      v' = Wv h  (H x vdim)
    q, k, v = silu(conv(q')), silu(conv(k')), silu(conv(v'))     conv: a few taps a channel over time, causal, no bias
    q <- q / sqrt(sum q^2 + unit_eps) * dim^-1/2,   k <- k / sqrt(sum k^2 + unit_eps)       (per head)
    beta = sigmoid(Wb h),   g = exp(-exp(A_log) * softplus(Wa h + dt_bias))                 (per head)
    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q                         (per head, token by token)
    y = Wo concat_h( o_h / rms(o_h) * w * silu(Wg h)_h )

One product makes q' | k' | v' | gate | beta logits | decay logits; everything after it up to the operand of Wo is
float (csrc/delta.hip). The state and the convolution's last taps - 1 inputs live in the request's state slot
(DeltaStateSpec); a request's first step (position 0) starts from zeros. Prompt portions of any size and single rows
run the same kernels and leave the same bits.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import CacheView, Mixer
from .linear import Linear
from .registry import MIXERS
from .spec import DeltaStateSpec, TensorSpec


@MIXERS.register("delta_rule")
class GatedDeltaRule(Mixer):
    capturable = True            # every kernel reads slots, lengths and row counts from the batch's device buffers
    capturable_portions = True

    NAMES = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "b": "b", "a": "a",
             "A_log": "A_log", "dt_bias": "dt_bias", "g": "g", "norm": "norm", "o": "o"}

    def __init__(self, hidden: int, heads: int, qk_heads: int, dim: int, vdim: int, taps: int, norm_eps: float,
                 unit_eps: float = 1e-6, out_scale: float = 1.0, names: dict | None = None):
        if heads % qk_heads:
            raise ValueError(f"delta rule: heads {heads} not divisible by query/key heads {qk_heads}")
        if not (0 < dim <= ops.DELTA_MAX_DIM and 0 < vdim <= ops.DELTA_MAX_HEAD and 0 < taps <= ops.DELTA_MAX_TAPS):
            raise ValueError(f"delta rule: dim {dim}, vdim {vdim} or {taps} taps have no kernel (dim up to "
                             f"{ops.DELTA_MAX_DIM}, vdim up to {ops.DELTA_MAX_HEAD}, taps up to {ops.DELTA_MAX_TAPS})")
        self.hidden, self.heads, self.qk_heads, self.dim, self.vdim, self.taps = hidden, heads, qk_heads, dim, vdim, taps
        self.norm_eps, self.unit_eps, self.out_scale = float(norm_eps), float(unit_eps), float(out_scale)
        self.names = dict(self.NAMES, **(names or {}))
        self.qk_size, self.v_size = qk_heads * dim, heads * vdim
        self.channels = 2 * self.qk_size + self.v_size
        # columns of the fused product: q' | k' | v' | gate | beta | decay, padded to a multiple of 8
        self.g_off = self.channels
        self.b_off = self.g_off + self.v_size
        self.a_off = self.b_off + heads
        self.used = self.a_off + heads
        self.proj = Linear(hidden, -(-self.used // 8) * 8)
        self.o = Linear(self.v_size, hidden)

    def cache_spec(self):
        return DeltaStateSpec(self.heads, self.dim, self.vdim, self.channels, self.taps)

    def tensors(self):
        n, Hd = self.names, self.hidden
        return {n["q"]: TensorSpec((self.qk_size, Hd)), n["k"]: TensorSpec((self.qk_size, Hd)),
                n["v"]: TensorSpec((self.v_size, Hd)), n["g"]: TensorSpec((self.v_size, Hd)),
                n["b"]: TensorSpec((self.heads, Hd)), n["a"]: TensorSpec((self.heads, Hd)),
                n["q_conv"]: TensorSpec((self.qk_size, self.taps)), n["k_conv"]: TensorSpec((self.qk_size, self.taps)),
                n["v_conv"]: TensorSpec((self.v_size, self.taps)),
                n["A_log"]: TensorSpec((self.heads,)), n["dt_bias"]: TensorSpec((self.heads,)),
                n["norm"]: TensorSpec((self.vdim,), init="gain"), n["o"]: TensorSpec((Hd, self.v_size))}

    # ---- the middle part alone, for a mixer that joins several (parts/joined.py) ------------------
    @property
    def in_columns(self) -> int:
        return self.proj.out_features

    @property
    def out_columns(self) -> int:
        return self.v_size

    def out_weight(self, get) -> torch.Tensor:
        return get(self.names["o"], compute=True)

    def weight_rows(self, get) -> torch.Tensor:
        """The rows of the fused product, in the order of its columns (padding included)."""
        n = self.names
        w = torch.cat([get(n[k], compute=True) for k in ("q", "k", "v", "g", "b", "a")], dim=0)
        if w.shape[0] < self.proj.out_features:
            w = torch.cat([w, w.new_zeros(self.proj.out_features - w.shape[0], self.hidden)], dim=0)
        return w

    def load_small(self, get) -> None:
        n = self.names
        # small parameters in 32 bits (exact for a bfloat16 file): they enter the recurrence
        self.conv_taps = torch.cat([get(n[k]).float() for k in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.conv_taps_t = self.conv_taps.t().contiguous()      # [taps, channels]: 8 channels' taps in one load
        self.a_log = get(n["A_log"]).float().contiguous()
        self.dt_bias = get(n["dt_bias"]).float().contiguous()
        self.norm_weight = get(n["norm"]).float().contiguous()

    def load(self, get):
        self.proj.set_weight(self.weight_rows(get))
        self.load_small(get)
        self.o.set_weight(self.out_weight(get))

    def bind(self, ctx):
        ws = ctx.workspace
        self.proj_buf = ws.buffer("delta_proj", self.proj.out_features)
        self.gated_buf = ws.buffer("delta_gated", self.v_size)
        self.out_buf = ws.buffer("mixer_out", self.hidden)
        self.bind_core(ctx)

    def bind_core(self, ctx):
        ws = ctx.workspace
        self.work = ws.buffer("delta_work", ops.delta_work_columns(self.qk_heads, self.heads, self.dim, self.vdim),
                              dtype=torch.float32)
        self.o_buf = ws.buffer("delta_o", self.v_size, dtype=torch.float32)

    def forward(self, x, batch, cache: CacheView):
        T = batch.num_tokens
        self.proj.forward(x, self.proj_buf, T, scratch=True)
        self.core(self.proj_buf, 0, self.gated_buf, 0, batch, cache)
        return self.o.forward(self.gated_buf, self.out_buf, T, scratch=True)

    def core(self, proj_buf, col, gated_buf, out_col, batch, cache: CacheView):
        """Everything between the two products: this mixer's columns start at `col` of proj_buf, the operand of the
        output product goes to column `out_col` of gated_buf."""
        T, B = batch.num_tokens, batch.num_reqs
        common = dict(state_slots=batch.state_slots, cu_seqlens=batch.cu_seqlens, seq_lens=batch.seq_lens, num_reqs=B)
        sizes = dict(qk_heads=self.qk_heads, heads=self.heads, dim=self.dim, vdim=self.vdim)
        ops.delta_prep(proj_buf, T, qkv_off=col, b_off=col + self.b_off, a_off=col + self.a_off, taps=self.conv_taps,
                       a_log=self.a_log, dt_bias=self.dt_bias, conv_state=cache.conv, work=self.work,
                       eps=self.unit_eps, q_scale=self.dim ** -0.5, taps_t=self.conv_taps_t, **common, **sizes)
        if cache.owner:
            ops.delta_conv_update(proj_buf, qkv_off=col, conv_state=cache.conv, **common)
        ops.delta_recurrence(self.work, cache.state, self.o_buf, **common, **sizes)
        ops.delta_out(self.o_buf, proj_buf, col + self.g_off, self.norm_weight, gated_buf, T, heads=self.heads,
                      vdim=self.vdim, eps=self.norm_eps, col_off=out_col, out_scale=self.out_scale)
