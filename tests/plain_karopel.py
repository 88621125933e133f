"""A plain, slow Karopel in float64 on the CPU: one function per mechanism, whole sequences at once, no cache.
It shares nothing with the engine; the tests compare the engine with it.

cfg is the parsed config.json (a dict), w a dict name -> float64 tensor.
"""
import math

import torch

F = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, weight, eps):
    """The layer norms and the model's norm: the gain is stored as its distance from one."""
    return rms_unit(x, eps) * (1.0 + weight)


def norm_plain(x, weight, eps):
    return rms_unit(x, eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def rotary_frequencies(rot):
    """One frequency a pair: base^(-2i/dims), then slowed where the wavelength is long (three zones)."""
    dims = rot["dims"]
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = rot["base"] ** (-2.0 * i / dims)
        if sc:
            wavelength = 2 * math.pi / f
            if wavelength < sc["original"] / sc["high"]:
                pass
            elif wavelength > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            else:
                s = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
                f = (1 - s) * f / sc["factor"] + s * f
        out.append(f)
    return torch.tensor(out, dtype=F)


def rotate_pairs(x, positions, rot):
    """x [T, heads, dim]: entries (2i, 2i+1) of the first rot['dims'] turn by position * f_i; the rest stay."""
    dims = rot["dims"]
    f = rotary_frequencies(rot)
    ang = positions.to(F)[:, None] * f[None, :]                 # [T, dims/2]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    y = x.clone()
    y[..., 0:dims:2] = a * c - b * s
    y[..., 1:dims:2] = b * c + a * s
    return y


def visible(T, size, keep_first=0):
    """[T, T] bool: row i sees column j."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def softmax_rows(scores, mask, sink=None):
    """Softmax over the visible columns; with a sink the denominator holds exp(sink) once more."""
    s = scores.masked_fill(~mask, float("-inf"))
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, torch.full_like(m, float(sink)))
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + math.exp(float(sink)) * torch.exp(-m)
    return e / den


def attention(h, w, p, m, eps):
    """The mixer 'attention'. h [T, width]; p the tensor prefix ('l0.mix'); m the mixer's config."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + ".q"].T).view(T, H, D)
    k = (h @ w[p + ".k"].T).view(T, G, D)
    v = (h @ w[p + ".v"].T).view(T, G, V)
    q = norm_plain(q, w[p + ".q.norm"], eps)
    k = norm_plain(k, w[p + ".k.norm"], eps)
    pos = torch.arange(T)
    if m.get("rot"):
        q, k = rotate_pairs(q, pos, m["rot"]), rotate_pairs(k, pos, m["rot"])
    mask = visible(T, m["mask"]["size"], m["mask"].get("keep_first", 0))
    out = torch.zeros(T, H, V, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        out[:, hd] = softmax_rows(s, mask, w[p + ".sink"][hd]) @ v[:, g]
    return out.reshape(T, H * V) @ w[p + ".o"].T


def biased_window_attention(h, w, p, m):
    """The left half of 'parallel': values are the keys, no rotation, a slope times the distance taken off."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[p + ".q"].T).view(T, H, D)
    k = (h @ w[p + ".k"].T).view(T, G, D)
    mask = visible(T, m["mask"]["size"])
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(F)
    out = torch.zeros(T, H, D, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        slope = 2.0 ** (-8.0 * (hd + 1) / H)
        s = (q[:, hd] @ k[:, g].T) * m["scale"] - slope * dist
        out[:, hd] = softmax_rows(s, mask) @ k[:, g]
    return out.reshape(T, H * D) @ w[p + ".o"].T


def short_convolution(x, taps):
    """x [T, C], taps [C, K]: y_t = sum_j taps[:, K-1-j] x_{t-j}, zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for j in range(K):
        if j < T:
            y[j:] += x[:T - j] * taps[:, K - 1 - j]
    return y


def gated_delta_rule(h, w, p, m, eps):
    """The right half of 'parallel'."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(h @ w[p + ".q"].T, w[p + ".q.conv"])).view(T, G, D)
    k = silu(short_convolution(h @ w[p + ".k"].T, w[p + ".k.conv"])).view(T, G, D)
    v = silu(short_convolution(h @ w[p + ".v"].T, w[p + ".v.conv"])).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + ".b"].T)                                        # [T, H]
    decay = torch.exp(-torch.exp(w[p + ".A_log"]) * softplus(h @ w[p + ".a"].T + w[p + ".dt_bias"]))
    gate = silu(h @ w[p + ".g"].T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(D, V, dtype=F)
        for t in range(T):
            S = decay[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hd] = S.T @ q[t, g]
    o = norm_plain(o, w[p + ".norm"], eps) * gate
    return o.reshape(T, H * V) @ w[p + ".o"].T


def parallel(h, w, p, m, eps):
    left = biased_window_attention(h, w, p + ".left", m["left"])
    right = gated_delta_rule(h, w, p + ".right", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def feed_forward(h, w, p):
    return (silu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def layer(x, w, i, spec, cfg):
    eps, mult, p = cfg["norm"]["eps"], cfg["residual_mult"], f"l{i}"
    h = norm_around_zero(x, w[p + ".norm1"], eps)
    if spec["type"] == "attention":
        y = attention(h, w, p + ".mix", spec["mixer"], eps)
    elif spec["type"] == "parallel":
        y = parallel(h, w, p + ".mix", spec["mixer"], eps)
    else:
        raise ValueError(spec["type"])
    x = x + mult * norm_around_zero(y, w[p + ".norm1b"], eps)
    if spec.get("mlp"):
        y = feed_forward(norm_around_zero(x, w[p + ".norm2"], eps), w, p + ".mlp")
        x = x + mult * norm_around_zero(y, w[p + ".norm2b"], eps)
    return x


def run_order(cfg):
    """[(layer index, pass number or None, first of its pass)]."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["times"] <= 0 or loop["stop"] <= loop["start"]:
        return [(i, None, False) for i in range(n)]
    order = [(i, None, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None, False) for i in range(loop["stop"], n)]


def forward(tokens, w, cfg):
    """-> (logits [T, vocab], [the stream after every layer run])."""
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x, streams = x0, []
    for i, t, first in run_order(cfg):
        if first:
            if t > 0:
                x = x + x0
            x = x + w["loop.step"][t]
        x = layer(x, w, i, cfg["layers"][i], cfg)
        streams.append(x)
    y = norm_around_zero(x, w["final.norm"], cfg["norm"]["eps"])
    return (y @ w["head"].T) * cfg["logit_scale"], streams


def tensor_shapes(cfg):
    """name -> shape of every tensor a model of this configuration has, written out from the design."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,), "head": (cfg["vocab"], W)}
    if cfg.get("loop"):
        out["loop.step"] = (cfg["loop"]["times"], W)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (W,)
        if l["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * D, W), p + "mix.k": (G * D, W), p + "mix.v": (G * V, W), p + "mix.q.norm": (D,),
                        p + "mix.k.norm": (D,), p + "mix.sink": (H,), p + "mix.o": (W, H * V)})
        else:
            a, r = m["left"], m["right"]
            out.update({p + "mix.left.q": (a["heads"] * a["dim"], W), p + "mix.left.k": (a["kv_heads"] * a["dim"], W),
                        p + "mix.left.o": (W, a["heads"] * a["dim"])})
            H, G, D, V, K = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
            q = p + "mix.right."
            out.update({q + "q": (G * D, W), q + "k": (G * D, W), q + "v": (H * V, W), q + "q.conv": (G * D, K),
                        q + "k.conv": (G * D, K), q + "v.conv": (H * V, K), q + "b": (H, W), q + "a": (H, W),
                        q + "A_log": (H,), q + "dt_bias": (H,), q + "g": (H * V, W), q + "norm": (V,), q + "o": (W, H * V)})
        if l.get("mlp"):
            ff = l["mlp"]["ff"]
            out[p + "norm2"] = out[p + "norm2b"] = (W,)
            out.update({p + "mlp.gate": (ff, W), p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
    return out


def random_weights(cfg, seed):
    """bfloat16 tensors of sizes that keep every mechanism awake: products of unit spread, gains around their
    neutral value, sinks and decay parameters spread over a few units."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        x = torch.randn(shape, generator=g)
        if name in ("embed", "loop.step"):
            t = x * (1.0 if name == "embed" else 0.3)
        elif last in ("norm1", "norm1b", "norm2", "norm2b") or name == "final.norm":
            t = x * 0.15                                   # stored around zero
        elif name.endswith("q.norm") or name.endswith("k.norm") or name.endswith("right.norm"):
            t = 1.0 + x * 0.15
        elif last == "sink":
            t = x * 1.5
        elif last in ("A_log", "dt_bias"):
            t = x * 0.7
        elif last == "conv":
            t = x * 0.6
        else:
            t = x * (1.5 / shape[-1] ** 0.5)
        out[name] = t.to(torch.bfloat16)
    return out


def as_float64(w):
    return {k: v.to(F) for k, v in w.items()}
