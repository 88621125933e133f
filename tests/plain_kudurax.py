"""A plain, slow Kudurax in float64 torch on the CPU: the oracle the engine is compared with.

One function per mechanism, written from the design's equations; nothing here is shared with the
engine's code. Weights are a dict name -> tensor with the names of the weight file; the configuration
is the parsed config.json.

Notation: W width, H heads, dn / dr the unrotated / rotated query-key sizes of a head, dv the value
size of a head, R the latent size, E experts, k the experts a token uses.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def rotary_frequencies(dims: int, base: float, scaling: dict | None):
    """(frequencies [dims / 2], factor on cos and sin)."""
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1


def rotate_interleaved(x, positions, dims: int, base: float, scaling: dict | None):
    """x [T, ..., D]: the first `dims` entries of the last axis turn, (2i, 2i + 1) a pair; positions [T]."""
    f, m = rotary_frequencies(dims, base, scaling)
    ang = positions.to(F)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = (ang.cos() * m).view(shape), (ang.sin() * m).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_of(h, positions, w, p, m, eps):
    """What a layer with a down projection of its own keeps per token: (c [T, R], rotated key part [T, dr])."""
    R, dr = m["kv_rank"], m["rot_dim"]
    d = h @ w[p + "dkv"].to(F).T
    c = rms_norm(d[:, :R], w[p + "dkv.norm"].to(F), eps)
    kr = rotate_interleaved(d[:, R:R + dr], positions, m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    return c, kr


def latent_attention(h, positions, w, p, m, latent):
    """h [T, W] (one sequence, positions ascending from any start), latent = (c, kr) of all keys [S, ...] with key j at
    position j. Causal softmax attention with an output gate per head."""
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    c, kr = latent
    S = c.shape[0]
    q = (h @ w[p + "q"].to(F).T).view(T, H, dn + dr)
    qn = q[..., :dn]
    qr = rotate_interleaved(q[..., dn:], positions, m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    kn = (c @ w[p + "uk"].to(F).T).view(S, H, dn)
    v = (c @ w[p + "uv"].to(F).T).view(S, H, dv)
    s = (torch.einsum("thd,shd->hts", qn, kn) + torch.einsum("thd,sd->hts", qr, kr)) * m["scale"]
    hidden = torch.arange(S)[None, :] > positions[:, None]
    a = torch.softmax(s.masked_fill(hidden[None], float("-inf")), dim=-1)
    o = torch.einsum("hts,shd->thd", a, v)
    g = torch.sigmoid(h @ w[p + "g"].to(F).T)
    o = o * g[:, :, None]
    return o.reshape(T, H * dv) @ w[p + "o"].to(F).T


def dense_ff(h, w, p):
    return torch.relu(h @ w[p + "up"].to(F).T) ** 2 @ w[p + "down"].to(F).T


def gated_expert(h, w, p):
    a = h @ w[p + "gate"].to(F).T
    return (a * torch.sigmoid(a) * (h @ w[p + "up"].to(F).T)) @ w[p + "down"].to(F).T


def routed_ff(h, w, p, mlp, forced=None):
    """forced [T, k]: experts to use instead of the k best. Where rounding makes a close call go the other way the
    rest of the computation can still be judged; every forced expert must be within a hair of the k best."""
    E, k = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ w[p + "router"].to(F).T
    idx = torch.argsort(-z, dim=-1, stable=True)[:, :k]      # the k largest; among equals the lowest index
    if forced is not None:
        kth = torch.gather(z, 1, idx)[:, -1:]
        behind = (kth - torch.gather(z, 1, forced)).max().item()
        assert behind <= 0.08 * z.std().item(), f"a forced expert is {behind:.3f} behind the k-th best: no close call"
        assert all(len(set(row)) == k for row in forced.tolist()), "an expert is chosen twice"
        idx = forced
    top = torch.gather(z, 1, idx)
    share = torch.softmax(top, dim=-1)
    out = torch.zeros_like(h)
    for e in range(E):
        rows, slot = (idx == e).nonzero(as_tuple=True)
        if rows.numel():
            out[rows] += gated_expert(h[rows], w, f"{p}e{e}.") * share[rows, slot][:, None]
    if mlp.get("shared"):
        out = out + gated_expert(h, w, p + "shared.") * torch.sigmoid(h @ w[p + "shared.sg"].to(F).T)
    return out


def forward(cfg: dict, w: dict, tokens, start: int = 0, latents: dict | None = None, layers_out: list | None = None,
            choices: dict | None = None):
    """Logits [T, vocab] of one sequence's tokens at positions start.. . latents: layer -> (c, kr) of the positions
    before `start`, extended in place, so that a sequence can be fed in pieces. choices: layer -> [T, k] experts that
    its routed feed-forward is to use (see routed_ff)."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.numel()
    positions = torch.arange(start, start + T)
    x = w["embed"].to(F)[tokens] * cfg["embedding"]["scale"]
    latents = {} if latents is None else latents
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        assert layer["type"] == "latent_attention"
        m = layer["mixer"]
        h = layer_norm(x, w[p + "norm1"].to(F), w[p + "norm1.b"].to(F), eps)
        src = m.get("kv_from")
        if src is None:
            c, kr = latent_of(h, positions, w, p + "mix.", m, eps)
            if i in latents:
                c, kr = torch.cat([latents[i][0], c]), torch.cat([latents[i][1], kr])
            latents[i] = (c, kr)
            src = i
        x = x + latent_attention(h, positions, w, p + "mix.", m, latents[src])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = layer_norm(x, w[p + "norm2"].to(F), w[p + "norm2.b"].to(F), eps)
            forced = None if choices is None else choices.get(i)
            x = x + (dense_ff(h, w, p + "mlp.") if mlp["kind"] == "dense" else routed_ff(h, w, p + "mlp.", mlp, forced))
        if layers_out is not None:
            layers_out.append(x.clone())
    x = layer_norm(x, w["final.norm"].to(F), w["final.norm.b"].to(F), eps)
    return x @ w["head"].to(F).T


def random_weights(cfg: dict, seed: int, spread: float = 1.0) -> dict:
    """name -> bfloat16 tensor for every tensor the configuration asks for; matrices N(0, spread / sqrt(inputs))."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    out = {}

    def mat(name, rows, cols):
        out[name] = (torch.randn(rows, cols, generator=g) * spread / math.sqrt(cols)).to(torch.bfloat16)

    def norm(name, n, bias=True):
        out[name] = (1 + 0.2 * torch.randn(n, generator=g)).to(torch.bfloat16)
        if bias:
            out[name + ".b"] = (0.1 * torch.randn(n, generator=g)).to(torch.bfloat16)

    out["embed"] = (torch.randn(cfg["vocab"], W, generator=g) / math.sqrt(W)).to(torch.bfloat16)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        norm(p + "norm1", W)
        mat(p + "mix.q", H * (dn + dr), W)
        if m.get("kv_from") is None:
            mat(p + "mix.dkv", R + dr, W)
            norm(p + "mix.dkv.norm", R, bias=False)
        mat(p + "mix.uk", H * dn, R)
        mat(p + "mix.uv", H * dv, R)
        mat(p + "mix.g", H, W)
        mat(p + "mix.o", W, H * dv)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        norm(p + "norm2", W)
        if mlp["kind"] == "dense":
            mat(p + "mlp.up", mlp["ff"], W)
            mat(p + "mlp.down", W, mlp["ff"])
        else:
            for e in range(mlp["router"]["experts"]):
                mat(f"{p}mlp.e{e}.gate", mlp["expert"]["ff"], W)
                mat(f"{p}mlp.e{e}.up", mlp["expert"]["ff"], W)
                mat(f"{p}mlp.e{e}.down", W, mlp["expert"]["ff"])
            mat(p + "mlp.router", mlp["router"]["experts"], W)
            if mlp.get("shared"):
                mat(p + "mlp.shared.gate", mlp["shared"]["ff"], W)
                mat(p + "mlp.shared.up", mlp["shared"]["ff"], W)
                mat(p + "mlp.shared.down", W, mlp["shared"]["ff"])
                mat(p + "mlp.shared.sg", 1, W)
    norm("final.norm", W)
    mat("head", cfg["vocab"], W)
    return out
