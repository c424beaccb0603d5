"""Plain, slow reference of the Vurizen design: one function per mechanism,
written token by token from the equations, in float64 unless told otherwise.
It shares nothing with the serving path (no paged cache, no batching, no
kernels): a sequence is a list of token ids and every layer sees the whole
sequence at once.

Weights are a dict name -> tensor, named as in a checkpoint
('l<i>.mix.q', 'l<i>.mlp.e<j>.gate', 'final.norm', ...). The configuration is
the checkpoint's config dict.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

DT = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def yarn_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """-> (frequency per pair [dims/2], multiplier of cos and sin)."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=DT)
    if not scaling:
        return f, 1.0
    factor = float(scaling["factor"])
    orig = float(scaling["original"])

    def dim_of(turns: float) -> float:
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = torch.tensor(
        [min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)],
        dtype=DT,
    )
    freq = f / factor * ramp + f * (1 - ramp)
    return freq, 0.1 * math.log(factor) + 1.0


def rotate(x, pos: int, freq, mult: float):
    """x [..., dims]; pair (i, i + dims/2)."""
    half = freq.shape[0]
    a = pos * freq
    c, s = torch.cos(a) * mult, torch.sin(a) * mult
    u, v = x[..., :half], x[..., half : 2 * half]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half : 2 * half] = v * c + u * s
    return out


def latent_kv(h, w, pre, mixer, eps):
    """The cached part of a latent-attention layer: (c [T, rank], rotated key
    part [T, rot_dim])."""
    r, dr = mixer["kv_rank"], mixer["rot_dim"]
    rot = mixer["rot"]
    freq, mult = yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    dkv = h @ w[pre + "dkv"].to(DT).T
    c = rms_norm(dkv[:, :r], w[pre + "dkv.norm"].to(DT), eps)
    kr = torch.stack([rotate(dkv[t, r:], t, freq, mult) for t in range(h.shape[0])])
    return c, kr


def latent_attention(h, w, pre, mixer, c, kr):
    """Sliding-window latent attention over the whole sequence h [T, width]
    with the latent c and rotated key part kr of this or of another layer."""
    T = h.shape[0]
    H, dn, dr, dv = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"]
    rot = mixer["rot"]
    freq, mult = yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    window = mixer["mask"]["size"]
    scale = mixer["scale"]
    q = (h @ w[pre + "q"].to(DT).T).view(T, H, dn + dr)
    kn = (c @ w[pre + "uk"].to(DT).T).view(T, H, dn)
    v = (c @ w[pre + "uv"].to(DT).T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=DT)
    for t in range(T):
        qn = q[t, :, :dn]
        qr = rotate(q[t, :, dn:], t, freq, mult)
        lo = max(0, t - window + 1)
        for hd in range(H):
            s = (kn[lo : t + 1, hd] @ qn[hd] + kr[lo : t + 1] @ qr[hd]) * scale
            p = torch.softmax(s, dim=0)
            out[t, hd] = p @ v[lo : t + 1, hd]
    return out.reshape(T, H * dv) @ w[pre + "o"].to(DT).T


def gla(h, w, pre, mixer, eps):
    """Gated linear attention, token by token."""
    T = h.shape[0]
    H, dk, dv, tau = mixer["heads"], mixer["dim"], mixer["vdim"], mixer["tau"]
    q = (h @ w[pre + "q"].to(DT).T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[pre + "k"].to(DT).T).view(T, H, dk)
    v = (h @ w[pre + "v"].to(DT).T).view(T, H, dv)
    z = (h @ w[pre + "a1"].to(DT).T) @ w[pre + "a2"].to(DT).T + w[pre + "a2.b"].to(DT)
    alpha = (torch.sigmoid(z) ** (1.0 / tau)).view(T, H, dk)
    S = torch.zeros(H, dk, dv, dtype=DT)
    o = torch.zeros(T, H, dv, dtype=DT)
    for t in range(T):
        S = alpha[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = rms_norm(o, w[pre + "norm"].to(DT), eps)
    gate = silu(h @ w[pre + "g"].to(DT).T)
    return (o.reshape(T, H * dv) * gate) @ w[pre + "o"].to(DT).T


def route(h, w, pre, router):
    """-> per token a list of (expert, weight)."""
    E, top = router["experts"], router["top"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    z = h @ w[pre + "router"].to(DT).T
    s = torch.sigmoid(z)
    choice = s + w[pre + "correction"].to(DT)
    per = E // groups["count"]
    picks = []
    for t in range(h.shape[0]):
        gscore = []
        for g in range(groups["count"]):
            part = sorted(choice[t, g * per : (g + 1) * per].tolist(), reverse=True)
            gscore.append(sum(part[:2]))
        best = sorted(range(groups["count"]), key=lambda g: -gscore[g])[: groups["keep"]]
        allowed = [e for e in range(E) if e // per in best]
        chosen = sorted(allowed, key=lambda e: -float(choice[t, e]))[:top]
        total = sum(float(s[t, e]) for e in chosen) + 1e-20
        picks.append([(e, float(s[t, e]) / total * router["scale"]) for e in chosen])
    return picks


def moe(h, w, pre, mlp):
    out = torch.zeros_like(h)
    picks = route(h, w, pre, mlp["router"])
    for t, chosen in enumerate(picks):
        for e, wt in chosen:
            p = "%se%d." % (pre, e)
            a = silu(w[p + "gate"].to(DT) @ h[t]) * (w[p + "up"].to(DT) @ h[t])
            out[t] += wt * (w[p + "down"].to(DT) @ a)
    return out


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int],
            return_layers: bool = False):
    """Logits [T, vocab] for one sequence (and the residual stream after every
    layer if asked)."""
    eps = cfg["norm"]["eps"]
    m = cfg["residual_mult"]
    x = w["embed"].to(DT)[torch.tensor(tokens)]
    kept = {}
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        L = "l%d." % i
        mixer = layer["mixer"]
        h = layer_norm(x, w[L + "norm1"].to(DT), w[L + "norm1.b"].to(DT), eps)
        if layer["type"] == "gla":
            y = gla(h, w, L + "mix.", mixer, eps)
        elif layer["type"] == "latent_attention":
            src = mixer.get("kv_from")
            if src is None:
                kept[i] = latent_kv(h, w, L + "mix.", mixer, eps)
                src = i
            y = latent_attention(h, w, L + "mix.", mixer, *kept[src])
        else:
            raise ValueError(layer["type"])
        x = x + m * (y * w[L + "ls1"].to(DT))
        if layer.get("mlp") is not None:
            h = layer_norm(x, w[L + "norm2"].to(DT), w[L + "norm2.b"].to(DT), eps)
            y = moe(h, w, L + "mlp.", layer["mlp"])
            x = x + m * (y * w[L + "ls2"].to(DT))
        streams.append(x.clone())
    x = layer_norm(x, w["final.norm"].to(DT), w["final.norm.b"].to(DT), eps)
    logits = x @ w["head"].to(DT).T
    if return_layers:
        return logits, torch.stack(streams)
    return logits


def random_weights(cfg: dict, seed: int = 0, std: float = 0.5) -> Dict[str, torch.Tensor]:
    """Random bfloat16-representable weights for a configuration, sized so
    that activations stay O(1) through the stack."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).bfloat16().float()

    def vec(n, mean=0.0, dev=0.1):
        return (mean + dev * torch.randn(n, generator=g)).bfloat16().float()

    w = {"embed": (torch.randn(cfg["vocab"], W, generator=g)).bfloat16().float(),
         "final.norm": vec(W, 1.0), "final.norm.b": vec(W),
         "head": mat(cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        L = "l%d." % i
        mx = layer["mixer"]
        for n in ("norm1", "norm2"):
            w[L + n] = vec(W, 1.0)
            w[L + n + ".b"] = vec(W)
        w[L + "ls1"] = vec(W, 1.0, 0.2)
        w[L + "ls2"] = vec(W, 1.0, 0.2)
        H = mx["heads"]
        if layer["type"] == "gla":
            dk, dv = mx["dim"], mx["vdim"]
            low = mx.get("decay_rank", 32)
            w[L + "mix.q"] = mat(H * dk, W)
            w[L + "mix.k"] = mat(H * dk, W)
            w[L + "mix.v"] = mat(H * dv, W)
            w[L + "mix.g"] = mat(H * dv, W)
            w[L + "mix.o"] = mat(W, H * dv)
            w[L + "mix.norm"] = vec(dv, 1.0)
            w[L + "mix.a1"] = mat(low, W)
            w[L + "mix.a2"] = mat(H * dk, low, 2.0)
            w[L + "mix.a2.b"] = vec(H * dk, 1.0, 1.0)
        else:
            dn, dr, dv, r = mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
            w[L + "mix.q"] = mat(H * (dn + dr), W, 2.0)
            if mx.get("kv_from") is None:
                w[L + "mix.dkv"] = mat(r + dr, W, 2.0)
                w[L + "mix.dkv.norm"] = vec(r, 1.0)
            w[L + "mix.uk"] = mat(H * dn, r, 2.0)
            w[L + "mix.uv"] = mat(H * dv, r)
            w[L + "mix.o"] = mat(W, H * dv)
        mlp = layer.get("mlp")
        if mlp is not None:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            w[L + "mlp.router"] = mat(E, W, 2.0)
            w[L + "mlp.correction"] = vec(E, 0.0, 0.3)
            for e in range(E):
                w[L + "mlp.e%d.gate" % e] = mat(ff, W)
                w[L + "mlp.e%d.up" % e] = mat(ff, W)
                w[L + "mlp.e%d.down" % e] = mat(W, ff)
    return w
