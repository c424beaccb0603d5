"""A plain, slow float64 implementation of the Sogidra design: one function
per mechanism, whole sequences only, no cache, no batching. It shares no code
with the serving path; the tests compare the engine against it.

Notation: n tokens, width W, H query heads, G key/value heads, d key width,
dv value width, positions p = 0 .. n - 1.
"""

import math
from typing import Dict, List

import torch

DT = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def zero_centred_norm(x, w, eps):
    """RMS norm whose stored weight is the deviation from one."""
    return rms_unit(x, eps) * (1.0 + w)


def depth_average(history: List[torch.Tensor], coeffs: torch.Tensor) -> torch.Tensor:
    """sum_j coeffs[j] * history[j] over everything produced so far."""
    assert len(history) == coeffs.numel()
    out = torch.zeros_like(history[0])
    for c, x in zip(coeffs.tolist(), history):
        out = out + c * x
    return out


def softplus(x: float) -> float:
    return math.log1p(math.exp(x))


def xielu(z: torch.Tensor, p: float, q: float) -> torch.Tensor:
    ap, an = softplus(p), softplus(q)
    pos = ap * z * z + z / 2
    neg = (0.5 + an) * (torch.exp(z) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def feed_forward(h, w, pre):
    p, q = w[pre + "act"].to(DT).tolist()
    return xielu(h @ w[pre + "up"].to(DT).T, p, q) @ w[pre + "down"].to(DT).T


def query_temperature(n: int, coef: float, every: int) -> torch.Tensor:
    p = torch.arange(n, dtype=DT)
    return 1.0 + coef * torch.log(torch.floor((p + 1) / every) + 1.0)


def diff_lambda(w, pre, diff: float) -> float:
    a = float((w[pre + "lq1"].to(DT) * w[pre + "lk1"].to(DT)).sum())
    b = float((w[pre + "lq2"].to(DT) * w[pre + "lk2"].to(DT)).sum())
    return math.exp(a) - math.exp(b) + diff


def diff_keys_values(h, w, pre, mx):
    n, G, d, dv = h.shape[0], mx["kv_heads"], mx["dim"], mx["vdim"]
    k = (h @ w[pre + "k"].to(DT).T + w[pre + "k.b"].to(DT)).view(n, G, 2, d)
    v = (h @ w[pre + "v"].to(DT).T + w[pre + "v.b"].to(DT)).view(n, G, dv)
    return k, v


def diff_attention(h, w, pre, mx, k, v, eps):
    """Two causal softmax maps per head over shared values, combined with one
    learned lambda, then a weightless RMS norm per head times (1 - diff)."""
    n, H, G, d, dv = h.shape[0], mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = (h @ w[pre + "q"].to(DT).T + w[pre + "q.b"].to(DT)).view(n, H, 2, d)
    t = mx.get("q_temp")
    if t:
        q = q * query_temperature(n, t["coef"], t["every"])[:, None, None, None]
    lam = diff_lambda(w, pre, mx["diff"])
    out = torch.zeros(n, H, dv, dtype=DT)
    for i in range(n):
        for hh in range(H):
            g = hh // (H // G)
            maps = []
            for m in range(2):
                s = (k[: i + 1, g, m] @ q[i, hh, m]) * mx["scale"]
                maps.append(torch.softmax(s, 0) @ v[: i + 1, g])
            o = maps[0] - lam * maps[1]
            out[i, hh] = rms_unit(o, eps) * (1.0 - mx["diff"])
    return out.reshape(n, H * dv) @ w[pre + "o"].to(DT).T


def pooled_keys_values(h, w, pre, mx, eps):
    """Keys as the cache holds them (unit RMS per head) and values = the
    projected keys before that norm."""
    n, G, d = h.shape[0], mx["kv_heads"], mx["dim"]
    raw = (h @ w[pre + "k"].to(DT).T).view(n, G, d)
    return rms_unit(raw, eps), raw


def visible(i: int, size: int, pool: int):
    """(pooled blocks, tokens) that position i sees."""
    toks = [j for j in range(i + 1) if i - j < size]
    blocks = []
    if pool > 0:
        b = 0
        while b * pool + pool - 1 <= i - size:
            blocks.append(b)
            b += 1
    return blocks, toks


def pooled_window_attention(h, w, pre, mx, k, v, eps):
    n, H, G, d = h.shape[0], mx["heads"], mx["kv_heads"], mx["dim"]
    q = rms_unit((h @ w[pre + "q"].to(DT).T).view(n, H, d), eps)
    size, pool = mx["mask"]["size"], mx["mask"].get("pool", 0)
    cap = mx.get("softcap", 0.0)
    out = torch.zeros(n, H, d, dtype=DT)
    for i in range(n):
        blocks, toks = visible(i, size, pool)
        for g in range(G):
            keys = torch.stack(
                [k[b * pool : (b + 1) * pool, g].mean(0) for b in blocks]
                + [k[j, g] for j in toks])
            vals = torch.stack(
                [v[b * pool : (b + 1) * pool, g].mean(0) for b in blocks]
                + [v[j, g] for j in toks])
            for hh in range(g * (H // G), (g + 1) * (H // G)):
                s = (keys @ q[i, hh]) * mx["scale"]
                if cap:
                    s = cap * torch.tanh(s / cap)
                out[i, hh] = torch.softmax(s, 0) @ vals
    return out.reshape(n, H * d) @ w[pre + "o"].to(DT).T


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int],
            return_layers: bool = False):
    eps = cfg["norm"]["eps"]
    n = len(tokens)
    x = w["embed"].to(DT)[tokens] + w["pos"].to(DT)[:n]
    history, streams, kv = [x], [], {}
    for i, sp in enumerate(cfg["layers"]):
        pre, mx = "l%d." % i, sp["mixer"]
        h = zero_centred_norm(x, w[pre + "norm1"].to(DT), eps)
        if sp["type"] == "attention":
            if mx.get("kv_from") is None:
                kv[i] = diff_keys_values(h, w, pre + "mix.", mx)
            k, v = kv[i if mx.get("kv_from") is None else mx["kv_from"]]
            y = diff_attention(h, w, pre + "mix.", mx, k, v, eps)
        else:
            if mx.get("kv_from") is None:
                kv[i] = pooled_keys_values(h, w, pre + "mix.", mx, eps)
            k, v = kv[i if mx.get("kv_from") is None else mx["kv_from"]]
            y = pooled_window_attention(h, w, pre + "mix.", mx, k, v, eps)
        x = x + zero_centred_norm(y, w[pre + "norm1b"].to(DT), eps)
        if sp.get("mlp") is not None:
            h = zero_centred_norm(x, w[pre + "norm2"].to(DT), eps)
            y = feed_forward(h, w, pre + "mlp.")
            x = x + zero_centred_norm(y, w[pre + "norm2b"].to(DT), eps)
        history.append(x)
        x = depth_average(history, w[pre + "dwa"].to(DT))
        streams.append(x)
    logits = zero_centred_norm(x, w["final.norm"].to(DT), eps) @ w["embed"].to(DT).T
    return (logits, streams) if return_layers else logits


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random weights, rounded to bf16 (as a checkpoint stores them)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, gain=1.0):
        return torch.randn(o, i, generator=g) * gain / math.sqrt(i)

    def vec(n, s):
        return torch.randn(n, generator=g) * s

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g),
         "pos": torch.randn(cfg["max_positions"], W, generator=g) * 0.5,
         "final.norm": vec(W, 0.2)}
    for i, sp in enumerate(cfg["layers"]):
        pre, mx = "l%d." % i, sp["mixer"]
        H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        own = mx.get("kv_from") is None
        w[pre + "norm1"], w[pre + "norm1b"] = vec(W, 0.2), vec(W, 0.2)
        if sp["type"] == "attention":
            w[pre + "mix.q"], w[pre + "mix.q.b"] = mat(H * 2 * d, W, 2.0), vec(H * 2 * d, 0.3)
            if own:
                w[pre + "mix.k"], w[pre + "mix.k.b"] = mat(G * 2 * d, W, 2.0), vec(G * 2 * d, 0.3)
                w[pre + "mix.v"], w[pre + "mix.v.b"] = mat(G * dv, W), vec(G * dv, 0.3)
            for name in ("lq1", "lk1", "lq2", "lk2"):
                w[pre + "mix." + name] = vec(d, 0.25)
        else:
            w[pre + "mix.q"] = mat(H * d, W)
            if own:
                w[pre + "mix.k"] = mat(G * d, W)
        w[pre + "mix.o"] = mat(W, H * dv)
        if sp.get("mlp") is not None:
            ff = sp["mlp"]["ff"]
            w[pre + "norm2"], w[pre + "norm2b"] = vec(W, 0.2), vec(W, 0.2)
            w[pre + "mlp.up"], w[pre + "mlp.down"] = mat(ff, W), mat(W, ff)
            w[pre + "mlp.act"] = vec(2, 1.0)
        c = vec(i + 2, 0.3)
        c[-1] += 1.0
        w[pre + "dwa"] = c
    return {k: v.to(torch.bfloat16).float() for k, v in w.items()}
