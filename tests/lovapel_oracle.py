"""Slow float64 definition of the Lovapel decoder, one function per mechanism, written from the
design's equations: dense attention over whole sequences, token-by-token routing, no paging, no
batching, nothing carried between calls.  It shares no code with the package; the tests compare
the engine (CPU tier and HIP kernels) with it.

A model is ``(cfg, st)``: the checkpoint's ``config.json`` as a dict and its tensors by name.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w over the last axis, var = mean squared deviation."""
    d = x - x.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w.to(F64)


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (the whole projection, all heads)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.to(F64)


def rotate(x, pos, dims, base):
    """x [T, H, d]: among the first ``dims`` channels of a head, channel i pairs with channel
    i + dims / 2 and the pair turns by the angle pos * base^(-2 i / dims)."""
    n = dims // 2
    if n == 0:
        return x
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(n)], dtype=F64)
    ang = pos.to(F64)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :n], x[..., n:2 * n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:]], -1)


def sink_window_attention(q, k, v, scale, window, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv], sink [H].  Row i attends rows j with
    0 <= i - j < window (window 0: every earlier row); the denominator of head h also holds
    exp(sink[h]), which has no value."""
    T, H, _ = q.shape
    rep = H // k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // rep
        for i in range(T):
            lo = max(0, i - window + 1) if window else 0
            sc = (k[lo:i + 1, g] @ q[i, h]) * scale
            m = torch.maximum(sc.max(), sink[h])
            e = torch.exp(sc - m)
            out[i, h] = (e @ v[lo:i + 1, g]) / (e.sum() + torch.exp(sink[h] - m))
    return out


def attention_mixer(h, m, st, p, eps):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = rms_norm(h @ st[p + "q"].to(F64).T, st[p + "q.norm"], eps).view(T, H, d)
    k = rms_norm(h @ st[p + "k"].to(F64).T, st[p + "k.norm"], eps).view(T, G, d)
    v = (h @ st[p + "v"].to(F64).T).view(T, G, dv)
    rot = m.get("rot") or {}
    pos = torch.arange(T)
    q = rotate(q, pos, int(rot.get("dims", 0)), rot.get("base", 10000.0))
    k = rotate(k, pos, int(rot.get("dims", 0)), rot.get("base", 10000.0))
    window = int((m.get("mask") or {}).get("size") or 0)
    o = sink_window_attention(q, k, v, float(m["scale"]), window, st[p + "sink"].to(F64))
    return o.reshape(T, H * dv) @ st[p + "o"].to(F64).T


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def glu(h, st, p, act):
    return (act(h @ st[p + "gate"].to(F64).T) * (h @ st[p + "up"].to(F64).T)) @ \
        st[p + "down"].to(F64).T


def route(z, correction, top, groups, keep):
    """One token's router logits z [N] -> (chosen indices, their weights).  The softmax scores
    plus ``correction`` decide the choice, inside the ``keep`` groups (of ``groups`` equal runs
    of neighbours) whose best such score is largest; the weights are the plain scores of the
    chosen, normalised to sum 1.  Also returns how far the choice is from another one: the gap
    between the last chosen and the best unchosen score, or between the last kept and the best
    dropped group if that is smaller."""
    s = torch.softmax(z, 0)
    c = s + correction
    n = z.shape[0]
    size = n // groups
    best = torch.stack([c[g * size:(g + 1) * size].max() for g in range(groups)])
    kept = torch.topk(best, keep).indices.tolist()
    masked = torch.full_like(c, -math.inf)
    for g in kept:
        masked[g * size:(g + 1) * size] = c[g * size:(g + 1) * size]
    idx = torch.topk(masked, top).indices
    w = s[idx]
    srt = torch.sort(masked, descending=True).values
    margin = float(srt[top - 1] - srt[top]) if n > top else 1.0
    if keep < groups:
        gs = torch.sort(best, descending=True).values
        margin = min(margin, float(gs[keep - 1] - gs[keep]))
    return idx, w / (w.sum() + 1e-20), margin


def moe_ff(h, mlp, st, p, margins=None):
    r = mlp["router"]
    E, ident, top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
    g = r.get("groups") or {}
    groups, keep = int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))
    corr = st[p + "correction"].to(F64) if p + "correction" in st else torch.zeros(E + ident, dtype=F64)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        # the router reads the 32-bit rounding of its input, like everything the model sees
        z = st[p + "router"].to(F64) @ h[t]
        idx, w, margin = route(z, corr, top, groups, keep)
        if margins is not None:
            margins.append(margin)
        for e, we in zip(idx.tolist(), w):
            out[t] += we * (h[t] if e >= E else glu(h[t], st, f"{p}e{e}.", silu))
    if mlp.get("shared"):
        out = out + glu(h, st, p + "shared.", silu)
    return out


def layer_runs(cfg):
    """Indices of the layers in the order they run: the looped span ``times`` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {}
    a, b, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg, st, tokens, layers_out=None, margins=None):
    """Logits [T, vocab] of a whole sequence."""
    eps = float(cfg["norm"]["eps"])
    x = st["embed"].to(F64)[torch.as_tensor(tokens)]
    for i in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        y = attention_mixer(layer_norm(x, st[p + "norm1"], eps), L["mixer"], st, p + "mix.", eps)
        x = x + layer_norm(y, st[p + "norm1b"], eps)
        mlp = L.get("mlp")
        if mlp:
            h = layer_norm(x, st[p + "norm2"], eps)
            y = glu(h, st, p + "mlp.", gelu_tanh) if mlp["kind"] == "dense" else \
                moe_ff(h, mlp, st, p + "mlp.", margins)
            x = x + layer_norm(y, st[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    z = layer_norm(x, st["final.norm"], eps) @ st["embed"].to(F64).T * float(cfg.get("logit_scale", 1.0))
    cap = float(cfg.get("logit_softcap") or 0.0)
    return cap * torch.tanh(z / cap) if cap else z
