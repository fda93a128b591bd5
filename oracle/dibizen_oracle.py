"""Plain, slow statement of the Dibizen design in float64 torch on the CPU: one function per mechanism, written from the
equations and sharing nothing with the product path (``promptcache_amd/model/dibizen_hip.py`` and its kernels).

Notation: n tokens of one sequence at positions 0 .. n-1; ``p`` a dict of float64 tensors keyed like the checkpoint; ``lay`` a
``config.DibizenLayer``.  Recurrences are written as literal loops over the tokens, one token at a time.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def silu(x):
    return x * torch.sigmoid(x)


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def dyt_norm(x, p, name):
    """Dynamic Tanh: tanh(alpha x) w + b -- no statistic of x enters."""
    return torch.tanh(p[name + ".alpha"] * x) * p[name] + p[name + ".b"]


def hyper_read(xs, p, pre):
    """xs [S, n, W] -> the sublayer's input, sum_s in[s] xs[s]."""
    return torch.einsum("s,snw->nw", p[pre + "in"], xs)


def hyper_write(xs, y, p, pre):
    """All streams at once from the old ones: new[t] = sum_s mix[s, t] old[s] + out[t] y."""
    return torch.einsum("st,snw->tnw", p[pre + "mix"], xs) + p[pre + "out"].view(-1, 1, 1) * y.unsqueeze(0)


def lightning_mixer(h, p, pre, lay, eps):
    n = h.shape[0]
    H, D, Dv = lay.heads, lay.dim, lay.vdim
    q = silu(h @ p[pre + "q"].T).view(n, H, D)
    k = silu(h @ p[pre + "k"].T).view(n, H, D)
    v = silu(h @ p[pre + "v"].T).view(n, H, Dv)
    out = torch.zeros(n, H, Dv, dtype=F)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F)
        lam = float(lay.decay[hd])
        for t in range(n):
            S = lam * S + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    o = unit_rms(out.reshape(n, H * Dv), eps) * p[pre + "norm"]
    o = o * torch.sigmoid(h @ p[pre + "g"].T)
    return o @ p[pre + "o"].T


def query_temperature(pos, lay):
    """1 + coef ln(floor((p + 1) / every) + 1), one factor per position."""
    if not lay.qt_every:
        return torch.ones(len(pos), dtype=F)
    return torch.tensor([1.0 + lay.qt_coef * math.log(math.floor((int(t) + 1) / lay.qt_every) + 1.0) for t in pos], dtype=F)


def attention_keys_values(h, p, pre, lay):
    n = h.shape[0]
    return (h @ p[pre + "k"].T).view(n, lay.kv_heads, lay.dim), (h @ p[pre + "v"].T).view(n, lay.kv_heads, lay.vdim)


def attention_mixer(h, p, pre, lay, k, v):
    """k, v: [n, G, dim], [n, G, vdim] of this layer or of the layer it borrows from."""
    n = h.shape[0]
    H, G = lay.heads, lay.kv_heads
    q = (h @ p[pre + "q"].T).view(n, H, lay.dim) * query_temperature(range(n), lay).view(n, 1, 1)
    causal = torch.tril(torch.ones(n, n, dtype=torch.bool))
    out = torch.zeros(n, H, lay.vdim, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * lay.scale
        s = torch.where(causal, s, torch.full_like(s, -math.inf))
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    o = out.reshape(n, H * lay.vdim) * torch.sigmoid(h @ p[pre + "g"].T)
    return o @ p[pre + "o"].T


def mamba_mixer(h, p, pre, lay):
    n = h.shape[0]
    C, N, R, taps = lay.inner, lay.state, lay.dt_rank, lay.conv
    xz = h @ p[pre + "in"].T
    x, z = xz[:, :C], xz[:, C:]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F), x])
    xc = torch.stack([(padded[t:t + taps] * p[pre + "conv"].T).sum(dim=0) for t in range(n)]) + p[pre + "conv.b"]
    xc = silu(xc)
    low = xc @ p[pre + "x"].T
    dt = torch.nn.functional.softplus(low[:, :R] @ p[pre + "dt"].T + p[pre + "dt.b"])
    Bm, Cm = low[:, R:R + N], low[:, R + N:R + 2 * N]
    A = -torch.exp(p[pre + "A_log"])
    S = torch.zeros(C, N, dtype=F)
    y = torch.zeros(n, C, dtype=F)
    for t in range(n):
        S = torch.exp(dt[t].view(C, 1) * A) * S + (dt[t] * xc[t]).view(C, 1) * Bm[t].view(1, N)
        y[t] = S @ Cm[t] + p[pre + "D"] * xc[t]
    return (y * silu(z)) @ p[pre + "o"].T


def route(h, p, pre, lay):
    """-> (chosen router outputs [n, top], their weights [n, top])."""
    s = torch.softmax(h @ p[pre + "router"].T, dim=-1)
    choice = s + p[pre + "correction"]
    n, E = s.shape
    per = E // lay.groups
    best = choice.view(n, lay.groups, per).max(dim=-1).values
    kept = best.topk(lay.groups_keep, dim=-1).indices
    allowed = torch.zeros(n, lay.groups, dtype=torch.bool).scatter_(1, kept, True).repeat_interleave(per, dim=1)
    choice = torch.where(allowed, choice, torch.full_like(choice, -math.inf))
    idx = choice.topk(lay.top, dim=-1).indices
    w = s.gather(1, idx)
    return idx, w / (w.sum(dim=-1, keepdim=True) + 1e-20)


def moe_ff(h, p, pre, lay):
    idx, w = route(h, p, pre, lay)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(idx[t].tolist(), w[t]):
            if e >= lay.experts:
                out[t] += wt * h[t]
            else:
                out[t] += wt * (torch.relu(p[pre + f"e{e}.up"] @ h[t]).pow(2) @ p[pre + f"e{e}.down"].T)
    return out


def forward(tokens, p, cfg, return_layers=False):
    """Logits [n, vocab] of one sequence (float64); with ``return_layers`` also the sum of the streams after every layer."""
    p = {k: v.to(F) for k, v in p.items()}
    n = len(tokens)
    x = p["embed"][torch.as_tensor(tokens, dtype=torch.long)] + p["pos"][:n]
    xs = x.unsqueeze(0).repeat(cfg.streams, 1, 1)
    kv, sums = {}, []
    for i, lay in enumerate(cfg.layers):
        pre = f"l{i}."
        h = dyt_norm(hyper_read(xs, p, pre + "hc1."), p, pre + "norm1")
        if lay.kind == "lightning":
            y = lightning_mixer(h, p, pre + "mix.", lay, cfg.norm_eps)
        elif lay.kind == "attention":
            if lay.kv_from < 0:
                kv[i] = attention_keys_values(h, p, pre + "mix.", lay)
            y = attention_mixer(h, p, pre + "mix.", lay, *kv[i if lay.kv_from < 0 else lay.kv_from])
        else:
            y = mamba_mixer(h, p, pre + "mix.", lay)
        xs = hyper_write(xs, y, p, pre + "hc1.")
        if lay.experts + lay.identity:
            h = dyt_norm(hyper_read(xs, p, pre + "hc2."), p, pre + "norm2")
            xs = hyper_write(xs, moe_ff(h, p, pre + "mlp.", lay), p, pre + "hc2.")
        sums.append(xs.sum(dim=0))
    logits = dyt_norm(xs.sum(dim=0), p, "final.norm") @ p["head"].T
    if cfg.logit_softcap:
        logits = cfg.logit_softcap * torch.tanh(logits / cfg.logit_softcap)
    return (logits, torch.stack(sums)) if return_layers else logits
