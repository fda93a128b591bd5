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


def decayed_linear_attention(q, k, v, decay, state=None):
    """q, k [n, H, D], v [n, H, Dv]; per head S <- decay S + k v^T, o = S^T q, token by token from ``state`` [H, D, Dv] (zeros
    when not given).  -> (o [n, H, Dv], the state after the last token)."""
    n, H, D = q.shape
    Dv = v.shape[-1]
    S = torch.zeros(H, D, Dv, dtype=F) if state is None else state.clone()
    out = torch.zeros(n, H, Dv, dtype=F)
    for t in range(n):
        for hd in range(H):
            S[hd] = float(decay[hd]) * S[hd] + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S[hd].T @ q[t, hd]
    return out, S


def lightning_mixer(h, p, pre, lay, eps):
    n = h.shape[0]
    H, D, Dv = lay.heads, lay.dim, lay.vdim
    q = silu(h @ p[pre + "q"].T).view(n, H, D)
    k = silu(h @ p[pre + "k"].T).view(n, H, D)
    v = silu(h @ p[pre + "v"].T).view(n, H, Dv)
    out, _ = decayed_linear_attention(q, k, v, lay.decay)
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


def causal_softmax_attention(q, k, v, scale, first_pos=0):
    """q [m, H, D] at positions first_pos .. first_pos + m - 1; k [n, G, D], v [n, G, Dv] at positions 0 .. n - 1
    (n = first_pos + m); query head h reads key/value head h // (H / G); position i sees every j <= i.  -> [m, H, Dv]."""
    m, H, _ = q.shape
    n, G, Dv = v.shape
    seen = torch.arange(n).view(1, n) <= torch.arange(first_pos, first_pos + m).view(m, 1)
    out = torch.zeros(m, H, Dv, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * scale
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def attention_mixer(h, p, pre, lay, k, v):
    """k, v: [n, G, dim], [n, G, vdim] of this layer or of the layer it borrows from."""
    n = h.shape[0]
    H = lay.heads
    q = (h @ p[pre + "q"].T).view(n, H, lay.dim) * query_temperature(range(n), lay).view(n, 1, 1)
    out = causal_softmax_attention(q, k, v, lay.scale)
    o = out.reshape(n, H * lay.vdim) * torch.sigmoid(h @ p[pre + "g"].T)
    return o @ p[pre + "o"].T


def causal_convolution(x, w, b, before=None):
    """x [n, C]; w [C, taps] whose LAST column multiplies the current token; ``before`` [taps - 1, C]: the inputs ahead of x
    (zeros when not given).  -> [n, C] (no activation)."""
    n, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F) if before is None else before, x])
    return torch.stack([(padded[t:t + taps] * w.T).sum(dim=0) for t in range(n)]) + b


def selective_scan(x, dt, Bm, Cm, A, D, state=None):
    """x, dt [n, C]; Bm, Cm [n, N]; A [C, N]; D [C]: S <- exp(dt A) S + dt x B, y = S C + D x, token by token from ``state``
    [C, N].  -> (y [n, C], the state after the last token)."""
    n, C = x.shape
    S = torch.zeros(C, A.shape[1], dtype=F) if state is None else state.clone()
    y = torch.zeros(n, C, dtype=F)
    for t in range(n):
        S = torch.exp(dt[t].view(C, 1) * A) * S + (dt[t] * x[t]).view(C, 1) * Bm[t].view(1, -1)
        y[t] = S @ Cm[t] + D * x[t]
    return y, S


def mamba_mixer(h, p, pre, lay):
    C, N, R = lay.inner, lay.state, lay.dt_rank
    xz = h @ p[pre + "in"].T
    x, z = xz[:, :C], xz[:, C:]
    xc = silu(causal_convolution(x, p[pre + "conv"], p[pre + "conv.b"]))
    low = xc @ p[pre + "x"].T
    dt = torch.nn.functional.softplus(low[:, :R] @ p[pre + "dt"].T + p[pre + "dt.b"])
    y, _ = selective_scan(xc, dt, low[:, R:R + N], low[:, R + N:R + 2 * N], -torch.exp(p[pre + "A_log"]), p[pre + "D"])
    return (y * silu(z)) @ p[pre + "o"].T


def choose(logits, correction, top, groups, keep):
    """Router choice from logits [n, E]: softmax scores; choice scores = scores + correction; only outputs of the ``keep`` groups
    (of ``groups`` equal runs of neighbours) with the largest single choice score can win; the ``top`` largest choice scores
    win; weights = their scores (without the correction) over their sum.  -> (indices [n, top], weights [n, top])."""
    s = torch.softmax(logits, dim=-1)
    choice = s + correction
    n, E = s.shape
    per = E // groups
    best = choice.view(n, groups, per).max(dim=-1).values
    kept = best.topk(keep, dim=-1).indices
    allowed = torch.zeros(n, groups, dtype=torch.bool).scatter_(1, kept, True).repeat_interleave(per, dim=1)
    choice = torch.where(allowed, choice, torch.full_like(choice, -math.inf))
    idx = choice.topk(top, dim=-1).indices
    w = s.gather(1, idx)
    return idx, w / (w.sum(dim=-1, keepdim=True) + 1e-20)


def route(h, p, pre, lay):
    return choose(h @ p[pre + "router"].T, p[pre + "correction"], lay.top, lay.groups, lay.groups_keep)


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


def greedy(cfg, p, prompt, n_new):
    """n_new tokens, each the arg-max of the whole sequence's last logits."""
    seq = list(prompt)
    for _ in range(n_new):
        seq.append(int(forward(seq, p, cfg)[-1].argmax()))
    return seq[len(prompt):]


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
