"""Plain, slow statement of the Kazolorn design in float64 torch on the CPU: one function per mechanism, written from the
equations and sharing nothing with the product path (``promptcache_amd/model/kazolorn_hip.py`` and its kernels).

Notation: n tokens of one sequence, positions 0 .. n-1; ``p`` a dict of float64 tensors keyed like the checkpoint.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps under the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, gain, eps):
    return unit_rms(x, eps) * gain


def poly_activation(z, coef, eps):
    """coef = (a, b, c, e):  a u(z) + b u(z^2) + c u(z^3) + e,  u = unit_rms over the feed-forward axis."""
    a, b, c, e = [float(v) for v in coef]
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


def head_slopes(n_heads):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads)], dtype=F)


def sink_softmax(s, allowed):
    """Row-wise over the last axis: exp(s_j) / (1 + sum_j' exp(s_j')), only over allowed entries (others get weight 0)."""
    s = torch.where(allowed, s, torch.full_like(s, -math.inf))
    top = torch.clamp(s.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - top)
    return e / (torch.exp(-top) + e.sum(dim=-1, keepdim=True))


def talking_attention(q, k, scale, window, talk, first_pos=0):
    """q [m, H, D] for positions first_pos .. first_pos+m-1; k [n, G, D] for positions 0 .. n-1 (n = first_pos + m); the values
    are the keys.  Scores: scaled dot products, minus slope_h * distance, mixed across heads by ``talk`` [H, H]; then the window
    (0 = none) and the causal rule; softmax with a sink.  Returns [m, H, D]."""
    m, H, D = q.shape
    n, G, _ = k.shape
    rep = H // G
    out = torch.zeros(m, H, D, dtype=F)
    slopes = head_slopes(H)
    pos_i = torch.arange(first_pos, first_pos + m).view(m, 1)
    pos_j = torch.arange(n).view(1, n)
    dist = (pos_i - pos_j).to(F)
    raw = torch.stack([(q[:, h, :] @ k[:, h // rep, :].T) * scale - slopes[h] * dist for h in range(H)])      # [H, m, n]
    mixed = torch.einsum("hg,gaj->haj", talk.to(F), raw)
    allowed = (pos_j <= pos_i)
    if window:
        allowed = allowed & (pos_i - pos_j < window)
    for h in range(H):
        w = sink_softmax(mixed[h], allowed)
        out[:, h, :] = w @ k[:, h // rep, :]
    return out


def attention_mixer(h, p, pre, lay):
    """Whole-sequence mixer: projections with biases, talking attention, output projection."""
    n = h.shape[0]
    q = (h @ p[pre + "q"].T + p[pre + "q.b"]).view(n, lay.heads, lay.dim)
    k = (h @ p[pre + "k"].T + p[pre + "k.b"]).view(n, lay.kv_heads, lay.dim)
    a = talking_attention(q, k, lay.scale, lay.window, p[pre + "talk"])
    return a.reshape(n, lay.heads * lay.dim) @ p[pre + "o"].T + p[pre + "o.b"]


def dense_ff(h, p, pre, eps):
    return poly_activation(h @ p[pre + "up"].T, p[pre + "act"], eps) @ p[pre + "down"].T


def route(h, router, top):
    """-> (chosen experts [n, top], their sigmoid scores [n, top])."""
    s = torch.sigmoid(h @ router.T)
    val, idx = torch.sort(s, dim=-1, descending=True, stable=True)
    return idx[:, :top], val[:, :top]


def sparse_ff(h, p, pre, lay):
    idx, val = route(h, p[pre + "router"], lay.top)
    out = torch.zeros(h.shape[0], p[pre + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), val[t].tolist()):
            x = w * h[t]                                   # the weight scales the expert's INPUT
            g = x @ p[f"{pre}e{e}.gate"].T
            u = x @ p[f"{pre}e{e}.up"].T
            out[t] += (g * torch.sigmoid(g) * u) @ p[f"{pre}e{e}.down"].T
    return out


def forward(cfg, weights, tokens, return_streams=False):
    """Logits [n, vocab] of one sequence (and, on request, what goes on to the next layer after each layer)."""
    p = {k: v.to(F) for k, v in weights.items()}
    eps = cfg.norm_eps
    x = p["embed"][torch.tensor(list(tokens))]
    results = [x]
    streams = []
    for i, lay in enumerate(cfg.layers):
        pre = f"l{i}."
        y = p[pre + "ls1"] * attention_mixer(rms_norm(x, p[pre + "norm1"], eps), p, pre + "mix.", lay)
        if lay.mlp_kind == "dense":
            y = y + p[pre + "ls2"] * dense_ff(rms_norm(x, p[pre + "norm2"], eps), p, pre + "mlp.", eps)
        elif lay.mlp_kind == "moe":
            y = y + p[pre + "ls2"] * sparse_ff(rms_norm(x, p[pre + "norm2"], eps), p, pre + "mlp.", lay)
        results.append(x + y)
        x = sum(float(c) * r for c, r in zip(p[pre + "dwa"], results))
        streams.append(x)
    logits = rms_norm(x, p["final.norm"], eps) @ p["head"].T
    return (logits, torch.stack(streams)) if return_streams else logits


def greedy(cfg, weights, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(forward(cfg, weights, toks)[-1])))
    return toks[len(prompt):]
