"""Dibizen on the GPU against the plain float64 oracle (``oracle/dibizen_oracle.py``): every new building-block kernel alone,
then the model through its arena -- prompts, token-by-token decoding, portions, unequal batches, reused slots and states, growth
of the arena, long decoding through captured graphs -- and greedy generation through both engines and the trace runner.
float32 runs are held to float32 accuracy; bfloat16 runs to what bf16 operands allow."""
import json
import math
import os
import subprocess

import pytest
import torch

from oracle import dibizen_oracle as O
from promptcache_amd.model import weights as W
from promptcache_amd.model.config import DibizenLayer, DibizenShape

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
F64 = torch.float64
DTYPES = [torch.float32, torch.bfloat16]


def rel(got, want):
    got, want = got.detach().to("cpu", F64), want.detach().to("cpu", F64)
    return float((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt().clamp_min(1e-30))


def tol(dtype, f32=2e-5, bf16=2e-2):
    return f32 if dtype == torch.float32 else bf16


def B():
    from promptcache_amd import _blocks
    return _blocks


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype).to(DEV)


def dev_i32(rows):
    return torch.tensor(rows, dtype=torch.int32, device=DEV).reshape(-1)


def moe(l, ff, experts, identity, top, groups=1, keep=1):
    l.ff, l.experts, l.identity, l.top, l.groups, l.groups_keep = ff, experts, identity, top, groups, keep
    return l


# ---- shapes: layers differ from one another, come in different orders, and no size is a round one -------------------------------
def shape_mixed():
    return DibizenShape(vocab_size=150, hidden_size=96, norm_eps=1e-5, streams=3, max_positions=400, logit_softcap=12.0, layers=[
        moe(DibizenLayer("attention", heads=6, kv_heads=3, dim=24, vdim=40, scale=0.25, qt_coef=0.3, qt_every=7), 24, 6, 2, 3, 4, 2),
        moe(DibizenLayer("mamba1", inner=72, state=10, conv=3, dt_rank=5), 16, 4, 0, 1),
        DibizenLayer("lightning", heads=3, kv_heads=3, dim=20, vdim=24, decay=(0.5, 0.9, 0.99)),
        moe(DibizenLayer("attention", heads=6, kv_heads=3, dim=24, vdim=40, scale=0.2, kv_from=0), 16, 3, 3, 2, 3, 2),
        moe(DibizenLayer("lightning", heads=2, kv_heads=2, dim=40, vdim=16, decay=(1.0, 0.75)), 8, 5, 0, 5),
    ])


def shape_odd():
    """Sizes that are no multiple of a 16-byte chunk in either element type; one stream, one head, one expert, two taps, one
    state, no temperature, no cap, a feed-forward of identity experts only."""
    return DibizenShape(vocab_size=75, hidden_size=50, norm_eps=1e-6, streams=1, max_positions=90, logit_softcap=0.0, layers=[
        moe(DibizenLayer("mamba1", inner=30, state=1, conv=2, dt_rank=1), 14, 1, 1, 2),
        moe(DibizenLayer("lightning", heads=1, kv_heads=1, dim=6, vdim=10, decay=(0.8,)), 6, 0, 2, 1),
        moe(DibizenLayer("attention", heads=3, kv_heads=1, dim=10, vdim=6, scale=0.4), 10, 2, 0, 2, 2, 2),
        DibizenLayer("mamba1", inner=17, state=7, conv=1, dt_rank=3),
    ])


def shape_wide():
    """Enough heads, columns, channels and states to reach the wider kernel instantiations."""
    return DibizenShape(vocab_size=320, hidden_size=128, norm_eps=1e-6, streams=2, max_positions=600, logit_softcap=30.0, layers=[
        moe(DibizenLayer("lightning", heads=4, kv_heads=4, dim=96, vdim=48, decay=(0.6, 0.9, 0.98, 0.999)), 64, 8, 0, 2),
        moe(DibizenLayer("attention", heads=8, kv_heads=2, dim=128, vdim=72, scale=0.09, qt_coef=0.2, qt_every=64), 32, 12, 4, 4, 4, 3),
        moe(DibizenLayer("mamba1", inner=200, state=40, conv=4, dt_rank=8), 64, 8, 0, 2),
        moe(DibizenLayer("attention", heads=4, kv_heads=4, dim=160, vdim=136, scale=0.08), 32, 4, 0, 1),
    ])


SHAPES = {"mixed": shape_mixed, "odd": shape_odd, "wide": shape_wide}
_models = {}


def model(name, dtype, seed=11):
    from promptcache_amd.model.dibizen_hip import DibizenHIP
    key = (name, dtype, seed)
    if key not in _models:
        s = SHAPES[name]()
        w = W.make_dibizen_weights(s, seed=seed)
        _models[key] = (s, w, DibizenHIP(s, w, device=DEV, dtype=dtype))
    return _models[key]


def toks(n, vocab, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def run_alone(m, tokens, cuts=None):
    """One request on a fresh arena, its tokens cut into the given portions; logits of every token."""
    ar = m.new_arena(1, 8)
    s = ar.alloc()
    cuts = cuts or [len(tokens)]
    assert sum(cuts) == len(tokens)
    out, at = [], 0
    for c in cuts:
        out.append(m.forward_rows(ar, [s], [tokens[at:at + c]], [list(range(c))]))
        at += c
    return torch.cat(out)


# =====================================================================================================================================
# building blocks alone
# =====================================================================================================================================
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M", [3, 40, 150])
def test_linear_activations_and_their_split(dtype, M):
    N, K = 52, 44
    x, w, b = rnd(M, K, dtype=dtype, seed=1), rnd(N, K, dtype=dtype, seed=2, scale=0.3), rnd(N, dtype=dtype, seed=3)
    z = x.to(F64) @ w.to(F64).T + b.to(F64)
    fns = {B().ACT_SILU: O.silu, B().ACT_SIGMOID: torch.sigmoid, B().ACT_RELU2: lambda t: torch.relu(t).pow(2),
           B().ACT_SOFTPLUS: torch.nn.functional.softplus, B().ACT_SOFTCAP: lambda t: 3.0 * torch.tanh(t / 3.0)}
    for act, fn in fns.items():
        y = torch.empty((M, N), dtype=torch.float32, device=DEV)
        B().linear(x, w, y, M=M, bias=b, act=act, act_param=3.0)
        assert rel(y, fn(z)) < tol(dtype, 1e-5, 1e-5), act
    y = torch.empty((M, N), dtype=dtype, device=DEV)
    B().linear(x, w, y, M=M, bias=b, act=B().ACT_SILU, act_split=20, act2=B().ACT_SIGMOID)
    assert rel(y, torch.cat([O.silu(z[:, :20]), torch.sigmoid(z[:, 20:])], dim=1)) < tol(dtype, 1e-5, 4e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M", [2, 37, 140])
def test_linear_three_destinations(dtype, M):
    # columns [0, 20) stay rows, [20, 32) go to a row-wise cache (2 heads of 6), [32, 52) to a column-wise cache (2 heads of 10)
    N, K, cap = 52, 44, 64
    x, w = rnd(M, K, dtype=dtype, seed=1), rnd(N, K, dtype=dtype, seed=2, scale=0.3)
    z = x.to(F64) @ w.to(F64).T
    slot = torch.arange(M) % 3
    pos = torch.arange(M) // 3
    kc = torch.zeros((3, 2, cap, 6), dtype=dtype, device=DEV)
    vc = torch.zeros((3, 2, 10, cap), dtype=dtype, device=DEV)
    off2 = (slot * (2 * cap * 6) + pos * 6).to(torch.int64).to(DEV)
    off3 = (slot * (2 * 10 * cap) + pos).to(torch.int64).to(DEV)
    y = torch.empty((M, 20), dtype=dtype, device=DEV)
    B().linear(x, w, y, M=M, act=B().ACT_SIGMOID, split_n=20, y2=kc, row_off2=off2, head_dim2=6, head_stride2=cap * 6, split_n3=32,
               y3=vc, row_off3=off3, col_stride3=cap)
    assert rel(y, torch.sigmoid(z[:, :20])) < tol(dtype, 1e-5, 4e-3)
    got_k = kc[slot, :, pos].reshape(M, 12)
    got_v = vc[slot, :, :, pos].reshape(M, 20)
    assert rel(got_k, z[:, 20:32]) < tol(dtype, 1e-5, 4e-3) and rel(got_v, z[:, 32:]) < tol(dtype, 1e-5, 4e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("S", [1, 2, 5])
def test_hyper_norm_write_read_gather_and_embedding(dtype, S):
    T, Wd = 9, 70
    table, pos = rnd(30, Wd, dtype=dtype, seed=1), rnd(20, Wd, dtype=dtype, seed=2)
    ids, ps = dev_i32([3, 29, 0, 7, 7, 12, 1, 2, 5]), dev_i32([0, 1, 2, 19, 0, 1, 2, 3, 4])
    xs = torch.empty((S, T, Wd), dtype=torch.float32, device=DEV)
    B().embed_pos_rows(table, pos, ids, ps, xs)
    want0 = table.to(F64)[ids.long()] + pos.to(F64)[ps.long()]
    assert all(rel(xs[s], want0) < 1e-7 for s in range(S))
    xs.copy_(rnd(S, T, Wd, seed=3))
    old = xs.to(F64).cpu()
    y, mix, ow, iw = rnd(T, Wd, seed=4), rnd(S, S, seed=5), rnd(S, seed=6), rnd(S, seed=7)
    gain, bias, alpha = rnd(Wd, seed=8), rnd(Wd, seed=9), torch.tensor([0.7], device=DEV)
    p = {"h.mix": mix.to(F64).cpu(), "h.out": ow.to(F64).cpu(), "h.in": iw.to(F64).cpu(), "n": gain.to(F64).cpu(),
         "n.b": bias.to(F64).cpu(), "n.alpha": alpha.to(F64).cpu()[0]}
    new = O.hyper_write(old, y.to(F64).cpu(), p, "h.")
    u = O.hyper_read(new, p, "h.")
    # gathered rows first: the streams must stay as they were
    rows = dev_i32([8, 2, 2])
    out = torch.empty((3, Wd), dtype=dtype, device=DEV)
    B().hyper_norm(xs, y=y, mix=mix, out_w=ow, norm=B().NORM_DYT, gain=gain, bias=bias, alpha=alpha, out=out, rows=rows)
    assert rel(out, O.dyt_norm(new.sum(dim=0), p, "n")[[8, 2, 2]]) < tol(dtype, 1e-5, 4e-3) and torch.equal(xs.cpu().to(F64), old)
    out, xo = torch.empty((T, Wd), dtype=dtype, device=DEV), torch.empty((T, Wd), dtype=torch.float32, device=DEV)
    B().hyper_norm(xs, y=y, mix=mix, out_w=ow, in_w=iw, norm=B().NORM_DYT, gain=gain, bias=bias, alpha=alpha, out=out, x_out=xo)
    assert rel(xs, new) < 1e-6 and rel(xo, u) < 1e-6 and rel(out, O.dyt_norm(u, p, "n")) < tol(dtype, 1e-5, 4e-3)
    B().hyper_norm(xs, in_w=iw, norm=B().NORM_RMS, gain=gain, eps=1e-5, out=out)                # read half alone, the other norm
    assert rel(xs, new) < 1e-6 and rel(out, O.unit_rms(u, 1e-5) * p["n"]) < tol(dtype, 1e-5, 4e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_norm(dtype):
    T, C = 7, 90
    x, gain, gate = rnd(T, C, seed=1, scale=3.0), rnd(C, seed=2), rnd(T, 2 * C, dtype=dtype, seed=3)
    out = torch.empty((T, C), dtype=dtype, device=DEV)
    B().gated_norm(x, gain, gate[:, C:], 2 * C, out, 1e-5, T)
    assert rel(out, O.unit_rms(x.to(F64).cpu(), 1e-5) * gain.to(F64).cpu() * gate.to(F64).cpu()[:, C:]) < tol(dtype, 1e-6, 4e-3)
    B().gated_norm(x, None, None, 0, out, 1e-5, T)
    assert rel(out, x) < tol(dtype, 1e-7, 4e-3)


@pytest.mark.parametrize("E,top,groups,keep", [(20, 3, 5, 3), (7, 7, 1, 1), (12, 1, 6, 1), (130, 6, 10, 4), (64, 8, 64, 8)])
def test_router_select_and_moe_mix(E, top, groups, keep):
    T = 37
    logits, corr = rnd(T, E, seed=E, scale=2.0), rnd(E, seed=E + 1, scale=0.1)
    corr[1] = -1.5                                          # a choice score below zero must still beat a dropped group's outputs
    expert = torch.empty(T * top, dtype=torch.int32, device=DEV)
    weight = torch.empty(T * top, dtype=torch.float32, device=DEV)
    B().router_select(logits, top, expert, weight, T, score_fn=B().SCORE_SOFTMAX, correction=corr, groups=groups, groups_keep=keep,
                      renorm=True)
    idx, w = O.choose(logits.to(F64).cpu(), corr.to(F64).cpu(), top, groups, keep)
    assert torch.equal(expert.view(T, top).cpu().long(), idx) and rel(weight.view(T, top), w) < 1e-6
    Wd, n_real = 30, max(1, E - 3)
    pair, h = rnd(T * top, Wd, seed=5), rnd(T, Wd, dtype=torch.bfloat16, seed=6)
    y = torch.empty((T, Wd), dtype=torch.float32, device=DEV)
    B().moe_mix(pair, expert, weight, h, n_real, y, T, top)
    pk = pair.to(F64).cpu().view(T, top, Wd)
    src = torch.where((idx >= n_real).unsqueeze(-1), h.to(F64).cpu().unsqueeze(1).expand(T, top, Wd), pk)
    assert rel(y, (w.unsqueeze(-1) * src).sum(dim=1)) < 1e-6


def attention_case(dtype, H, G, D, Dv, lens, news, seed=0, boost=None, splits=1, v_cols=False):
    """``lens[b]`` keys of request b are in the cache (its slot b), the last ``news[b]`` of them belong to this step's queries.
    The cache is one plane with interleaved key | value rows, or (``v_cols``) key rows plus a value plane kept column by column.
    Returns (kernel output, oracle output)."""
    cap, Bn = -(-(max(lens) + 3) // 32) * 32, len(lens)
    plane = rnd(Bn, G, cap, D + Dv, dtype=dtype, seed=seed + 1)
    T = sum(news)
    q = rnd(T, H * D + 5, dtype=dtype, seed=seed + 2)
    gate = rnd(T, H * Dv, dtype=dtype, seed=seed + 3)
    qs = (1.0 + rnd(T, seed=seed + 4).abs())
    if boost:                                               # one far key made to stand out for one query head
        b, key, head, amount = boost
        row = sum(news[:b]) + news[b] - 1
        plane[b, head // (H // G), key, :D] = (amount * q[row, head * D:(head + 1) * D].float() /
                                               q[row, head * D:(head + 1) * D].float().norm()).to(dtype)
    tiles, row0 = [], 0
    for b, (n, m) in enumerate(zip(lens, news)):
        for c in range(0, m, 16):
            tiles.append((b, n - m + c, min(16, m - c), row0 + c))
        row0 += m
    out = torch.empty((T, H * Dv), dtype=dtype, device=DEV)
    part = torch.empty(B().attn_softmax_part(T, H, splits, Dv), dtype=torch.float32, device=DEV) if splits > 1 else None
    rows = (G * cap * (D + Dv), cap * (D + Dv), D + Dv)
    if v_cols:
        vt = plane[..., D:].permute(0, 1, 3, 2).contiguous()                     # [slots, G, Dv, cap]
        for b, n in enumerate(lens):
            vt[b, :, :, n:] = float("nan")                                       # what lies past a request's keys need not be numbers
        B().attn_softmax(q, H * D + 5, dev_i32(tiles), len(tiles), plane, rows, vt, 0, (G * Dv * cap, Dv * cap, cap), True, H, G, D, Dv,
                         0.3, out, q_scale=qs, gate=gate, ldg=H * Dv, n_splits=splits, part=part)
    else:
        B().attn_softmax(q, H * D + 5, dev_i32(tiles), len(tiles), plane, rows, plane, D, rows, False, H, G, D, Dv, 0.3, out,
                         q_scale=qs, gate=gate, ldg=H * Dv, n_splits=splits, part=part)
    want, row0 = [], 0
    for b, (n, m) in enumerate(zip(lens, news)):
        qq = q[row0:row0 + m, :H * D].to(F64).cpu().view(m, H, D) * qs[row0:row0 + m].to(F64).cpu().view(m, 1, 1)
        kv = plane[b, :, :n].to(F64).cpu().permute(1, 0, 2)
        o = O.causal_softmax_attention(qq, kv[:, :, :D], kv[:, :, D:], 0.3, first_pos=n - m)
        want.append(o.reshape(m, H * Dv) * gate[row0:row0 + m].to(F64).cpu())
        row0 += m
    return out, torch.cat(want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("v_cols", [False, True])
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 56, 48), (3, 1, 10, 6), (8, 8, 32, 64), (2, 1, 128, 72), (2, 2, 160, 136), (5, 5, 64, 20)])
def test_softmax_attention_alone(dtype, H, G, D, Dv, v_cols):
    # prompts that end inside a 32-key block and a 16-query tile, a one-token step far into a cache, a first token
    got, want = attention_case(dtype, H, G, D, Dv, lens=[45, 131, 1, 32, 33], news=[45, 1, 1, 17, 2], seed=H, v_cols=v_cols)
    assert rel(got, want) < tol(dtype, 1e-5, 1.5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits,v_cols", [(2, False), (5, True), (16, True), (16, False)])
def test_softmax_attention_in_runs_of_the_keys(dtype, splits, v_cols):
    # more runs than some requests have key blocks: empty runs must drop out of the merge
    got, want = attention_case(dtype, 4, 2, 48, 40, lens=[45, 700, 1, 32, 33, 257], news=[45, 1, 1, 17, 2, 1], seed=splits, splits=splits,
                               v_cols=v_cols)
    assert rel(got, want) < tol(dtype, 1e-5, 1.5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("key,splits", [(0, 1), (31, 1), (32, 4), (127, 1), (128, 4), (299, 1), (299, 7)])
def test_softmax_attention_finds_a_far_key(dtype, key, splits):
    # the last query's score for ONE key of 300 is raised far above the rest: its head's output must be that key's value
    got, want = attention_case(dtype, 2, 1, 40, 24, lens=[300, 300], news=[1, 20], seed=3, boost=(1, key, 1, 60.0), splits=splits,
                               v_cols=key % 2 == 1)
    assert rel(got, want) < tol(dtype, 1e-5, 1.5e-2)
    assert rel(got[-1, 24:], want[-1, 24:]) < tol(dtype, 1e-5, 1.5e-2)


def decay_case(dtype, H, D, Dv, decay, counts, carried, seed=0):
    """Requests of ``counts[b]`` tokens; ``carried[b]``: the slot holds a state (the request does not start at position 0)."""
    Bn, T = len(counts), sum(counts)
    ld = 2 * H * D + H * Dv + 3
    x = rnd(T, ld, dtype=dtype, seed=seed + 1, scale=0.7)
    state = rnd(Bn + 1, H, D, Dv, seed=seed + 2)
    before = state.to(F64).cpu()
    reqs, row0 = [], 0
    for b, c in enumerate(counts):
        reqs.append((b + 1, 5 if carried[b] else 0, c, row0))
        row0 += c
    out = torch.empty((T, H * Dv), dtype=torch.float32, device=DEV)
    dec = torch.tensor(decay, dtype=torch.float32, device=DEV)
    B().decay_attn(x, x[:, H * D:], x[:, 2 * H * D:], ld, dev_i32(reqs), Bn, state, dec, H, D, Dv, out)
    xf = x.to(F64).cpu()
    row0 = 0
    for b, c in enumerate(counts):
        r = xf[row0:row0 + c]
        o, S = O.decayed_linear_attention(r[:, :H * D].view(c, H, D), r[:, H * D:2 * H * D].view(c, H, D),
                                          r[:, 2 * H * D:2 * H * D + H * Dv].view(c, H, Dv), decay,
                                          state=before[b + 1] if carried[b] else None)
        assert rel(out[row0:row0 + c], o.reshape(c, H * Dv)) < 5e-6, (b, c)
        assert rel(state[b + 1], S) < 5e-6, (b, c)
        row0 += c
    assert torch.equal(state[0].to(F64).cpu(), before[0])                                        # a slot nobody used


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv,decay", [(3, 64, 48, (0.6, 0.95, 0.999)), (1, 6, 10, (0.8,)), (2, 40, 16, (1.0, 0.3)),
                                           (2, 96, 48, (0.9, 0.99)), (1, 200, 20, (0.97,))])
def test_decayed_linear_attention_alone(dtype, H, D, Dv, decay):
    # chunks of 16: counts just below, at and above a chunk's edge, a single token, carried and fresh states
    decay_case(dtype, H, D, Dv, decay, counts=[15, 16, 17, 1, 49, 1], carried=[False, True, True, True, False, False], seed=H + D)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,taps", [(30, 2), (72, 4), (300, 1), (17, 7)])
def test_causal_convolution_and_its_state(dtype, C, taps):
    # requests: a fresh one, one whose step is shorter than the taps (the state is shifted, not replaced), one long, one token
    counts, firsts = [5, 2, 20, 1, 1], [0, 9, 3, 0, 1]
    T, Bn = sum(counts), len(counts)
    x = rnd(T, C + 4, dtype=dtype, seed=1)
    w, b = rnd(C, taps, dtype=dtype, seed=2), rnd(C, dtype=dtype, seed=3)
    state = rnd(Bn, taps - 1, C, dtype=dtype, seed=4)
    before = state.to(F64).cpu()
    meta, reqs, row0 = [], [], 0
    for s_, (c, f) in enumerate(zip(counts, firsts)):
        reqs.append((s_, f, c, row0))
        meta += [(s_, f + i, i, 0) for i in range(c)]
        row0 += c
    out = torch.empty((T, C), dtype=dtype, device=DEV)
    B().causal_conv(x, C + 4, w, b, True, dev_i32(meta), state, out, T)
    B().conv_state_update(x, C + 4, dev_i32(reqs), Bn, state)
    xf, row0 = x.to(F64).cpu()[:, :C], 0
    for s_, (c, f) in enumerate(zip(counts, firsts)):
        prev = before[s_].clone()
        if taps > 1 and f < taps - 1:
            prev[:taps - 1 - f] = 0.0                      # positions before the start are zeros whatever the slot held
        want = O.silu(O.causal_convolution(xf[row0:row0 + c], w.to(F64).cpu(), b.to(F64).cpu(), before=prev))
        assert rel(out[row0:row0 + c], want) < tol(dtype, 1e-6, 6e-3), s_
        if taps > 1:
            hist = torch.cat([prev, xf[row0:row0 + c]])[-(taps - 1):]
            assert torch.equal(state[s_].to(F64).cpu()[-min(taps - 1, f + c):], hist[-min(taps - 1, f + c):]), s_
        row0 += c


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,N", [(72, 10), (30, 1), (200, 40), (64, 16), (10, 100)])
def test_selective_scan_alone(dtype, C, N):
    counts, carried = [33, 1, 1, 6], [False, True, False, True]
    T, Bn = sum(counts), len(counts)
    x, z = rnd(T, C, dtype=dtype, seed=1), rnd(T, 2 * C, dtype=dtype, seed=2)
    dt = torch.nn.functional.softplus(rnd(T, C, seed=3) - 1.0).contiguous()
    bc = rnd(T, 2 * N, seed=4, scale=0.5)
    A, D = (-rnd(C, N, seed=5).abs() - 0.05).contiguous(), rnd(C, seed=6)
    state = rnd(Bn, C, N, seed=7)
    before = state.to(F64).cpu()
    reqs, row0 = [], 0
    for b, c in enumerate(counts):
        reqs.append((b, 3 if carried[b] else 0, c, row0))
        row0 += c
    out = torch.empty((T, C), dtype=dtype, device=DEV)
    B().selective_scan(x, dt, bc, z[:, C:], 2 * C, A, D, dev_i32(reqs), Bn, state, out)
    f = lambda t: t.to(F64).cpu()
    row0 = 0
    for b, c in enumerate(counts):
        sl = slice(row0, row0 + c)
        y, S = O.selective_scan(f(x)[sl], f(dt)[sl], f(bc)[sl, :N], f(bc)[sl, N:], f(A), f(D), state=before[b] if carried[b] else None)
        assert rel(out[sl], y * O.silu(f(z)[sl, C:])) < tol(dtype, 2e-6, 6e-3), b
        assert rel(state[b], S) < 2e-6, b
        row0 += c


# =====================================================================================================================================
# the model through its arena
# =====================================================================================================================================
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,n", [("mixed", 41), ("odd", 19), ("wide", 70), ("mixed", 1)])
def test_prompt_matches_oracle_layer_by_layer(name, n, dtype):
    s, w, m = model(name, dtype)
    t = toks(n, s.vocab_size, seed=n)
    want, sums = O.forward(t, w, s, return_layers=True)
    ar = m.new_arena(1, 8)
    got, got_sums = m.forward_rows(ar, [ar.alloc()], [t], [list(range(n))], return_streams=True)
    for i in range(len(s.layers)):
        assert rel(got_sums[i], sums[i]) < tol(dtype, 2e-5, 2.5e-2), (i, s.layers[i].kind)
    assert rel(got, want) < tol(dtype, 2e-5, 3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,n", [("mixed", 37), ("odd", 12), ("wide", 35)])
def test_decoding_token_by_token_equals_the_prompt(name, n, dtype):
    s, w, m = model(name, dtype)
    t = toks(n, s.vocab_size, seed=100 + n)
    want = O.forward(t, w, s)
    assert rel(run_alone(m, t, [1] * n), want) < tol(dtype, 2e-5, 3e-2)
    assert rel(run_alone(m, t, [n - 20 if n > 20 else 1] + [1] * min(20, n - 1)), want) < tol(dtype, 2e-5, 3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cuts", [[2] * 20, [17, 2, 16, 5], [33, 7], [1, 15, 1, 16, 1, 6], [3, 37]])
def test_portions_of_a_prompt(cuts, dtype):
    s, w, m = model("mixed", dtype)
    t = toks(40, s.vocab_size, seed=7)
    assert rel(run_alone(m, t, cuts), O.forward(t, w, s)) < tol(dtype, 2e-5, 3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "odd"])
def test_segmented_prefill_of_the_recurrent_mixers(name, dtype, monkeypatch):
    # segments of 16 tokens: prompts of several ragged segments, a portion that continues a carried state, an unequal batch
    s, w, m = model(name, dtype)
    monkeypatch.setattr(m, "SEGMENT", 16)
    t = toks(75, s.vocab_size, seed=3)
    want = O.forward(t, w, s)
    assert rel(run_alone(m, t), want) < tol(dtype, 2e-5, 3e-2)
    assert rel(run_alone(m, t, [3, 40, 32]), want) < tol(dtype, 2e-5, 3e-2)
    u = toks(17, s.vocab_size, seed=4)
    ar = m.new_arena(2, 8)
    got = m.forward_rows(ar, [ar.alloc(), ar.alloc()], [u, t], [list(range(17)), list(range(75))])
    assert rel(got, torch.cat([O.forward(u, w, s), want])) < tol(dtype, 2e-5, 3e-2)
    monkeypatch.setattr(m, "MAX_SEGMENTS", 2)              # longer segments rather than more of them
    assert rel(run_alone(m, t), want) < tol(dtype, 2e-5, 3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_past_block_and_temperature_edges(dtype):
    # 150 prompt tokens, then 120 decoded one by one through the captured graph: the attention crosses several 32-key blocks,
    # the temperature steps every 7 positions, the lightning and scan states are carried 120 times
    s, w, m = model("mixed", dtype)
    t = toks(270, s.vocab_size, seed=9)
    want = O.forward(t, w, s)
    ar = m.new_arena(1, 512)
    sl = ar.alloc()
    got = [m.forward_rows(ar, [sl], [t[:150]], [[149]])]
    for p in range(150, 270):
        got.append(m.forward_rows(ar, [sl], [[t[p]]], [[0]]))
    assert rel(torch.cat(got), want[149:]) < tol(dtype, 3e-5, 3e-2)
    assert rel(got[-1], want[-1:]) < tol(dtype, 3e-5, 3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_batch_equals_each_alone_and_slots_are_reused(dtype):
    s, w, m = model("mixed", dtype)
    prompts = [toks(n, s.vocab_size, seed=50 + n) for n in (1, 23, 9, 40)]
    alone = [O.forward(p + toks(6, s.vocab_size, seed=70 + i), w, s) for i, p in enumerate(prompts)]
    tails = [toks(6, s.vocab_size, seed=70 + i) for i in range(4)]
    ar = m.new_arena(2, 16)                                 # fewer slots and shorter rows than the batch needs: both grow
    slots = [ar.alloc() for _ in prompts]
    got = m.forward_rows(ar, slots, prompts, [list(range(len(p))) for p in prompts])
    at = 0
    for i, p in enumerate(prompts):
        assert rel(got[at:at + len(p)], alone[i][:len(p)]) < tol(dtype, 2e-5, 3e-2), i
        at += len(p)
    for k in range(6):                                      # decoded together; request 1 leaves after three tokens
        live = [i for i in range(4) if not (i == 1 and k >= 3)]
        got = m.forward_rows(ar, [slots[i] for i in live], [[tails[i][k]] for i in live], [[0]] * len(live))
        for r, i in enumerate(live):
            assert rel(got[r], alone[i][len(prompts[i]) + k]) < tol(dtype, 3e-5, 3e-2), (k, i)
        if k == 2:
            ar.free(slots[1])
    # the freed slot goes to a newcomer: what its last owner left in the cache and in the states must not show
    sl = ar.alloc()
    assert sl == slots[1]
    fresh = toks(11, s.vocab_size, seed=90)
    got = m.forward_rows(ar, [sl, slots[3]], [fresh, [3]], [list(range(11)), []])
    assert rel(got, O.forward(fresh, w, s)) < tol(dtype, 2e-5, 3e-2)


def test_same_rows_same_values_whatever_the_company():
    s, w, m = model("mixed", torch.float32)
    a, b = toks(21, s.vocab_size, seed=1), toks(5, s.vocab_size, seed=2)
    ar = m.new_arena(3, 64)
    s0, s1, s2 = ar.alloc(), ar.alloc(), ar.alloc()
    both = m.forward_rows(ar, [s1, s0], [b, a], [[4], list(range(21))])
    alone = m.forward_rows(ar, [s2], [a], [list(range(21))])
    assert rel(both[1:], alone) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
def test_graph_replays_equal_eager_steps(dtype):
    s, w, m = model("wide", dtype)
    prompts = [toks(n, s.vocab_size, seed=20 + n) for n in (30, 3)]
    steps = [toks(2, s.vocab_size, seed=40 + k) for k in range(5)]

    def run(graphs):
        m.use_graphs = graphs
        ar = m.new_arena(2, 64)
        sl = [ar.alloc(), ar.alloc()]
        out = [m.forward_rows(ar, sl, prompts)]
        for st in steps:
            out.append(m.forward_rows(ar, sl, [[st[0]], [st[1]]]))
            torch.cuda.synchronize()
        return torch.cat(out)
    try:
        eager, replayed = run(False), run(True)
    finally:
        m.use_graphs = True
    assert rel(replayed, eager) < 1e-6


def test_greedy_generation_through_both_engines():
    from promptcache_amd import BatchEngine, GenerationEngine, GenerationParameters
    from promptcache_amd.model import Dibizen
    s = shape_mixed()
    w = W.make_dibizen_weights(s, seed=21)
    lm = Dibizen(shape=s, weights=w, device=DEV, dtype=torch.float32)
    prompts = [toks(13, s.vocab_size, 30), toks(5, s.vocab_size, 31), toks(22, s.vocab_size, 32)]
    want = [O.greedy(s, w, p, 6) for p in prompts]
    params = GenerationParameters(temperature=0.0, max_new_tokens=6, stop_token_ids=[])
    assert BatchEngine(lm).generate(prompts, params) == want
    assert BatchEngine(lm, max_tokens=30).generate(prompts, params) == want        # admitted in turns: same tokens
    p = prompts[0]
    out = None
    for out in GenerationEngine(lm).generate(p, list(range(len(p))), params):
        pass
    assert out is not None and lm.decode(want[0]) == out.new_text
    ids = torch.zeros((2, 13), dtype=torch.long)
    mask = torch.zeros((2, 13), dtype=torch.long)
    ids[0, :13], mask[0, :13] = torch.tensor(prompts[0]), 1
    ids[1, :5], mask[1, :5] = torch.tensor(prompts[1]), 1
    res = lm(input_ids=ids, attention_mask=mask, past_key_values=None, use_cache=True)
    assert int(res.logits[0, 12].argmax()) == want[0][0] and int(res.logits[1, 4].argmax()) == want[1][0]


def test_positions_beyond_the_table_are_refused():
    s, w, m = model("odd", torch.float32)
    ar = m.new_arena(1, 8)
    with pytest.raises(ValueError, match="position"):
        m.forward_rows(ar, [ar.alloc()], [toks(s.max_positions + 1, s.vocab_size)])


def test_trace_runner_replays_steps(tmp_path):
    from safetensors.torch import save_file
    import numpy as np
    s = shape_odd()
    w = W.make_dibizen_weights(s, seed=40)
    mdir = tmp_path / "model"
    mdir.mkdir()
    save_file(w, str(mdir / "model.safetensors"))
    (mdir / "config.json").write_text(json.dumps(s.to_config()))
    a, b = toks(9, s.vocab_size, 41), toks(4, s.vocab_size, 42)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:8], "want": [0, 7]}, {"id": "b", "tokens": b[:3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[8:], "want": [0]}, {"id": "b", "tokens": b[3:], "want": [0]}], "end": ["a", "b"]},
             {"step": 2, "entries": [{"id": "c", "tokens": b, "want": [3]}], "end": ["c"]}]
    for dtype, lim in (("float32", 5e-6), ("bfloat16", 3e-2)):
        out = tmp_path / ("out_" + dtype)
        r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dtype, "--out", str(out),
                            "--max-tokens", "32"], input="\n".join(json.dumps(x) for x in steps) + "\n", capture_output=True,
                           text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
        wa, wb = O.forward(a, w, s), O.forward(b, w, s)
        g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4")).view(2, -1)
        g1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4")).view(2, -1)
        g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4")).view(1, -1)
        assert rel(g0, wa[[0, 7]]) < lim and rel(g1, torch.stack([wa[8], wb[3]])) < lim and rel(g2, wb[3:4]) < lim
