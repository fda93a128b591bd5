"""Kazolorn on the GPU against the plain float64 oracle (``oracle/kazolorn_oracle.py``): every building-block kernel alone,
then the model through its arena -- prompts, token-by-token decoding, portions, unequal batches, reused slots, window edges,
growth of the arena -- and greedy generation through both engines.  float32 runs are held to float32 accuracy; bfloat16 runs to
what bf16 operands allow, and to themselves (the same position must not depend on how it was reached)."""
import json
import os
import subprocess
import sys

import pytest
import torch

from oracle import kazolorn_oracle as O
from promptcache_amd.model import weights as W
from promptcache_amd.model.config import KazolornLayer, KazolornShape

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


# ---- shapes (none of them a round power-of-two model; layers differ from one another) -----------------------------------------------
def shape_mixed():
    return KazolornShape(vocab_size=160, hidden_size=96, norm_eps=1e-5, layers=[
        KazolornLayer(heads=4, kv_heads=4, dim=20, scale=0.3, window=9, mlp_kind="dense", ff=40),
        KazolornLayer(heads=6, kv_heads=3, dim=16, scale=0.35, window=0, mlp_kind="moe", ff=24, experts=5, top=2),
        KazolornLayer(heads=2, kv_heads=1, dim=32, scale=0.2, window=5, mlp_kind=None),
        KazolornLayer(heads=8, kv_heads=2, dim=8, scale=0.5, window=20, mlp_kind="moe", ff=16, experts=3, top=3),
    ])


def shape_odd():
    """Widths that are no multiple of a 16-byte chunk in either element type, one head, one expert, window 1."""
    return KazolornShape(vocab_size=75, hidden_size=50, norm_eps=1e-6, layers=[
        KazolornLayer(heads=1, kv_heads=1, dim=10, scale=0.4, window=1, mlp_kind="moe", ff=14, experts=1, top=1),
        KazolornLayer(heads=3, kv_heads=1, dim=6, scale=0.6, window=4, mlp_kind="dense", ff=22),
    ])


def shape_wide():
    """Enough rows, heads and keys to cross every tile edge: 16 heads, windows over several 64-key blocks."""
    return KazolornShape(vocab_size=320, hidden_size=128, norm_eps=1e-6, layers=[
        KazolornLayer(heads=16, kv_heads=4, dim=32, scale=0.18, window=70, mlp_kind="dense", ff=192),
        KazolornLayer(heads=16, kv_heads=4, dim=32, scale=0.18, window=131, mlp_kind="moe", ff=64, experts=8, top=2),
    ])


SHAPES = {"mixed": shape_mixed, "odd": shape_odd, "wide": shape_wide}
_models = {}


def model(name, dtype, seed=11):
    from promptcache_amd.model.kazolorn_hip import KazolornHIP
    key = (name, dtype, seed)
    if key not in _models:
        s = SHAPES[name]()
        w = W.make_kazolorn_weights(s, seed=seed)
        _models[key] = (s, w, KazolornHIP(s, w, device=DEV, dtype=dtype))
    return _models[key]


def toks(n, vocab, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def run_alone(m, tokens, cuts=None, want=None):
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
@pytest.mark.parametrize("M,N,K", [(1, 24, 20), (5, 130, 96), (70, 40, 100), (200, 150, 50), (33, 16, 7)])
def test_linear_store_and_bias(dtype, M, N, K):
    x, w, b = rnd(M, K, dtype=dtype, seed=1), rnd(N, K, dtype=dtype, seed=2, scale=0.2), rnd(N, dtype=dtype, seed=3)
    want = x.to(F64) @ w.to(F64).T + b.to(F64)
    y = torch.empty((M, N), dtype=dtype, device=DEV)
    B().linear(x, w, y, M=M, bias=b)
    assert rel(y, want) < tol(dtype, 1e-6, 4e-3)
    y32 = torch.empty((M, N), dtype=torch.float32, device=DEV)
    B().linear(x, w, y32, M=M, bias=b)
    assert rel(y32, want) < tol(dtype, 1e-6, 1e-4 if K < 60 else 3e-4)       # fp32 out: only the operands are rounded, and they are exact here


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_scale_add_and_split_destination(dtype):
    M, N, K = 37, 52, 44
    x, w, b = rnd(M, K, dtype=dtype, seed=1), rnd(N, K, dtype=dtype, seed=2, scale=0.3), rnd(N, dtype=dtype, seed=3)
    cs, base = rnd(N, seed=4), rnd(M, N, seed=5)
    lin = x.to(F64) @ w.to(F64).T + b.to(F64)
    y = torch.full((M, N), 9.0, dtype=torch.float32, device=DEV)
    B().linear(x, w, y, M=M, epilogue=B().EPI_SCALE_ADD, bias=b, base=base, col_scale=cs)
    assert rel(y, base.to(F64).cpu() + cs.to(F64).cpu() * lin.cpu()) < 1e-5
    B().linear(x, w, y, M=M, epilogue=B().EPI_SCALE_ADD, bias=b, col_scale=cs)          # no base: accumulate
    assert rel(y, base.to(F64).cpu() + 2 * cs.to(F64).cpu() * lin.cpu()) < 1e-5
    # columns >= split go to a [slot][head][pos][dim] cache through per-row offsets
    G, D, cap, split = 3, 4, 11, 40
    cache = torch.zeros((5, G, cap, D), dtype=dtype, device=DEV)
    slot = torch.tensor([(r * 3) % 5 for r in range(M)])
    pos = torch.tensor([r // 5 for r in range(M)])
    off = (slot * G * cap * D + pos * D).to(torch.int64).to(DEV)
    q = torch.empty((M, split), dtype=dtype, device=DEV)
    B().linear(x, w, q, M=M, bias=b, split_n=split, y2=cache, row_off2=off, head_dim2=D, head_stride2=cap * D)
    assert rel(q, lin[:, :split]) < tol(dtype, 1e-6, 4e-3)
    for r in range(M):
        got = cache[slot[r], :, pos[r], :].reshape(-1)
        assert rel(got, lin[r, split:]) < tol(dtype, 1e-6, 6e-3), r


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows_per", [3, 90])
def test_linear_groups_gather_scale_and_gate(dtype, rows_per):
    E, N, K, T = 4, 28, 36, 50
    g = torch.Generator().manual_seed(7)
    sizes = [rows_per, 0, rows_per + 5, 1]
    off = torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32)
    P = int(off[-1])
    src = torch.randint(0, T, (P,), generator=g, dtype=torch.int32)
    scl = torch.rand(P, generator=g) + 0.25
    dst = torch.randperm(P, generator=g).to(torch.int32)
    x = rnd(T, K, dtype=dtype, seed=1)
    wg, wu = rnd(E, N, K, dtype=dtype, seed=2, scale=0.3), rnd(E, N, K, dtype=dtype, seed=3, scale=0.3)
    y = torch.empty((P, N), dtype=dtype, device=DEV)
    B().linear(x, wg, y, M=P, epilogue=B().EPI_SILU_MUL, w2=wu, row_src=src.to(DEV), row_scale=scl.to(DEV),
               group_off=off.to(DEV), n_groups=E)
    y2 = torch.zeros((P, N), dtype=torch.float32, device=DEV)
    B().linear(x, wg, y2, M=P, row_src=src.to(DEV), group_off=off.to(DEV), n_groups=E, row_dst=dst.to(DEV))
    for e in range(E):
        for r in range(int(off[e]), int(off[e + 1])):
            xr = (scl[r].to(F64) * x[src[r]].to(F64).cpu())
            if dtype == torch.bfloat16:
                xr = xr.to(torch.bfloat16).to(F64)                      # the scaled row is rounded to the element type
            a, u = xr @ wg[e].to(F64).cpu().T, xr @ wu[e].to(F64).cpu().T
            assert rel(y[r], a * torch.sigmoid(a) * u) < tol(dtype, 1e-5, 8e-3), (e, r)
            plain = x[src[r]].to(F64).cpu() @ wg[e].to(F64).cpu().T
            assert rel(y2[dst[r]], plain) < 1e-4, (e, r)


@pytest.mark.parametrize("dtype", DTYPES)
def test_mix_norm_and_embedding(dtype):
    S, T, Wd = 4, 9, 50
    table = rnd(30, Wd, dtype=dtype, seed=1)
    ids = torch.tensor([3, 29, 0, 7, 7, 12, 1, 2, 28], dtype=torch.int32, device=DEV)
    hist = rnd(S, T, Wd, seed=2)
    B().embed_rows(table, ids, hist[0])
    assert torch.equal(hist[0], table[ids.long()].float())
    coef, g1, g2 = rnd(S, seed=3), rnd(Wd, seed=4), rnd(Wd, seed=5)
    o1, o2 = torch.empty((T, Wd), dtype=dtype, device=DEV), torch.empty((T, Wd), dtype=dtype, device=DEV)
    x = torch.empty((T, Wd), dtype=torch.float32, device=DEV)
    B().mix_norm(hist, 3, coef, g1, o1, g2, o2, x_out=x, eps=1e-3, n_rows=T)
    want_x = sum(coef[j].to(F64) * hist[j].to(F64) for j in range(3))              # only the first three streams
    assert rel(x, want_x) < 1e-6
    assert rel(o1, O.rms_norm(want_x.cpu(), g1.to(F64).cpu(), 1e-3)) < tol(dtype, 1e-6, 4e-3)
    assert rel(o2, O.rms_norm(want_x.cpu(), g2.to(F64).cpu(), 1e-3)) < tol(dtype, 1e-6, 4e-3)
    rows = torch.tensor([8, 2, 2], dtype=torch.int32, device=DEV)                  # gathered rows, no sum: stream 0 as it is
    o3 = torch.empty((3, Wd), dtype=dtype, device=DEV)
    B().mix_norm(hist, 1, None, g1, o3, rows=rows, eps=1e-3)
    assert rel(o3, O.rms_norm(hist[0].to(F64).cpu()[[8, 2, 2]], g1.to(F64).cpu(), 1e-3)) < tol(dtype, 1e-6, 4e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_polynorm(dtype):
    z = rnd(7, 333, seed=1, scale=2.0)
    coef = torch.tensor([0.7, -0.4, 0.3, 0.2], device=DEV)
    out = torch.empty((7, 333), dtype=dtype, device=DEV)
    B().polynorm(z, coef, out, 1e-4, 7)
    assert rel(out, O.poly_activation(z.to(F64).cpu(), coef.cpu(), 1e-4)) < tol(dtype, 1e-6, 4e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top", [(5, 2), (1, 1), (70, 3), (12, 12)])
def test_router_and_plan(dtype, E, top):
    T, Wd = 23, 44
    h, wr = rnd(T, Wd, dtype=dtype, seed=1), rnd(E, Wd, dtype=dtype, seed=2, scale=0.4)
    ex = torch.empty(T * top, dtype=torch.int32, device=DEV)
    wt = torch.empty(T * top, dtype=torch.float32, device=DEV)
    logits = torch.empty((T, E), dtype=torch.float32, device=DEV)
    B().linear(h, wr, logits, M=T)
    B().router_topk(logits, top, ex, wt, T)
    idx, val = O.route(h.to(F64).cpu(), wr.to(F64).cpu(), top)
    assert torch.equal(ex.view(T, top).cpu().long(), idx)
    assert rel(wt.view(T, top), val) < 1e-5
    P = T * top
    goff = torch.empty(E + 1, dtype=torch.int32, device=DEV)
    src, dst = torch.empty(P, dtype=torch.int32, device=DEV), torch.empty(P, dtype=torch.int32, device=DEV)
    scl = torch.empty(P, dtype=torch.float32, device=DEV)
    B().moe_plan(ex, wt, P, top, E, goff, src, dst, scl)
    goff, src, dst, scl = goff.cpu(), src.cpu(), dst.cpu(), scl.cpu()
    assert int(goff[0]) == 0 and int(goff[-1]) == P and sorted(dst.tolist()) == list(range(P))
    for e in range(E):
        for r in range(int(goff[e]), int(goff[e + 1])):
            p = int(dst[r])
            assert int(ex[p]) == e and int(src[r]) == p // top and float(scl[r]) == float(wt[p])
    pair, ls = rnd(P, 10, seed=3), rnd(10, seed=4)
    y = rnd(T, 10, seed=5)
    want = y.to(F64) + ls.to(F64) * pair.to(F64).view(T, top, 10).sum(1)
    B().moe_combine(pair, ls, y, T, top)
    assert rel(y, want) < 1e-6


def _attn_case(dtype, H, G, D, window, n, first, talk_noise=0.2, seed=0, spike=None):
    """Queries for positions first .. n-1 over cached keys 0 .. n-1 in slot 1 of a 3-slot cache; returns (got, want)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n - first, H, D, generator=g)
    k = torch.randn(n, G, D, generator=g)
    if spike is not None:                      # one (query row, key) pair whose score towers over the rest, in every head
        qi, kj, gain = spike
        k[kj] = 0.0
        k[kj, :, 0] = gain
        q[qi - first, :, 0] = gain
    q, k = q.to(dtype), k.to(dtype)
    talk = torch.eye(H) + talk_noise * torch.randn(H, H, generator=g)
    cap = n + 3
    cache = torch.zeros((3, G, cap, D), dtype=dtype, device=DEV)
    cache[1, :, :n] = k.permute(1, 0, 2).to(DEV)
    m = n - first
    tiles = torch.tensor([[1, first + t, min(16, m - t), t] for t in range(0, m, 16)], dtype=torch.int32, device=DEV)
    band = B().attn_talk_band(window, n)
    scratch = torch.empty(tiles.shape[0] * 16 * H * band, dtype=torch.float32, device=DEV)
    out = torch.empty((m, H * D), dtype=dtype, device=DEV)
    slopes = O.head_slopes(H).float().to(DEV)
    B().attn_talk(q.reshape(m, H * D).contiguous().to(DEV), tiles, tiles.shape[0], cache, G * cap * D, cap * D, H, G, D, 0.3, window, n,
                  slopes, talk.to(DEV), True, scratch, out)
    want = O.talking_attention(q.to(F64), k.to(F64), 0.3, window, talk.to(F64), first_pos=first)
    return out.view(m, H, D), want, k


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,window,n,first", [
    (4, 2, 16, 9, 40, 0),        # a prompt
    (4, 2, 16, 9, 40, 39),       # one decoded token
    (6, 3, 20, 0, 150, 100),     # a portion, no window, keys over several 64-key blocks, head size off the 16-byte grid
    (1, 1, 10, 1, 20, 0),        # window 1: every token sees itself and the sink only
    (16, 4, 32, 70, 200, 0),     # many heads, window across key blocks
    (3, 3, 6, 4, 19, 17),        # two rows ending a sequence
    (32, 8, 8, 33, 50, 0),       # the most heads the kernel takes
    (12, 4, 24, 0, 70, 0),       # head counts between the kernel's register tiers
    (24, 24, 16, 21, 45, 40),
    (2, 1, 160, 40, 90, 0),      # heads wider than 128 columns (the 8-step score kernel, 16 value subtiles)
    (4, 2, 256, 0, 37, 30),      # ... and the widest
    (20, 5, 136, 17, 40, 0),     # many heads AND wide heads
])
def test_attention_alone(dtype, H, G, D, window, n, first):
    got, want, _ = _attn_case(dtype, H, G, D, window, n, first)
    assert rel(got, want) < tol(dtype, 2e-6, 1.5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("first", [0, 30, 63])           # in a prompt, in a portion, decoded alone
def test_attention_window_edges_and_far_keys(dtype, first):
    H, G, D, window, n = 4, 2, 16, 25, 64
    qi = 63
    inside, outside = qi - (window - 1), qi - window
    # a towering key on the last position the window keeps: the row's output is that key
    got, want, k = _attn_case(dtype, H, G, D, window, n, first, talk_noise=0.0, spike=(qi, inside, 9.0))
    assert rel(got, want) < tol(dtype, 2e-6, 1.5e-2)
    assert rel(got[qi - first, 0], k[inside, 0].to(F64)) < 2e-2
    # the same key one step further back is out of sight: the row must not move towards it
    got, want, k = _attn_case(dtype, H, G, D, window, n, first, talk_noise=0.0, spike=(qi, outside, 9.0))
    assert rel(got, want) < tol(dtype, 2e-6, 1.5e-2)
    assert float((got[qi - first, 0].to("cpu", F64) - k[outside, 0].to(F64)).abs().max()) > 3.0
    # without a window a key 60 positions back, among all the others, still decides the row
    got, want, k = _attn_case(dtype, H, G, D, 0, n, first, talk_noise=0.0, spike=(qi, 3, 12.0))
    assert rel(got, want) < tol(dtype, 2e-6, 1.5e-2)
    assert rel(got[qi - first, 3], k[3, 1].to(F64)) < 2e-2


def test_attention_sink_and_mixing_matter():
    """Dropping the sink or the head mixing is visible at fp32 accuracy (so the comparisons above cover them)."""
    H, G, D, n = 4, 2, 16, 12
    got, want, k = _attn_case(torch.float32, H, G, D, 0, n, 0, talk_noise=0.5, seed=3)
    q_dummy = torch.zeros(n, H, D, dtype=F64)
    zero = O.talking_attention(q_dummy, k.to(F64), 0.3, 0, torch.eye(H, dtype=F64))
    first_row = zero[0, 0]                     # one key with score 0 and the sink: weight exactly one half
    assert torch.allclose(first_row, 0.5 * k[0, 0].to(F64))
    assert rel(got, want) < 2e-6


# =====================================================================================================================================
# the model through its arena
# =====================================================================================================================================
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,n", [("mixed", 45), ("odd", 19), ("wide", 150), ("wide", 330)])      # 330: > 64 rows per expert
def test_prompt_matches_oracle_layer_by_layer(name, n, dtype):
    s, w, m = model(name, dtype)
    t = toks(n, s.vocab_size, seed=1)
    ar = m.new_arena(1, 4)
    logits, streams = m.forward_rows(ar, [ar.alloc()], [t], [list(range(n))], return_streams=True)
    want, wstreams = O.forward(s, w, t, return_streams=True)
    for l in range(len(s.layers)):
        assert rel(streams[l], wstreams[l]) < tol(dtype, 2e-6, 1.5e-2), l
    assert rel(logits, want) < tol(dtype, 5e-6, 3e-2)
    # the first tokens of a sequence: one key, then two (nothing but the sink beside them)
    assert rel(logits[:2], want[:2]) < tol(dtype, 5e-6, 3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,n", [("mixed", 40), ("odd", 12)])
def test_decoding_token_by_token_equals_the_prompt(name, n, dtype):
    s, w, m = model(name, dtype)
    t = toks(n, s.vocab_size, seed=2)
    whole = run_alone(m, t)
    stepped = run_alone(m, t, cuts=[1] * n)                      # from the very first token on, one at a time
    assert rel(stepped, whole) < tol(dtype, 2e-6, 1.5e-2)
    assert rel(stepped, O.forward(s, w, t)) < tol(dtype, 5e-6, 3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cuts", [[2] * 20, [17, 3, 2, 16, 2], [1, 2, 33, 4], [39, 1], [16, 16, 8]])
def test_portions_of_a_prompt(cuts, dtype):
    s, w, m = model("mixed", dtype)
    n = sum(cuts)
    t = toks(n, s.vocab_size, seed=3)
    whole = run_alone(m, t)
    assert rel(run_alone(m, t, cuts=cuts), whole) < tol(dtype, 2e-6, 1.5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_window_passes_over_decoded_tokens_and_long_decoding(dtype):
    """A 70- and a 131-key window slide over decoded tokens (prompt 60, 120 decoded); rows past both edges match the oracle."""
    s, w, m = model("wide", dtype)
    t = toks(180, s.vocab_size, seed=4)
    got = run_alone(m, t, cuts=[60] + [1] * 120)
    want = O.forward(s, w, t)
    assert rel(got, want) < tol(dtype, 5e-6, 3e-2)
    for p in (68, 69, 70, 71, 129, 130, 131, 132, 179):          # just inside / outside either window
        assert rel(got[p], want[p]) < tol(dtype, 8e-6, 4e-2), p


@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_batch_equals_each_alone_and_slots_are_reused(dtype):
    s, w, m = model("mixed", dtype)
    from promptcache_amd import BatchEngine
    reqs = {"a": toks(37, s.vocab_size, 5), "b": toks(1, s.vocab_size, 6), "c": toks(18, s.vocab_size, 7), "d": toks(26, s.vocab_size, 8)}
    alone = {k: run_alone(m, v) for k, v in reqs.items()}
    eng = BatchEngine(m)
    # prompts of different lengths in one step (the last 4 tokens of each are left for decoding), then decode together;
    # shorter requests end earlier
    cut = {k: max(1, len(v) - 4) for k, v in reqs.items()}
    got = {k: [] for k in reqs}
    names = ["a", "b", "c"]
    out = eng.step([(k, reqs[k][:cut[k]], list(range(cut[k]))) for k in names])
    at = 0
    for k in names:
        got[k].append(out[at:at + cut[k]]); at += cut[k]
    pos = dict(cut)
    while names:
        live = [k for k in names if pos[k] < len(reqs[k])]
        ended = [k for k in names if pos[k] + 1 >= len(reqs[k])]
        if live:
            out = eng.step([(k, [reqs[k][pos[k]]], [0]) for k in live], end=ended)
            for r, k in enumerate(live):
                got[k].append(out[r:r + 1]); pos[k] += 1
        else:
            eng.step([], end=ended)
        names = [k for k in names if k not in ended]
    for k in ("a", "b", "c"):
        assert rel(torch.cat(got[k]), alone[k]) < tol(dtype, 1e-6, 1.5e-2), k
    # every slot was given back; a newcomer takes a used one and must not see what it held
    assert eng.held_tokens() == 0 and eng.arena.slots == 3
    out = eng.step([("d", reqs["d"], list(range(26)))], end=["d"])
    assert rel(out, alone["d"]) < tol(dtype, 1e-6, 1.5e-2)
    assert rel(alone["a"], O.forward(s, w, reqs["a"])) < tol(dtype, 5e-6, 3e-2)


def test_same_rows_same_values_whatever_the_company():
    """float32: a request's logits alone, in a batch and on another slot differ by summation order at most (which GEMM tiling a
    step's row count selects), never by what the other rows hold."""
    s, w, m = model("mixed", torch.float32)
    a, b = toks(21, s.vocab_size, 9), toks(30, s.vocab_size, 10)
    alone = run_alone(m, a)
    ar = m.new_arena(3, 8)
    s0, s1, s2 = ar.alloc(), ar.alloc(), ar.alloc()
    both = m.forward_rows(ar, [s2, s0], [b, a], [[], list(range(21))])
    assert rel(both, alone) < 1e-6
    other = m.forward_rows(ar, [s1], [a], [list(range(21))])              # same row count, another slot, dirty neighbours
    assert torch.equal(other, alone)
    # one-token steps (captured graph): logits of the rows that ask for them only, whatever the others ask for
    nxt_a, nxt_b = 5, 9
    full = m.forward_rows(ar, [s0, s2], [[nxt_a], [nxt_b]], [[0], [0]])
    ar2 = m.new_arena(2, 64)
    t0, t1 = ar2.alloc(), ar2.alloc()
    m.forward_rows(ar2, [t0, t1], [a, b], [[], []])
    part = m.forward_rows(ar2, [t0, t1], [[nxt_a], [nxt_b]], [[], [0]])
    none = m.forward_rows(ar2, [t0, t1], [[1], [2]], [[], []])
    assert part.shape == (1, s.vocab_size) and none.shape == (0, s.vocab_size)
    assert rel(part, full[1:2]) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
def test_arena_grows_under_a_live_request(dtype):
    s, w, m = model("mixed", dtype)
    t = toks(50, s.vocab_size, seed=12)
    ar = m.new_arena(1, 4)
    a = ar.alloc()
    first = m.forward_rows(ar, [a], [t[:20]], [list(range(20))])      # 20 > 4: rows grow before anything is written
    b = ar.alloc()                                                   # a second slot: the planes move, slot a keeps its rows
    rest = m.forward_rows(ar, [b, a], [t[:7], t[20:]], [[], list(range(30))])
    assert ar.cap >= 50 and ar.slots >= 2
    assert rel(torch.cat([first, rest]), run_alone(m, t)) < tol(dtype, 1e-6, 1.5e-2)


def test_long_prompt_in_several_attention_calls(monkeypatch):
    """A prompt whose score band would not fit the scratch budget runs its attention over runs of tiles; same logits."""
    from promptcache_amd.model import kazolorn_hip
    s, w, m = model("wide", torch.float32)
    t = toks(150, s.vocab_size, seed=13)
    whole = run_alone(m, t)
    monkeypatch.setattr(kazolorn_hip, "ATTN_SCRATCH_FLOATS", 3 * 16 * 16 * 160)      # three 16-row tiles per call
    assert rel(run_alone(m, t), whole) < 1e-6


def test_greedy_generation_through_both_engines():
    from promptcache_amd import BatchEngine, GenerationEngine, GenerationParameters
    from promptcache_amd.model import Kazolorn
    s = shape_mixed()
    w = W.make_kazolorn_weights(s, seed=21)
    lm = Kazolorn(shape=s, weights=w, device=DEV, dtype=torch.float32)
    prompts = [toks(13, s.vocab_size, 30), toks(5, s.vocab_size, 31), toks(22, s.vocab_size, 32)]
    want = [O.greedy(s, w, p, 6) for p in prompts]
    params = GenerationParameters(temperature=0.0, max_new_tokens=6, stop_token_ids=[])
    assert BatchEngine(lm).generate(prompts, params) == want
    assert BatchEngine(lm, max_tokens=30).generate(prompts, params) == want        # admitted in turns: same tokens
    # the single-request engine drives the same model through the adapter's calling convention
    p = prompts[0]
    out = None
    for out in GenerationEngine(lm).generate(p, list(range(len(p))), params):
        pass
    assert out is not None and lm.decode(want[0]) == out.new_text
    # the adapter call with a right-padded batch: each row's last logits equal its own prompt's
    ids = torch.zeros((2, 13), dtype=torch.long)
    mask = torch.zeros((2, 13), dtype=torch.long)
    ids[0, :13], mask[0, :13] = torch.tensor(prompts[0]), 1
    ids[1, :5], mask[1, :5] = torch.tensor(prompts[1]), 1
    res = lm(input_ids=ids, attention_mask=mask, past_key_values=None, use_cache=True)
    assert int(res.logits[0, 12].argmax()) == want[0][0] and int(res.logits[1, 4].argmax()) == want[1][0]
    assert float(res.logits[1, 5:].abs().max()) == 0.0


def test_trace_runner_replays_steps(tmp_path):
    from safetensors.torch import save_file
    s = shape_odd()
    w = W.make_kazolorn_weights(s, seed=40)
    mdir = tmp_path / "model"
    mdir.mkdir()
    save_file(w, str(mdir / "model.safetensors"))
    (mdir / "config.json").write_text(json.dumps(s.to_config()))
    a, b = toks(9, s.vocab_size, 41), toks(4, s.vocab_size, 42)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:8], "want": [0, 7]}, {"id": "b", "tokens": b[:3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[8:], "want": [0]}, {"id": "b", "tokens": b[3:], "want": [0]}], "end": ["a", "b"]},
             {"step": 2, "entries": [{"id": "c", "tokens": b, "want": [3]}], "end": ["c"]}]
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "32"], input="\n".join(json.dumps(x) for x in steps) + "\n", capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np
    wa, wb = O.forward(s, w, a), O.forward(s, w, b)
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4")).view(2, -1)
    g1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4")).view(2, -1)
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4")).view(1, -1)
    assert rel(g0, wa[[0, 7]]) < 5e-6 and rel(g1, torch.stack([wa[8], wb[3]])) < 5e-6 and rel(g2, wb[3:4]) < 5e-6
