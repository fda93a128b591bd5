"""CPU-side checks of the Dibizen integration: configuration reader, tensor naming, checkpoint directories, per-slot states of the
slot arena, the blocks library's argument structures, and properties of the plain oracle itself (each mechanism made visible by
inputs built for it)."""
import ctypes
import json
import math
import os
import subprocess

import pytest
import torch

from oracle import dibizen_oracle as O
from promptcache_amd.model import weights as W
from promptcache_amd.model.config import DibizenLayer, DibizenShape, architecture_of
from promptcache_amd.model.kv_arena import SlotArena

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F = torch.float64


def moe(l, ff, experts, identity, top, groups=1, keep=1):
    l.ff, l.experts, l.identity, l.top, l.groups, l.groups_keep = ff, experts, identity, top, groups, keep
    return l


def mixed_shape():
    return DibizenShape(vocab_size=90, hidden_size=40, norm_eps=1e-5, streams=3, max_positions=64, logit_softcap=9.0, layers=[
        moe(DibizenLayer("attention", heads=4, kv_heads=2, dim=12, vdim=8, scale=0.3, qt_coef=0.4, qt_every=5), 16, 6, 2, 3, 4, 2),
        moe(DibizenLayer("mamba1", inner=24, state=5, conv=3, dt_rank=3), 12, 3, 0, 1),
        DibizenLayer("lightning", heads=2, kv_heads=2, dim=8, vdim=12, decay=(0.5, 0.97)),
        moe(DibizenLayer("attention", heads=4, kv_heads=2, dim=12, vdim=8, scale=0.2, kv_from=0), 8, 2, 2, 2, 2, 1),
    ])


# ---- configuration and tensors -------------------------------------------------------------------------------------------------
def test_config_round_trip_and_every_branch():
    s = mixed_shape()
    c = s.to_config()
    assert c["architecture"] == "Dibizen" and c["layers"][2]["mlp"] is None and c["layers"][3]["mixer"]["kv_from"] == 0
    assert "q_temp" not in c["layers"][3]["mixer"] and c["layers"][0]["mixer"]["q_temp"] == {"coef": 0.4, "every": 5}
    s2 = DibizenShape.from_config(json.loads(json.dumps(c)))
    assert s2.layers == s.layers and (s2.streams, s2.max_positions, s2.logit_softcap, s2.norm_eps) == (3, 64, 9.0, 1e-5)
    # what a configuration leaves out does not exist: no groups, no identity experts, no temperature, no cap
    c["layers"][0]["mlp"]["router"] = {"experts": 6, "top": 2}
    del c["layers"][0]["mixer"]["q_temp"]
    del c["logit_softcap"]
    s3 = DibizenShape.from_config(c)
    assert (s3.layers[0].groups, s3.layers[0].groups_keep, s3.layers[0].identity, s3.layers[0].qt_every) == (1, 1, 0, 0)
    assert s3.logit_softcap == 0.0


@pytest.mark.parametrize("edit,msg", [
    (lambda c: c["layers"][0].update(type="conv"), "unknown mixer type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "do not divide"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=16), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.5]), "decays"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=3), "groups"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "top"),
    (lambda c: c.update(architecture="Other"), "not Dibizen"),
])
def test_config_errors_are_loud(edit, msg):
    c = mixed_shape().to_config()
    edit(c)
    with pytest.raises(ValueError, match=msg):
        DibizenShape.from_config(c)


def test_weight_names_follow_the_layers():
    s = mixed_shape()
    n = W.dibizen_weight_shapes(s)
    assert n["pos"] == (64, 40) and n["l0.norm1.alpha"] == () and n["l0.hc1.mix"] == (3, 3) and n["l0.hc2.in"] == (3,)
    assert n["l0.mix.k"] == (24, 40) and n["l0.mix.v"] == (16, 40) and n["l0.mix.g"] == (32, 40) and n["l0.mix.o"] == (40, 32)
    assert "l3.mix.k" not in n and "l3.mix.v" not in n and n["l3.mix.q"] == (48, 40)            # the borrowing layer has no k / v
    assert n["l1.mix.in"] == (48, 40) and n["l1.mix.conv"] == (24, 3) and n["l1.mix.x"] == (13, 24) and n["l1.mix.dt"] == (24, 3)
    assert n["l2.mix.norm"] == (24,) and n["l2.mix.q"] == (16, 40) and n["l2.mix.v"] == (24, 40)
    assert "l2.norm2" not in n and "l2.hc2.in" not in n and "l2.mlp.router" not in n            # no feed-forward, none of its tensors
    assert n["l0.mlp.router"] == (8, 40) and n["l0.mlp.correction"] == (8,) and "l0.mlp.e5.up" in n and "l0.mlp.e6.up" not in n
    w = W.make_dibizen_weights(s, seed=3)
    assert sorted(w) == sorted(n) and all(tuple(w[k].shape) == tuple(n[k]) and w[k].dtype == torch.bfloat16 for k in n)
    assert all(torch.equal(w[k], v) for k, v in W.make_dibizen_weights(s, seed=3).items())


def test_checkpoint_directory_round_trip(tmp_path):
    from safetensors.torch import save_file
    s = mixed_shape()
    w = W.make_dibizen_weights(s, seed=1)
    save_file(w, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(s.to_config()))
    assert architecture_of(str(tmp_path)) == "dibizen"
    s2 = DibizenShape.from_dir(str(tmp_path))
    got = W.load_dibizen_safetensors(str(tmp_path), s2)
    assert all(torch.equal(got[k], w[k]) for k in w)
    bad = dict(w)
    bad["l1.mix.A_log"] = bad["l1.mix.A_log"][:, :-1].contiguous()
    save_file(bad, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="l1.mix.A_log"):
        W.load_dibizen_safetensors(str(tmp_path), s2)
    del bad["l0.hc2.mix"]
    save_file(bad, str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError, match="l0.hc2.mix"):
        W.load_dibizen_safetensors(str(tmp_path), s2)


# ---- slot arena: states beside the key planes --------------------------------------------------------------------------------------
def test_slot_arena_states_follow_their_slots():
    ar = SlotArena([(2, 6), (0, 0)], 1, 4, "cpu", torch.float32, states=[[], [((3, 2), torch.float32), ((2, 5), torch.bfloat16)]])
    assert ar.planes[1].numel() == 0 and [tuple(t.shape) for t in ar.states[1]] == [(1, 3, 2), (1, 2, 5)] and ar.states[0] == []
    assert ar.state_bytes_per_slot() == 3 * 2 * 4 + 2 * 5 * 2
    a = ar.alloc()
    ar.states[1][0][a] = 7.0
    ar.planes[0][a, :, :3] = 2.0
    ar.lengths[a] = 3
    gen = ar.generation
    b = ar.alloc()                                   # a second slot: every tensor grows, the live slot keeps what it holds
    assert ar.generation > gen and ar.slots >= 2 and b != a
    assert float(ar.states[1][0][a].min()) == 7.0 and float(ar.planes[0][a, :, :3].min()) == 2.0
    assert ar.states[1][1].dtype == torch.bfloat16 and ar.states[1][1].shape[0] == ar.slots
    ar.room_for(a, 40)                               # longer rows only: the states do not move
    keep = ar.states[1][0].data_ptr()
    assert ar.cap >= 43 and ar.states[1][0].data_ptr() == keep and float(ar.states[1][0][a].max()) == 7.0
    ar.free(a)
    assert ar.alloc() == a and ar.lengths[a] == 0   # handed out again; whoever takes it starts at position 0


def test_slot_arena_column_planes_keep_their_columns_when_rows_grow():
    ar = SlotArena([(2, 4)], 1, 5, "cpu", torch.float32, col_dims=[(2, 3)])
    assert ar.cap == 32 and tuple(ar.col_planes[0].shape) == (1, 2, 3, 32) and ar.col_head_stride(0) == 96 and ar.col_slot_stride(0) == 192
    a = ar.alloc()
    ar.col_planes[0][a, :, :, :7] = torch.arange(7.0)
    ar.lengths[a] = 7
    ar.room_for(a, 40)                               # rows grow: every column keeps its first 7 positions
    assert ar.cap == 64 and torch.equal(ar.col_planes[0][a, 1, 2, :7], torch.arange(7.0))
    assert ar.bytes_per_token() == (2 * 4 + 2 * 3) * 4


# ---- the blocks library's argument structures --------------------------------------------------------------------------------------
def test_blocks_struct_layouts_match_the_header(tmp_path):
    from promptcache_amd import _blocks
    structs = (("pcb_hyper_norm_args", _blocks.HyperNormArgs), ("pcb_attn_softmax_args", _blocks.AttnSoftmaxArgs),
               ("pcb_decay_attn_args", _blocks.DecayAttnArgs), ("pcb_selective_scan_args", _blocks.SelectiveScanArgs),
               ("pcb_linear_args", _blocks.LinearArgs))
    body = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{ROOT}/include/promptcache_blocks.h"', 'int main(void) {']
    for st, cls in structs:
        body.append(f'  printf("{st} %zu\\n", sizeof({st}));')
        for f, _ in cls._fields_:
            body.append(f'  printf("{st}.{f} %zu\\n", offsetof({st}, {f}));')
    body += ['  return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(body))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", str(src), "-o", str(exe)])
    got = dict(line.rsplit(" ", 1) for line in subprocess.check_output([str(exe)], text=True).strip().splitlines())
    for st, cls in structs:
        assert int(got[st]) == ctypes.sizeof(cls), st
        for name, _ in cls._fields_:
            assert int(got[f"{st}.{name}"]) == getattr(cls, name).offset, (st, name)


def test_blocks_reject_bad_arguments_on_the_host():
    from promptcache_amd import _blocks
    assert os.path.exists(_blocks.lib_path()), "run __graft_entry__.build() first"
    lb = _blocks.load(build_missing=False)
    assert lb.pcb_router_select(None, 4, 12, 2, 1, None, 5, 2, 1, None, None, None) == -2001 and b"groups" in lb.pcb_last_error_string()
    assert lb.pcb_router_select(None, 4, 12, 7, 1, None, 4, 2, 1, None, None, None) == -2001      # top beyond the kept groups
    assert lb.pcb_causal_conv(None, 8, None, None, 0, 1, None, None, 0, None, 8, 3, 8, 17, None) == -2001
    a = _blocks.HyperNormArgs(ctypes.sizeof(_blocks.HyperNormArgs), 0, None, 0, 9, None, None, None, None, 0, None, None, None, 0.0,
                              None, None, None, 2, 8)
    assert lb.pcb_hyper_norm(ctypes.byref(a), None) == -2001 and b"streams" in lb.pcb_last_error_string()
    a.struct_bytes -= 4
    assert lb.pcb_hyper_norm(ctypes.byref(a), None) == -2001 and b"struct size" in lb.pcb_last_error_string()


# ---- the oracle's own properties ---------------------------------------------------------------------------------------------------
def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F)


def test_oracle_forward_does_not_look_ahead_and_layers_matter():
    s = mixed_shape()
    w = W.make_dibizen_weights(s, seed=5)
    t = torch.randint(0, s.vocab_size, (14,), generator=torch.Generator().manual_seed(1)).tolist()
    full, sums = O.forward(t, w, s, return_layers=True)
    assert torch.allclose(O.forward(t[:9], w, s), full[:9], atol=1e-10)
    assert float(full.abs().max()) < s.logit_softcap and sums.shape == (4, 14, 40)
    for i in range(1, 4):
        assert float((sums[i] - sums[i - 1]).abs().max()) > 1e-3


def test_oracle_one_stream_with_unit_weights_is_the_plain_residual():
    p = {"h.in": torch.ones(1, dtype=F), "h.out": torch.ones(1, dtype=F), "h.mix": torch.ones(1, 1, dtype=F)}
    xs, y = rnd(1, 5, 7, seed=2), rnd(5, 7, seed=3)
    assert torch.equal(O.hyper_read(xs, p, "h."), xs[0]) and torch.allclose(O.hyper_write(xs, y, p, "h.")[0], xs[0] + y)
    # [from, to]: a mix matrix that only feeds stream 0 into stream 1 moves stream 0 there and clears stream 0
    p = {"h.in": torch.tensor([1.0, 0.0], dtype=F), "h.out": torch.zeros(2, dtype=F), "h.mix": torch.tensor([[0.0, 1.0], [0.0, 0.0]], dtype=F)}
    xs = rnd(2, 3, 4, seed=4)
    new = O.hyper_write(xs, torch.zeros(3, 4, dtype=F), p, "h.")
    assert torch.equal(new[1], xs[0]) and float(new[0].abs().max()) == 0.0


def test_oracle_decayed_attention_forgets_at_its_rate_and_carries_its_state():
    n, H, D, Dv = 9, 2, 3, 4
    q, k, v = rnd(n, H, D, seed=1), rnd(n, H, D, seed=2), rnd(n, H, Dv, seed=3)
    out, S = O.decayed_linear_attention(q, k, v, (0.5, 1.0))
    t = 6
    direct = sum((0.5 ** (t - j)) * float(q[t, 0] @ k[j, 0]) * v[j, 0] for j in range(t + 1))
    assert torch.allclose(out[t, 0], direct, atol=1e-12)
    plain = sum(float(q[t, 1] @ k[j, 1]) * v[j, 1] for j in range(t + 1))                       # decay 1: nothing is forgotten
    assert torch.allclose(out[t, 1], plain, atol=1e-12)
    a, Sa = O.decayed_linear_attention(q[:4], k[:4], v[:4], (0.5, 1.0))
    b, Sb = O.decayed_linear_attention(q[4:], k[4:], v[4:], (0.5, 1.0), state=Sa)
    assert torch.allclose(torch.cat([a, b]), out, atol=1e-12) and torch.allclose(Sb, S, atol=1e-12)


def test_oracle_attention_is_causal_grouped_and_tempered():
    m, H, G, D, Dv = 6, 4, 2, 5, 3
    q, k, v = rnd(m, H, D, seed=1), rnd(m, G, D, seed=2), rnd(m, G, Dv, seed=3)
    out = O.causal_softmax_attention(q, k, v, 0.4)
    assert torch.allclose(out[0, 3], v[0, 1], atol=1e-12)                                        # the first position sees itself only
    k2 = k.clone()
    k2[4:] += 1.0
    assert torch.allclose(O.causal_softmax_attention(q, k2, v, 0.4)[:4], out[:4], atol=1e-12)   # later keys change nothing earlier
    assert torch.allclose(O.causal_softmax_attention(q[3:], k, v, 0.4, first_pos=3), out[3:], atol=1e-12)
    lay = DibizenLayer("attention", heads=1, kv_heads=1, dim=2, vdim=2, qt_coef=0.5, qt_every=4)
    f = O.query_temperature(range(9), lay)
    assert float(f[2]) == 1.0 and abs(float(f[3]) - (1 + 0.5 * math.log(2))) < 1e-12 and float(f[6]) == float(f[3])
    assert abs(float(f[7]) - (1 + 0.5 * math.log(3))) < 1e-12
    assert float(O.query_temperature(range(3), DibizenLayer("attention")).min()) == 1.0


def test_oracle_convolution_and_scan_carry_their_state():
    n, C, N, taps = 8, 3, 4, 3
    x, w, b = rnd(n, C, seed=1), rnd(C, taps, seed=2), rnd(C, seed=3)
    y = O.causal_convolution(x, w, b)
    assert torch.allclose(y[0], b + w[:, -1] * x[0], atol=1e-12)                                 # zeros before the start; last tap = now
    assert torch.allclose(y[2], b + w[:, 0] * x[0] + w[:, 1] * x[1] + w[:, 2] * x[2], atol=1e-12)
    assert torch.allclose(O.causal_convolution(x[5:], w, b, before=x[3:5]), y[5:], atol=1e-12)
    dt, Bm, Cm = rnd(n, C, seed=4).abs(), rnd(n, N, seed=5), rnd(n, N, seed=6)
    A, D = -rnd(C, N, seed=7).abs(), rnd(C, seed=8)
    full, S = O.selective_scan(x, dt, Bm, Cm, A, D)
    a, Sa = O.selective_scan(x[:3], dt[:3], Bm[:3], Cm[:3], A, D)
    b2, Sb = O.selective_scan(x[3:], dt[3:], Bm[3:], Cm[3:], A, D, state=Sa)
    assert torch.allclose(torch.cat([a, b2]), full, atol=1e-12) and torch.allclose(Sb, S, atol=1e-12)
    assert torch.allclose(full[0], (dt[0] * x[0]) * float(Bm[0] @ Cm[0]) + D * x[0], atol=1e-12)


def test_oracle_router_groups_correction_and_identity():
    # 8 outputs in 4 groups of 2, two groups kept, top 3.  Scores favour outputs 0, 1 (group 0) and 6 (group 3); the correction
    # lifts output 4 (group 2) above every other choice score, so groups 2 and 0 are kept and group 3 is out, although its output
    # 6 scores higher than output 1.
    logits = torch.log(torch.tensor([[0.35, 0.20, 0.02, 0.02, 0.05, 0.01, 0.33, 0.02]], dtype=F))
    corr = torch.tensor([0, 0, 0, 0, 0.5, 0, 0, 0], dtype=F)
    idx, w = O.choose(logits, corr, 3, 4, 2)
    assert idx.tolist() == [[4, 0, 1]]
    assert torch.allclose(w, torch.tensor([[0.05, 0.35, 0.20]], dtype=F) / 0.60, atol=1e-12)     # the weights leave the correction out
    # negative choice scores still beat the outputs of dropped groups
    idx, _ = O.choose(logits, torch.tensor([0, 0, 0, 0, 0.5, -1.0, 0, 0], dtype=F), 4, 4, 2)
    assert sorted(idx.tolist()[0]) == [0, 1, 4, 5]
    # an identity expert returns its input times its weight
    lay = moe(DibizenLayer("lightning"), 4, 1, 1, 2)
    p = {"m.router": torch.zeros(2, 6, dtype=F), "m.correction": torch.zeros(2, dtype=F), "m.e0.up": rnd(4, 6, seed=1), "m.e0.down": rnd(6, 4, seed=2)}
    h = rnd(3, 6, seed=3)
    want = 0.5 * h + 0.5 * (torch.relu(h @ p["m.e0.up"].T).pow(2) @ p["m.e0.down"].T)
    assert torch.allclose(O.moe_ff(h, p, "m.", lay), want, atol=1e-12)
