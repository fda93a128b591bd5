"""ctypes binding of ``libpromptcache_blocks.so`` (C-ABI declared in ``include/promptcache_blocks.h``): the bf16 / fp32
building-block kernels.  No fallback: a missing library is built once from ``csrc/pb_*.hip`` (a fresh checkout's first use),
and a failing call raises ``RuntimeError`` with the library's own message.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _buildlib

_vp, _i32, _i64, _f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_float
_lib: Optional[C.CDLL] = None

BF16, F32 = 0, 1
EPI_STORE, EPI_SILU_MUL, EPI_SCALE_ADD = 0, 1, 2
DTYPES = {torch.bfloat16: BF16, torch.float32: F32}


class MixNormArgs(C.Structure):
    """``pcb_mix_norm_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("hist", _vp), ("hist_stride", _i64), ("coef", _vp), ("n_terms", _i32),
                ("x_out", _vp), ("rows", _vp), ("gain1", _vp), ("out1", _vp), ("gain2", _vp), ("out2", _vp),
                ("eps", _f32), ("n_rows", _i32), ("width", _i32)]


class LinearArgs(C.Structure):
    """``pcb_linear_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32), ("epilogue", _i32),
                ("x", _vp), ("ldx", _i64), ("row_src", _vp), ("row_scale", _vp),
                ("w", _vp), ("w2", _vp), ("ldw", _i64), ("bias", _vp),
                ("M", _i32), ("N", _i32), ("K", _i32),
                ("group_off", _vp), ("n_groups", _i32), ("w_group_stride", _i64),
                ("y", _vp), ("ldy", _i64), ("out_f32", _i32), ("row_dst", _vp),
                ("base", _vp), ("ldbase", _i64), ("col_scale", _vp),
                ("split_n", _i32), ("y2", _vp), ("row_off2", _vp), ("head_dim2", _i32), ("head_stride2", _i64)]


class AttnTalkArgs(C.Structure):
    """``pcb_attn_talk_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("q", _vp), ("ldq", _i64), ("tiles", _vp), ("n_tiles", _i32),
                ("cache", _vp), ("slot_stride", _i64), ("head_stride", _i64),
                ("H", _i32), ("Hkv", _i32), ("head_dim", _i32), ("scale", _f32), ("window", _i32), ("max_kv_len", _i32),
                ("slopes", _vp), ("talk", _vp), ("sink", _i32),
                ("scratch", _vp), ("scratch_floats", _i64), ("out", _vp), ("ldo", _i64),
                ("tiles64", _vp), ("n_tiles64", _i32), ("max_tile_rows", _i32)]


# name -> (restype, argtypes); mirrors include/promptcache_blocks.h one to one
SIGNATURES = {
    "pcb_version": (C.c_int, []),
    "pcb_last_error_string": (C.c_char_p, []),
    "pcb_embed_rows": (C.c_int, [_vp, _i32, _vp, _vp, _i32, _i32, _i32, _vp]),
    "pcb_mix_norm": (C.c_int, [C.POINTER(MixNormArgs), _vp]),
    "pcb_linear": (C.c_int, [C.POINTER(LinearArgs), _vp]),
    "pcb_polynorm": (C.c_int, [_vp, _vp, _vp, _i32, _f32, _i32, _i32, _vp]),
    "pcb_router_topk": (C.c_int, [_vp, _i32, _i32, _i32, _vp, _vp, _vp]),
    "pcb_moe_plan": (C.c_int, [_vp, _vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp]),
    "pcb_moe_combine": (C.c_int, [_vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "pcb_attn_talk_band": (C.c_int32, [_i32, _i32]),
    "pcb_attn_talk": (C.c_int, [C.POINTER(AttnTalkArgs), _vp]),
}


def lib_path() -> str:
    return _buildlib.lib_path("blocks")


def load(build_missing: bool = True) -> C.CDLL:
    """Load the library (once); a missing one is compiled first unless ``build_missing`` is off."""
    global _lib
    if _lib is not None:
        return _lib
    import os
    if not os.path.exists(lib_path()):
        if not build_missing:
            raise RuntimeError(f"{lib_path()} not found: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
        _buildlib.build("blocks")
    lib = C.CDLL(lib_path())
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    if lib.pcb_version() != 1:
        raise RuntimeError("libpromptcache_blocks.so: ABI version mismatch (rebuild it)")
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().pcb_last_error_string()
        raise RuntimeError(f"{what} failed (code {rc}): {msg.decode() if msg else ''}")


def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _code(t: torch.Tensor) -> int:
    try:
        return DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"element type {t.dtype} is not one of bfloat16 / float32") from None


def _want(t: Optional[torch.Tensor], dtype, what: str) -> None:
    if t is not None and (t.dtype != dtype or not t.is_cuda or not t.is_contiguous()):
        raise TypeError(f"{what}: need a contiguous {dtype} device tensor, got {t.dtype} on {t.device} (contiguous={t.is_contiguous()})")


# ---- wrappers: shapes are checked here, on the host, before the library sees a pointer ---------------------------------------
def embed_rows(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    n, width = out.shape
    _want(ids, torch.int32, "embed_rows ids"); _want(out, torch.float32, "embed_rows out")
    assert ids.numel() == n and table.shape[1] == width and table.is_contiguous()
    check(load().pcb_embed_rows(_p(table), _code(table), _p(ids), _p(out), n, width, table.shape[0], _stream()), "pcb_embed_rows")


def mix_norm(hist: torch.Tensor, n_streams: int, coef: Optional[torch.Tensor], gain1: Optional[torch.Tensor],
             out1: Optional[torch.Tensor], gain2: Optional[torch.Tensor] = None, out2: Optional[torch.Tensor] = None,
             x_out: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None, eps: float = 1e-6,
             n_rows: Optional[int] = None) -> None:
    """``hist`` fp32 [streams, T, W]; ``coef`` fp32 [n_streams] or None (then stream 0 is taken as it is)."""
    _want(hist, torch.float32, "mix_norm hist")
    S, T, W = hist.shape
    n = (rows.numel() if rows is not None else T) if n_rows is None else n_rows
    some = out1 if out1 is not None else out2
    assert coef is None or (coef.numel() >= n_streams and n_streams <= S)
    for g, o in ((gain1, out1), (gain2, out2)):
        if o is not None:
            _want(g, torch.float32, "mix_norm gain")
            assert g.numel() == W and o.is_contiguous() and o.shape[-1] == W and o.numel() >= n * W
    if x_out is not None:
        _want(x_out, torch.float32, "mix_norm x_out")
        assert x_out.numel() >= n * W
    if rows is not None:
        _want(rows, torch.int32, "mix_norm rows")
    a = MixNormArgs(C.sizeof(MixNormArgs), _code(some) if some is not None else BF16, _p(hist), T * W, _p(coef),
                    n_streams if coef is not None else 0, _p(x_out), _p(rows), _p(gain1), _p(out1), _p(gain2), _p(out2),
                    float(eps), n, W)
    check(load().pcb_mix_norm(C.byref(a), _stream()), "pcb_mix_norm")


def linear(x: torch.Tensor, w: torch.Tensor, y: torch.Tensor, *, M: int, epilogue: int = EPI_STORE, bias=None, w2=None,
           row_src=None, row_scale=None, group_off=None, n_groups: int = 0, row_dst=None, base=None, col_scale=None,
           split_n: int = 0, y2=None, row_off2=None, head_dim2: int = 0, head_stride2: int = 0) -> None:
    """``w``: [N, K], or [groups, N, K] with ``group_off``.  ``x``: [rows, K] of the weights' element type."""
    code = _code(w)
    assert x.dtype == w.dtype and x.is_contiguous() and w.is_contiguous() and x.is_cuda and w.is_cuda
    N, K = w.shape[-2], w.shape[-1]
    assert x.shape[-1] == K
    if n_groups:
        assert w.dim() == 3 and w.shape[0] == n_groups and group_off is not None and group_off.numel() == n_groups + 1
        _want(group_off, torch.int32, "linear group_off")
    else:
        assert w.dim() == 2
    if w2 is not None:
        assert w2.shape == w.shape and w2.dtype == w.dtype and w2.is_contiguous()
    if bias is not None:
        assert bias.dtype == w.dtype and bias.numel() == N
    for t, nm in ((row_src, "row_src"), (row_dst, "row_dst")):
        if t is not None:
            _want(t, torch.int32, "linear " + nm)
            assert t.numel() >= M
    if row_scale is not None:
        _want(row_scale, torch.float32, "linear row_scale")
        assert row_scale.numel() >= M
    if row_src is None:
        assert x.shape[0] >= M
    out_f32 = int(y.dtype == torch.float32 and (code == BF16 or epilogue == EPI_SCALE_ADD))
    if epilogue == EPI_SCALE_ADD:
        _want(y, torch.float32, "linear y"); _want(col_scale, torch.float32, "linear col_scale")
        assert col_scale.numel() == N and y.shape[-1] == N and y.shape[0] >= M
        if base is not None:
            _want(base, torch.float32, "linear base")
            assert base.shape[-1] == N and base.shape[0] >= M
    else:
        assert y.is_contiguous() and (y.dtype == w.dtype or y.dtype == torch.float32)
        cols = split_n if split_n else N
        assert y.shape[-1] == cols and (row_dst is not None or y.shape[0] >= M)
    if split_n:
        _want(row_off2, torch.int64, "linear row_off2")
        assert y2 is not None and y2.dtype == w.dtype and row_off2.numel() >= M and head_dim2 > 0
    a = LinearArgs(C.sizeof(LinearArgs), code, epilogue, _p(x), K, _p(row_src), _p(row_scale), _p(w), _p(w2), K, _p(bias),
                   M, N, K, _p(group_off), n_groups, N * K if n_groups else 0, _p(y), y.shape[-1], out_f32, _p(row_dst),
                   _p(base), N, _p(col_scale), split_n, _p(y2), _p(row_off2), head_dim2, head_stride2)
    check(load().pcb_linear(C.byref(a), _stream()), "pcb_linear")


def polynorm(z: torch.Tensor, coef: torch.Tensor, out: torch.Tensor, eps: float, n_rows: int) -> None:
    _want(z, torch.float32, "polynorm z"); _want(coef, torch.float32, "polynorm coef")
    ff = z.shape[-1]
    assert coef.numel() == 4 and out.shape[-1] == ff and out.is_contiguous() and z.shape[0] >= n_rows and out.shape[0] >= n_rows
    check(load().pcb_polynorm(_p(z), _p(coef), _p(out), _code(out), float(eps), n_rows, ff, _stream()), "pcb_polynorm")


def router_topk(logits: torch.Tensor, top: int, expert: torch.Tensor, weight: torch.Tensor, n_rows: int) -> None:
    _want(logits, torch.float32, "router_topk logits"); _want(expert, torch.int32, "router_topk expert")
    _want(weight, torch.float32, "router_topk weight")
    E = logits.shape[-1]
    assert logits.shape[0] >= n_rows and expert.numel() >= n_rows * top and weight.numel() >= n_rows * top
    check(load().pcb_router_topk(_p(logits), n_rows, E, top, _p(expert), _p(weight), _stream()), "pcb_router_topk")


def moe_plan(expert: torch.Tensor, weight: torch.Tensor, n_pairs: int, top: int, n_experts: int, group_off: torch.Tensor,
             row_src: torch.Tensor, row_dst: torch.Tensor, row_scale: torch.Tensor) -> None:
    for t in (expert, group_off, row_src, row_dst):
        _want(t, torch.int32, "moe_plan")
    _want(weight, torch.float32, "moe_plan weight"); _want(row_scale, torch.float32, "moe_plan row_scale")
    assert group_off.numel() >= n_experts + 1 and min(row_src.numel(), row_dst.numel(), row_scale.numel()) >= n_pairs
    check(load().pcb_moe_plan(_p(expert), _p(weight), n_pairs, top, n_experts, _p(group_off), _p(row_src), _p(row_dst),
                              _p(row_scale), _stream()), "pcb_moe_plan")


def moe_combine(pair_out: torch.Tensor, col_scale: torch.Tensor, y: torch.Tensor, n_rows: int, top: int) -> None:
    _want(pair_out, torch.float32, "moe_combine pair_out"); _want(col_scale, torch.float32, "moe_combine col_scale")
    _want(y, torch.float32, "moe_combine y")
    W = y.shape[-1]
    assert pair_out.shape[-1] == W and pair_out.shape[0] >= n_rows * top and col_scale.numel() == W and y.shape[0] >= n_rows
    check(load().pcb_moe_combine(_p(pair_out), _p(col_scale), _p(y), n_rows, W, top, _stream()), "pcb_moe_combine")


def attn_talk_band(window: int, max_kv_len: int) -> int:
    return int(load().pcb_attn_talk_band(window, max_kv_len))


def attn_talk(q: torch.Tensor, tiles: torch.Tensor, n_tiles: int, cache: torch.Tensor, slot_stride: int, head_stride: int,
              H: int, Hkv: int, head_dim: int, scale: float, window: int, max_kv_len: int, slopes, talk, sink: bool,
              scratch: torch.Tensor, out: torch.Tensor, tiles64: Optional[torch.Tensor] = None, n_tiles64: int = 0,
              max_tile_rows: int = 0) -> None:
    _want(tiles, torch.int32, "attn_talk tiles"); _want(scratch, torch.float32, "attn_talk scratch")
    assert q.dtype == cache.dtype == out.dtype and q.is_contiguous() and out.is_contiguous() and cache.is_cuda
    assert tiles.numel() >= 4 * n_tiles and q.shape[-1] == H * head_dim and out.shape[-1] == H * head_dim
    assert min(q.shape[0], out.shape[0]) * 1 >= 1
    if slopes is not None:
        _want(slopes, torch.float32, "attn_talk slopes"); assert slopes.numel() == H
    if talk is not None:
        _want(talk, torch.float32, "attn_talk talk"); assert talk.numel() == H * H
    a = AttnTalkArgs(C.sizeof(AttnTalkArgs), _code(q), _p(q), q.shape[-1], _p(tiles), n_tiles, _p(cache), slot_stride,
                     head_stride, H, Hkv, head_dim, float(scale), int(window), int(max_kv_len), _p(slopes), _p(talk), int(sink),
                     _p(scratch), scratch.numel(), _p(out), out.shape[-1], _p(tiles64), n_tiles64 if tiles64 is not None else 0,
                     int(max_tile_rows))
    if tiles64 is not None:
        _want(tiles64, torch.int32, "attn_talk tiles64")
        assert tiles64.numel() >= 4 * n_tiles64 > 0
    check(load().pcb_attn_talk(C.byref(a), _stream()), "pcb_attn_talk")
