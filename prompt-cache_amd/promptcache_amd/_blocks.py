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
ACT_NONE, ACT_SILU, ACT_SIGMOID, ACT_RELU2, ACT_SOFTPLUS, ACT_SOFTCAP, ACT_RELU, ACT_GELU_TANH, ACT_LOGSIGMOID, ACT_SCALE = range(10)
NORM_NONE, NORM_RMS, NORM_DYT = 0, 1, 2
SCORE_SIGMOID, SCORE_SOFTMAX = 0, 1
ABI_VERSION = 4
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
                ("split_n", _i32), ("y2", _vp), ("row_off2", _vp), ("head_dim2", _i32), ("head_stride2", _i64),
                ("split_n3", _i32), ("y3", _vp), ("row_off3", _vp), ("col_stride3", _i64),
                ("act", _i32), ("act_split", _i32), ("act2", _i32), ("act_param", _f32), ("bias2", _vp)]


class AttnTalkArgs(C.Structure):
    """``pcb_attn_talk_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("q", _vp), ("ldq", _i64), ("tiles", _vp), ("n_tiles", _i32),
                ("cache", _vp), ("slot_stride", _i64), ("head_stride", _i64),
                ("H", _i32), ("Hkv", _i32), ("head_dim", _i32), ("scale", _f32), ("window", _i32), ("max_kv_len", _i32),
                ("slopes", _vp), ("talk", _vp), ("sink", _i32),
                ("scratch", _vp), ("scratch_floats", _i64), ("out", _vp), ("ldo", _i64),
                ("tiles64", _vp), ("n_tiles64", _i32), ("max_tile_rows", _i32)]


class HyperNormArgs(C.Structure):
    """``pcb_hyper_norm_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("streams", _vp), ("stream_stride", _i64), ("n_streams", _i32),
                ("y", _vp), ("mix", _vp), ("out_w", _vp), ("in_w", _vp),
                ("norm", _i32), ("gain", _vp), ("bias", _vp), ("alpha", _vp), ("eps", _f32),
                ("out", _vp), ("x_out", _vp), ("rows", _vp), ("n_rows", _i32), ("width", _i32)]


class AttnSoftmaxArgs(C.Structure):
    """``pcb_attn_softmax_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("q", _vp), ("ldq", _i64), ("q_scale", _vp), ("tiles", _vp), ("n_tiles", _i32),
                ("kcache", _vp), ("vcache", _vp), ("slot_stride", _i64), ("head_stride", _i64), ("row_stride", _i64),
                ("v_slot_stride", _i64), ("v_head_stride", _i64), ("v_stride", _i64), ("v_cols", _i32),
                ("H", _i32), ("Hkv", _i32), ("dim", _i32), ("vdim", _i32), ("scale", _f32), ("window", _i32),
                ("gate", _vp), ("ldg", _i64), ("out", _vp), ("ldo", _i64), ("n_splits", _i32), ("part", _vp),
                ("block", _i32), ("sink", _vp), ("gate_per_head", _i32), ("head_rows", _i32), ("keep_first", _i32)]


class DecayAttnArgs(C.Structure):
    """``pcb_decay_attn_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("q", _vp), ("k", _vp), ("v", _vp), ("ldq", _i64), ("ldk", _i64), ("ldv", _i64),
                ("reqs", _vp), ("n_reqs", _i32), ("state", _vp), ("slot_stride", _i64), ("decay", _vp),
                ("H", _i32), ("dim", _i32), ("vdim", _i32), ("out", _vp), ("ldo", _i64)]


class SelectiveScanArgs(C.Structure):
    """``pcb_selective_scan_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("x", _vp), ("ldx", _i64), ("dt", _vp), ("lddt", _i64), ("B", _vp), ("Cm", _vp), ("ldbc", _i64),
                ("z", _vp), ("ldz", _i64), ("A", _vp), ("D", _vp), ("reqs", _vp), ("n_reqs", _i32),
                ("state", _vp), ("slot_stride", _i64), ("C", _i32), ("N", _i32), ("out", _vp), ("ldo", _i64), ("dt_sum", _vp)]


class PostNormArgs(C.Structure):
    """``pcb_post_norm_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("x", _vp), ("y", _vp), ("gate", _vp), ("ldg", _i64), ("post_gain", _vp), ("gain", _vp),
                ("out", _vp), ("x_out", _vp), ("rows", _vp), ("eps", _f32), ("n_rows", _i32), ("width", _i32),
                ("y_scale", _f32), ("layer_norm", _i32), ("bias", _vp)]


class HeadPrepSeg(C.Structure):
    """``pcb_head_prep_seg`` (field for field)."""
    _fields_ = [("src", _vp), ("ld_src", _i64), ("src_head_stride", _i64), ("heads", _i32), ("head_dim", _i32), ("norm", _i32), ("gain", _vp),
                ("blend", _vp), ("other", _vp), ("ld_other", _i64), ("keep", _vp), ("ld_keep", _i64),
                ("rot_off", _i32), ("rot_dims", _i32), ("dst", _vp), ("ld_dst", _i64), ("row_off", _vp),
                ("head_stride", _i64), ("col_stride", _i64)]


class HeadPrepArgs(C.Structure):
    """``pcb_head_prep_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32), ("n_rows", _i32), ("n_segs", _i32),
                ("pos", _vp), ("freqs", _vp), ("rot_mag", _f32), ("eps", _f32), ("seg", HeadPrepSeg * 4)]


class MlstmArgs(C.Structure):
    """``pcb_mlstm_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("q", _vp), ("k", _vp), ("v", _vp), ("gi", _vp), ("gf", _vp),
                ("ldq", _i64), ("ldk", _i64), ("ldv", _i64), ("ldgi", _i64), ("ldgf", _i64),
                ("reqs", _vp), ("n_reqs", _i32), ("state", _vp), ("slot_stride", _i64),
                ("H", _i32), ("dim", _i32), ("vdim", _i32), ("q_scale", _f32), ("gate_cap", _f32), ("out", _vp), ("ldo", _i64),
                ("from_nothing", _i32), ("log_f_sum", _vp), ("end_slots", _vp), ("end_state", _vp), ("end_slot_stride", _i64)]


class GlaArgs(C.Structure):
    """``pcb_gla_args`` (field for field)."""
    _fields_ = [("struct_bytes", C.c_uint32), ("dtype", _i32),
                ("q", _vp), ("k", _vp), ("v", _vp), ("ldq", _i64), ("ldk", _i64), ("ldv", _i64),
                ("ld", _vp), ("ldld", _i64), ("dcols", _i32), ("ld_coef", _vp), ("v_scale", _vp), ("ldvs", _i64),
                ("reqs", _vp), ("n_reqs", _i32), ("state", _vp), ("slot_stride", _i64),
                ("H", _i32), ("Hk", _i32), ("dim", _i32), ("vdim", _i32), ("q_scale", _f32), ("out", _vp), ("ldo", _i64), ("ld_sum", _vp)]


# name -> (restype, argtypes); mirrors include/promptcache_blocks.h one to one
SIGNATURES = {
    "pcb_version": (C.c_int, []),
    "pcb_last_error_string": (C.c_char_p, []),
    "pcb_embed_rows": (C.c_int, [_vp, _i32, _vp, _vp, _i32, _i32, _i32, _vp]),
    "pcb_embed_scaled_rows": (C.c_int, [_vp, _i32, _vp, _f32, _vp, _i32, _i32, _i32, _vp]),
    "pcb_mix_norm": (C.c_int, [C.POINTER(MixNormArgs), _vp]),
    "pcb_linear": (C.c_int, [C.POINTER(LinearArgs), _vp]),
    "pcb_polynorm": (C.c_int, [_vp, _vp, _vp, _i32, _f32, _i32, _i32, _vp]),
    "pcb_router_topk": (C.c_int, [_vp, _i32, _i32, _i32, _vp, _vp, _vp]),
    "pcb_moe_plan": (C.c_int, [_vp, _vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp]),
    "pcb_moe_combine": (C.c_int, [_vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "pcb_attn_talk_band": (C.c_int32, [_i32, _i32]),
    "pcb_attn_talk": (C.c_int, [C.POINTER(AttnTalkArgs), _vp]),
    "pcb_embed_pos_rows": (C.c_int, [_vp, _vp, _i32, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
    "pcb_hyper_norm": (C.c_int, [C.POINTER(HyperNormArgs), _vp]),
    "pcb_gated_norm": (C.c_int, [_vp, _i64, _vp, _vp, _i64, _vp, _i64, _i32, _f32, _i32, _i32, _i32, _i32, _vp, _i64, _vp, _i32, _vp]),
    "pcb_router_select": (C.c_int, [_vp, _i32, _i32, _i32, _i32, _vp, _i32, _i32, _i32, _vp, _vp, _vp]),
    "pcb_moe_mix": (C.c_int, [_vp, _vp, _vp, _vp, _i32, _i32, _vp, _i32, _i32, _i32, _vp]),
    "pcb_attn_softmax": (C.c_int, [C.POINTER(AttnSoftmaxArgs), _vp]),
    "pcb_decay_attn": (C.c_int, [C.POINTER(DecayAttnArgs), _vp]),
    "pcb_causal_conv": (C.c_int, [_vp, _i64, _vp, _vp, _i32, _i32, _vp, _vp, _i64, _vp, _i64, _i32, _i32, _i32, _vp]),
    "pcb_conv_state_update": (C.c_int, [_vp, _i64, _i32, _vp, _i32, _vp, _i64, _i32, _i32, _vp]),
    "pcb_selective_scan": (C.c_int, [C.POINTER(SelectiveScanArgs), _vp]),
    "pcb_state_chain": (C.c_int, [_vp, _vp, _vp, _i64, _vp, _i32, _vp, _vp, _i32, _i32, _vp]),
    "pcb_post_norm": (C.c_int, [C.POINTER(PostNormArgs), _vp]),
    "pcb_head_prep": (C.c_int, [C.POINTER(HeadPrepArgs), _vp]),
    "pcb_mlstm": (C.c_int, [C.POINTER(MlstmArgs), _vp]),
    "pcb_mlstm_chain": (C.c_int, [_vp, _vp, _vp, _vp, _i64, _vp, _i32, _i32, _i32, _i32, _vp]),
    "pcb_gla": (C.c_int, [C.POINTER(GlaArgs), _vp]),
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
    if lib.pcb_version() != ABI_VERSION:
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


def embed_scaled_rows(table: torch.Tensor, ids: torch.Tensor, scale: float, out: torch.Tensor) -> None:
    """``out`` fp32 [rows, width] = scale * table[ids]."""
    n, width = out.shape
    _want(ids, torch.int32, "embed_scaled_rows ids"); _want(out, torch.float32, "embed_scaled_rows out")
    assert ids.numel() >= n and table.shape[1] == width and table.is_contiguous()
    check(load().pcb_embed_scaled_rows(_p(table), _code(table), _p(ids), float(scale), _p(out), n, width, table.shape[0], _stream()),
          "pcb_embed_scaled_rows")


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
           split_n: int = 0, y2=None, row_off2=None, head_dim2: int = 0, head_stride2: int = 0, split_n3: int = 0, y3=None,
           row_off3=None, col_stride3: int = 0, act: int = ACT_NONE,
           act_split: int = 0, act2: int = ACT_NONE, act_param: float = 0.0, ldy: Optional[int] = None, bias2=None,
           ldx: Optional[int] = None) -> None:
    """``w``: [N, K], or [groups, N, K] with ``group_off``.  ``x``: [rows, K] of the weights' element type.  ``act`` (and ``act2``
    from column ``act_split`` on): the element-wise function of a plain store.  ``ldy``: row stride of ``y`` when it is a
    column block of a wider matrix."""
    code = _code(w)
    assert x.dtype == w.dtype and (x.is_contiguous() or ldx is not None) and w.is_contiguous() and x.is_cuda and w.is_cuda
    N, K = w.shape[-2], w.shape[-1]
    assert x.shape[-1] == K or (ldx is not None and ldx >= K)
    if n_groups:
        assert w.dim() == 3 and w.shape[0] == n_groups and group_off is not None and group_off.numel() == n_groups + 1
        _want(group_off, torch.int32, "linear group_off")
    else:
        assert w.dim() == 2
    if w2 is not None:
        assert w2.shape == w.shape and w2.dtype == w.dtype and w2.is_contiguous()
    for b_ in (bias, bias2):
        if b_ is not None:
            assert b_.dtype == w.dtype and b_.numel() == N and b_.is_cuda
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
        cols = split_n if split_n else (split_n3 if split_n3 else N)
        assert (y.shape[-1] == cols or (ldy is not None and ldy >= cols)) and (row_dst is not None or y.shape[0] >= M)
    if split_n:
        _want(row_off2, torch.int64, "linear row_off2")
        assert y2 is not None and y2.dtype == w.dtype and row_off2.numel() >= M and head_dim2 > 0
    if split_n3:
        _want(row_off3, torch.int64, "linear row_off3")
        assert y3 is not None and y3.dtype == w.dtype and row_off3.numel() >= M and col_stride3 > 0 and split_n3 > split_n
    a = LinearArgs(C.sizeof(LinearArgs), code, epilogue, _p(x), K if ldx is None else ldx, _p(row_src), _p(row_scale), _p(w), _p(w2), K, _p(bias),
                   M, N, K, _p(group_off), n_groups, N * K if n_groups else 0, _p(y), y.shape[-1] if ldy is None else ldy, out_f32,
                   _p(row_dst), _p(base), N, _p(col_scale), split_n, _p(y2), _p(row_off2), head_dim2, head_stride2,
                   split_n3, _p(y3), _p(row_off3), col_stride3, int(act), int(act_split), int(act2), float(act_param), _p(bias2))
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


# ---- blocks of designs with several residual streams, gated / recurrent mixers and group-limited routers ----------------------
def embed_pos_rows(table: torch.Tensor, pos_table: Optional[torch.Tensor], ids: torch.Tensor, positions: Optional[torch.Tensor],
                   out: torch.Tensor) -> None:
    """``out`` fp32 [streams, rows, width]: every stream receives table[ids] + pos_table[positions]."""
    S, n, width = out.shape
    _want(ids, torch.int32, "embed_pos_rows ids"); _want(out, torch.float32, "embed_pos_rows out")
    assert ids.numel() >= n and table.shape[1] == width and table.is_contiguous()
    if pos_table is not None:
        _want(positions, torch.int32, "embed_pos_rows positions")
        assert pos_table.dtype == table.dtype and pos_table.shape[1] == width and pos_table.is_contiguous() and positions.numel() >= n
    check(load().pcb_embed_pos_rows(_p(table), _p(pos_table), _code(table), _p(ids), _p(positions), _p(out), n * width, S, n, width,
                                    table.shape[0], pos_table.shape[0] if pos_table is not None else 0, _stream()), "pcb_embed_pos_rows")


def hyper_norm(streams: torch.Tensor, *, y=None, mix=None, out_w=None, in_w=None, norm: int = NORM_NONE, gain=None, bias=None,
               alpha=None, eps: float = 1e-6, out=None, x_out=None, rows=None, n_rows: Optional[int] = None) -> None:
    """``streams`` fp32 [S, T, W].  With ``y`` (fp32 [T, W]) the streams are rewritten through ``mix`` [S, S] / ``out_w`` [S]; with
    ``out`` (E) or ``x_out`` (fp32) the ``in_w``-weighted sum of the streams is normed and stored (rows ``rows`` only, if given)."""
    _want(streams, torch.float32, "hyper_norm streams")
    S, T, W = streams.shape
    n = (rows.numel() if rows is not None else T) if n_rows is None else n_rows
    for t, nm in ((y, "y"), (mix, "mix"), (out_w, "out_w"), (in_w, "in_w"), (gain, "gain"), (bias, "bias"), (alpha, "alpha"), (x_out, "x_out")):
        _want(t, torch.float32, "hyper_norm " + nm)
    if y is not None:
        assert y.shape[-1] == W and y.shape[0] >= (T if rows is not None else n) and mix.numel() == S * S and out_w.numel() == S
    assert in_w is None or in_w.numel() == S
    assert rows is not None or n <= T
    if out is not None:
        assert out.is_contiguous() and out.shape[-1] == W and out.numel() >= n * W
        if norm != NORM_NONE:
            assert gain is not None and gain.numel() == W and (bias is None or bias.numel() == W)
    if x_out is not None:
        assert x_out.numel() >= n * W
    if rows is not None:
        _want(rows, torch.int32, "hyper_norm rows")
    a = HyperNormArgs(C.sizeof(HyperNormArgs), _code(out) if out is not None else BF16, _p(streams), T * W, S, _p(y), _p(mix), _p(out_w),
                      _p(in_w), int(norm), _p(gain), _p(bias), _p(alpha), float(eps), _p(out), _p(x_out), _p(rows), n, W)
    check(load().pcb_hyper_norm(C.byref(a), _stream()), "pcb_hyper_norm")


def gated_norm(x: torch.Tensor, gain: Optional[torch.Tensor], gate: Optional[torch.Tensor], ldg: int, out: torch.Tensor, eps: float,
               n_rows: int, group: int = 0, gate_first: bool = False, skip: Optional[torch.Tensor] = None, lds: int = 0,
               skip_w: Optional[torch.Tensor] = None, skip_group: int = 0) -> None:
    """``x`` fp32 [rows, cols]; ``gate`` E, a column block (row stride ``ldg``) of a wider matrix; ``out`` E [rows, cols].
    ``group`` > 0: a norm per run of that many columns (per head) instead of one over the row.  ``skip`` (E rows of stride
    ``lds``) with ``skip_w`` (fp32, one weight per ``skip_group`` columns): x + skip_w * skip stands for x.  ``gate_first``: the
    gate is applied before the norm."""
    _want(x, torch.float32, "gated_norm x"); _want(gain, torch.float32, "gated_norm gain"); _want(skip_w, torch.float32, "gated_norm skip_w")
    cols = x.shape[-1]
    assert out.is_contiguous() and out.shape[-1] == cols and x.shape[0] >= n_rows and out.shape[0] >= n_rows
    assert gain is None or gain.numel() == cols
    if gate is not None:
        assert gate.dtype == out.dtype and gate.is_cuda and ldg >= cols
    if skip is not None:
        assert skip.dtype == out.dtype and skip.is_cuda and lds >= cols and skip_group > 0 and cols % skip_group == 0
        assert skip_w is not None and skip_w.numel() == cols // skip_group
    assert group == 0 or cols % group == 0
    check(load().pcb_gated_norm(_p(x), cols, _p(gain), _p(gate), ldg, _p(out), cols, _code(out), float(eps), n_rows, cols, int(group),
                                int(gate_first), _p(skip), int(lds), _p(skip_w), int(skip_group), _stream()), "pcb_gated_norm")


def router_select(logits: torch.Tensor, top: int, expert: torch.Tensor, weight: torch.Tensor, n_rows: int, *, score_fn: int,
                  correction: Optional[torch.Tensor] = None, groups: int = 1, groups_keep: int = 1, renorm: bool = False) -> None:
    _want(logits, torch.float32, "router_select logits"); _want(expert, torch.int32, "router_select expert")
    _want(weight, torch.float32, "router_select weight"); _want(correction, torch.float32, "router_select correction")
    n_out = logits.shape[-1]
    assert logits.shape[0] >= n_rows and expert.numel() >= n_rows * top and weight.numel() >= n_rows * top
    assert correction is None or correction.numel() == n_out
    check(load().pcb_router_select(_p(logits), n_rows, n_out, top, int(score_fn), _p(correction), groups, groups_keep, int(renorm),
                                   _p(expert), _p(weight), _stream()), "pcb_router_select")


def moe_mix(pair_out: torch.Tensor, expert: torch.Tensor, weight: torch.Tensor, h: torch.Tensor, n_real: int, y: torch.Tensor,
            n_rows: int, top: int) -> None:
    _want(pair_out, torch.float32, "moe_mix pair_out"); _want(expert, torch.int32, "moe_mix expert")
    _want(weight, torch.float32, "moe_mix weight"); _want(y, torch.float32, "moe_mix y")
    W = y.shape[-1]
    assert pair_out.shape[-1] == W and pair_out.shape[0] >= n_rows * top and h.shape[-1] == W and h.shape[0] >= n_rows and h.is_contiguous()
    assert y.shape[0] >= n_rows and expert.numel() >= n_rows * top and weight.numel() >= n_rows * top
    check(load().pcb_moe_mix(_p(pair_out), _p(expert), _p(weight), _p(h), _code(h), n_real, _p(y), n_rows, W, top, _stream()), "pcb_moe_mix")


def attn_softmax(q: torch.Tensor, ldq: int, tiles: torch.Tensor, n_tiles: int, kcache: torch.Tensor, k_strides, vcache: torch.Tensor,
                 v_offset: int, v_strides, v_cols: bool, H: int, Hkv: int, dim: int, vdim: int, scale: float, out: torch.Tensor, *,
                 q_scale: Optional[torch.Tensor] = None, window: int = 0, gate: Optional[torch.Tensor] = None, ldg: int = 0,
                 n_splits: int = 1, part: Optional[torch.Tensor] = None, block: int = 0, sink: Optional[torch.Tensor] = None,
                 gate_per_head: bool = False, head_rows: bool = False, keep_first: int = 0) -> None:
    """``q``: E rows (row stride ``ldq``, head h at column h * dim); ``kcache`` with ``k_strides`` = (slot, head, row) strides in
    elements; the values start ``v_offset`` elements into ``vcache`` (which may be the same plane) with ``v_strides`` = (slot, head,
    row) strides, or (slot, head, column) strides when ``v_cols`` (a cache kept column by column, columns readable in multiples of
    32 keys); ``gate``: E rows of stride ``ldg``; ``out`` E [rows, H * vdim].  ``n_splits`` > 1: each (tile, head) runs as that many
    workgroups over runs of the keys, merged by a second launch; ``part``: fp32 scratch of ``attn_softmax_part(rows, H, n_splits,
    vdim)`` floats.  ``block`` > 0: a key is seen only inside the query's own block of that many positions; ``sink`` fp32 [H]: one
    more exp(sink[h]) in the denominator; ``gate_per_head``: the gate has one column per head; ``head_rows``: every tile has one row and
    there is one key head -- a workgroup then serves 16 heads of the row at once; ``keep_first`` > 0: behind a window the keys at
    positions below it stay visible."""
    _want(tiles, torch.int32, "attn_softmax tiles"); _want(q_scale, torch.float32, "attn_softmax q_scale")
    _want(sink, torch.float32, "attn_softmax sink")
    assert sink is None or sink.numel() == H
    assert q.dtype == kcache.dtype == vcache.dtype == out.dtype and out.is_contiguous() and kcache.is_cuda and vcache.is_cuda and q.is_cuda
    assert tiles.numel() >= 4 * n_tiles and out.shape[-1] == H * vdim and ldq >= H * dim
    assert gate is None or (gate.dtype == q.dtype and ldg >= (H if gate_per_head else H * vdim))
    es = vcache.element_size()
    a = AttnSoftmaxArgs(C.sizeof(AttnSoftmaxArgs), _code(q), _p(q), ldq, _p(q_scale), _p(tiles), n_tiles, _p(kcache),
                        vcache.data_ptr() + v_offset * es, int(k_strides[0]), int(k_strides[1]), int(k_strides[2]), int(v_strides[0]),
                        int(v_strides[1]), int(v_strides[2]), int(v_cols), H, Hkv, dim, vdim, float(scale), int(window), _p(gate), ldg,
                        _p(out), out.shape[-1], int(n_splits), _p(part), int(block), _p(sink), int(gate_per_head), int(head_rows), int(keep_first))
    if n_splits > 1:
        _want(part, torch.float32, "attn_softmax part")
        assert part.numel() >= attn_softmax_part(out.shape[0], H, n_splits, vdim)
    check(load().pcb_attn_softmax(C.byref(a), _stream()), "pcb_attn_softmax")


def attn_softmax_part(rows: int, H: int, n_splits: int, vdim: int) -> int:
    return rows * H * n_splits * (vdim + 2)


def decay_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, ld: int, reqs: torch.Tensor, n_reqs: int, state: torch.Tensor,
               decay: torch.Tensor, H: int, dim: int, vdim: int, out: Optional[torch.Tensor]) -> None:
    """``q``, ``k``, ``v``: column blocks (row stride ``ld``) of one E matrix; ``state`` fp32 [slots, H, dim, vdim]; ``out`` fp32
    [rows, H * vdim], or None: only the states move."""
    _want(reqs, torch.int32, "decay_attn reqs"); _want(state, torch.float32, "decay_attn state"); _want(decay, torch.float32, "decay_attn decay")
    _want(out, torch.float32, "decay_attn out")
    assert q.dtype == k.dtype == v.dtype and q.is_cuda and reqs.numel() >= 4 * n_reqs and decay.numel() == H
    assert tuple(state.shape[1:]) == (H, dim, vdim) and (out is None or out.shape[-1] == H * vdim)
    a = DecayAttnArgs(C.sizeof(DecayAttnArgs), _code(q), _p(q), _p(k), _p(v), ld, ld, ld, _p(reqs), n_reqs, _p(state), H * dim * vdim,
                      _p(decay), H, dim, vdim, _p(out), H * vdim)
    check(load().pcb_decay_attn(C.byref(a), _stream()), "pcb_decay_attn")


def causal_conv(x: torch.Tensor, ldx: int, w: torch.Tensor, bias: Optional[torch.Tensor], silu: bool, row_meta: torch.Tensor,
                state: torch.Tensor, out: torch.Tensor, n_rows: int) -> None:
    """``x``: E rows (stride ``ldx``) of C channels; ``w`` E [C, taps]; ``state`` E [slots, taps - 1, C]; ``out`` E [rows, C]."""
    C_, taps = w.shape
    _want(row_meta, torch.int32, "causal_conv row_meta")
    assert x.dtype == w.dtype == out.dtype == state.dtype and out.is_contiguous() and out.shape[-1] == C_ and w.is_contiguous()
    assert row_meta.numel() >= 4 * n_rows and tuple(state.shape[1:]) == (taps - 1, C_) and (bias is None or bias.numel() == C_)
    check(load().pcb_causal_conv(_p(x), ldx, _p(w), _p(bias), _code(x), int(silu), _p(row_meta), _p(state), (taps - 1) * C_, _p(out),
                                 C_, n_rows, C_, taps, _stream()), "pcb_causal_conv")


def conv_state_update(x: torch.Tensor, ldx: int, reqs: torch.Tensor, n_reqs: int, state: torch.Tensor) -> None:
    _want(reqs, torch.int32, "conv_state_update reqs")
    taps, C_ = state.shape[1] + 1, state.shape[2]
    assert x.dtype == state.dtype and reqs.numel() >= 4 * n_reqs and state.is_contiguous()
    check(load().pcb_conv_state_update(_p(x), ldx, _code(x), _p(reqs), n_reqs, _p(state), (taps - 1) * C_, C_, taps, _stream()),
          "pcb_conv_state_update")


def selective_scan(x: torch.Tensor, dt: torch.Tensor, bc: torch.Tensor, z: Optional[torch.Tensor], ldz: int, A: torch.Tensor,
                   D: Optional[torch.Tensor], reqs: torch.Tensor, n_reqs: int, state: torch.Tensor, out: Optional[torch.Tensor],
                   dt_sum: Optional[torch.Tensor] = None) -> None:
    """``x`` E [rows, C]; ``dt`` fp32 [rows, C]; ``bc`` fp32 [rows, 2 N] = B | C; ``z`` E rows of stride ``ldz``; ``A`` fp32 [C, N];
    ``state`` fp32 [slots, C, N]; ``out`` E [rows, C], or None: only the states move; ``dt_sum`` fp32 [n_reqs, C]: each request's
    sum of dt."""
    C_, N = A.shape
    for t, nm in ((dt, "dt"), (bc, "bc"), (A, "A"), (D, "D"), (state, "state")):
        _want(t, torch.float32, "selective_scan " + nm)
    _want(reqs, torch.int32, "selective_scan reqs")
    assert x.is_contiguous() and x.shape[-1] == C_ == dt.shape[-1]
    assert out is None or (x.dtype == out.dtype and out.is_contiguous() and out.shape[-1] == C_)
    assert bc.shape[-1] == 2 * N and tuple(state.shape[1:]) == (C_, N) and reqs.numel() >= 4 * n_reqs
    assert z is None or (z.dtype == x.dtype and ldz >= C_)
    _want(dt_sum, torch.float32, "selective_scan dt_sum")
    assert dt_sum is None or dt_sum.numel() >= n_reqs * C_
    a = SelectiveScanArgs(C.sizeof(SelectiveScanArgs), _code(x), _p(x), C_, _p(dt), C_, _p(bc), bc.data_ptr() + 4 * N, 2 * N, _p(z), ldz,
                          _p(A), _p(D), _p(reqs), n_reqs, _p(state), C_ * N, C_, N, _p(out), C_, _p(dt_sum))
    check(load().pcb_selective_scan(C.byref(a), _stream()), "pcb_selective_scan")


def state_chain(local: torch.Tensor, start: torch.Tensor, state: torch.Tensor, chains: torch.Tensor, n_chains: int, coef: torch.Tensor,
                x: torch.Tensor, group: int) -> None:
    """``local``, ``start`` fp32 [segments, elems]; ``state`` fp32 [slots, ...elems]; ``chains`` int32 {slot, first position, first
    segment, segments} x n_chains; ``coef`` fp32 [elems]; ``x`` fp32 [segments, elems / group]."""
    for t, nm in ((local, "local"), (start, "start"), (state, "state"), (coef, "coef"), (x, "x")):
        _want(t, torch.float32, "state_chain " + nm)
    _want(chains, torch.int32, "state_chain chains")
    elems = coef.numel()
    n_seg = local.shape[0]
    assert local.numel() == n_seg * elems == start.numel() and state[0].numel() == elems and chains.numel() >= 4 * n_chains
    assert elems % group == 0 and x.numel() >= n_seg * (elems // group)
    check(load().pcb_state_chain(_p(local), _p(start), _p(state), elems, _p(chains), n_chains, _p(coef), _p(x), elems, group, _stream()),
          "pcb_state_chain")


# ---- sublayers between two norms, per-head preparation, matrix memories ----------------------------------------------------------
def post_norm(x: torch.Tensor, *, y=None, gate=None, ldg: int = 0, post_gain=None, gain=None, out=None, x_out=None, rows=None,
              eps: float = 1e-6, n_rows: Optional[int] = None, y_scale: float = 1.0, layer_norm: bool = False, bias=None) -> None:
    """``x`` fp32 [T, W] (the residual).  With ``y`` (fp32 [T, W]): x += norm(y * gate) * post_gain (``gate`` E rows of stride
    ``ldg``; without ``post_gain`` the gated y is added as it is).  With ``out`` (E): out = norm(x) * gain, for the rows ``rows``
    only if given (then x itself is not rewritten); ``x_out`` fp32 receives those rows of x.  ``y_scale``: the factor on what is
    added to x; ``layer_norm``: out = (x - mean) / sqrt(variance + eps) * gain + bias instead of the RMS form."""
    _want(x, torch.float32, "post_norm x"); _want(bias, torch.float32, "post_norm bias")
    assert bias is None or (layer_norm and bias.numel() == x.shape[-1])
    T, W = x.shape
    n = (rows.numel() if rows is not None else T) if n_rows is None else n_rows
    for t, nm in ((y, "y"), (post_gain, "post_gain"), (gain, "gain"), (x_out, "x_out")):
        _want(t, torch.float32, "post_norm " + nm)
    assert rows is not None or n <= T
    if y is not None:
        assert y.shape[-1] == W and y.shape[0] >= (T if rows is not None else n)
    if gate is not None:
        assert y is not None and gate.is_cuda and ldg >= W and gate.dtype in DTYPES
    code = _code(out) if out is not None else (_code(gate) if gate is not None else BF16)
    if out is not None:
        assert out.is_contiguous() and out.shape[-1] == W and out.numel() >= n * W and gain is not None and gain.numel() == W
        assert gate is None or gate.dtype == out.dtype
    assert post_gain is None or post_gain.numel() == W
    if x_out is not None:
        assert x_out.numel() >= n * W
    if rows is not None:
        _want(rows, torch.int32, "post_norm rows")
    a = PostNormArgs(C.sizeof(PostNormArgs), code, _p(x), _p(y), _p(gate), ldg, _p(post_gain), _p(gain), _p(out), _p(x_out), _p(rows),
                     float(eps), n, W, float(y_scale), int(layer_norm), _p(bias))
    check(load().pcb_post_norm(C.byref(a), _stream()), "pcb_post_norm")


def head_seg(src: torch.Tensor, ld_src: int, heads: int, head_dim: int, dst: torch.Tensor, *, norm: bool = False, gain=None, blend=None,
             other=None, keep=None, rot_off: int = 0, rot_dims: int = 0, ld_dst: int = 0, row_off=None, head_stride: Optional[int] = None,
             col_stride: int = 1, dst_offset: int = 0, src_head_stride: Optional[int] = None) -> HeadPrepSeg:
    """One segment of ``head_prep``: ``src`` E, a column block (row stride ``ld_src``) whose first ``heads * head_dim`` columns are
    the heads; ``dst`` E: a row matrix (``ld_dst``, heads ``head_stride`` apart, starting ``dst_offset`` elements in) or a cache
    (``row_off`` int64 per row; ``col_stride`` > 1 for one kept column by column).  ``other`` / ``keep``: fp32 [rows, heads *
    head_dim]."""
    for t, nm in ((gain, "gain"), (blend, "blend"), (other, "other"), (keep, "keep")):
        _want(t, torch.float32, "head_prep " + nm)
    _want(row_off, torch.int64, "head_prep row_off")
    shs = head_dim if src_head_stride is None else src_head_stride
    assert src.dtype == dst.dtype and src.is_cuda and dst.is_cuda and ld_src >= (heads - 1) * shs + head_dim
    assert gain is None or gain.numel() == head_dim
    assert blend is None or (other is not None and other.shape[-1] == heads * head_dim)
    assert keep is None or keep.shape[-1] == heads * head_dim
    assert row_off is not None or ld_dst > 0
    return HeadPrepSeg(_p(src), ld_src, shs, heads, head_dim, int(norm), _p(gain), _p(blend), _p(other), heads * head_dim, _p(keep),
                       heads * head_dim, rot_off, rot_dims, dst.data_ptr() + dst_offset * dst.element_size(), ld_dst, _p(row_off),
                       head_dim if head_stride is None else head_stride, col_stride)


def head_prep(segs, n_rows: int, dtype, *, pos: Optional[torch.Tensor] = None, freqs: Optional[torch.Tensor] = None, rot_mag: float = 1.0,
              eps: float = 1e-6) -> None:
    """``segs``: one to four ``head_seg`` records; ``pos`` int32 [rows]; ``freqs`` float64 [rot_dims / 2]."""
    _want(pos, torch.int32, "head_prep pos"); _want(freqs, torch.float64, "head_prep freqs")
    assert 1 <= len(segs) <= 4
    rot = {s.rot_dims for s in segs if s.rot_dims}
    assert len(rot) <= 1 and (not rot or (pos is not None and freqs is not None and pos.numel() >= n_rows and 2 * freqs.numel() == rot.pop()))
    a = HeadPrepArgs(C.sizeof(HeadPrepArgs), DTYPES[dtype], n_rows, len(segs), _p(pos), _p(freqs), float(rot_mag), float(eps))
    for i, sg in enumerate(segs):
        a.seg[i] = sg
    check(load().pcb_head_prep(C.byref(a), _stream()), "pcb_head_prep")


def mlstm_state_floats(H: int, dim: int, vdim: int) -> int:
    """fp32 elements of a slot's state: per head S [dim][vdim], then n [dim], then the running maximum."""
    return H * (dim * vdim + dim + 1)


def mlstm(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gi: torch.Tensor, gf: torch.Tensor, ld: int, reqs: torch.Tensor, n_reqs: int,
          state: torch.Tensor, H: int, dim: int, vdim: int, q_scale: float, gate_cap: float, out: Optional[torch.Tensor],
          from_nothing: bool = False, log_f_sum: Optional[torch.Tensor] = None, end_slots: Optional[torch.Tensor] = None,
          end_state: Optional[torch.Tensor] = None) -> None:
    """``q``, ``k``, ``v``, ``gi``, ``gf``: column blocks (row stride ``ld``) of one E matrix; ``state`` fp32 [slots,
    mlstm_state_floats]; ``out`` fp32 [rows, H * vdim], or None: only the states move.  ``from_nothing``: every request is a
    segment that starts from an empty memory; ``log_f_sum`` fp32 [n_reqs, H] receives its sum of log forget gates.  ``end_slots``
    int32 [n_reqs]: where >= 0, the request's last state goes to that slot of ``end_state`` instead of its own record."""
    _want(reqs, torch.int32, "mlstm reqs"); _want(state, torch.float32, "mlstm state"); _want(out, torch.float32, "mlstm out")
    _want(log_f_sum, torch.float32, "mlstm log_f_sum")
    assert log_f_sum is None or log_f_sum.numel() >= n_reqs * H
    _want(end_slots, torch.int32, "mlstm end_slots"); _want(end_state, torch.float32, "mlstm end_state")
    assert end_slots is None or (end_slots.numel() >= n_reqs and end_state is not None and end_state[0].numel() == state[0].numel())
    assert q.dtype == k.dtype == v.dtype == gi.dtype == gf.dtype and q.is_cuda and reqs.numel() >= 4 * n_reqs
    assert state[0].numel() == mlstm_state_floats(H, dim, vdim) and (out is None or out.shape[-1] == H * vdim)
    a = MlstmArgs(C.sizeof(MlstmArgs), _code(q), _p(q), _p(k), _p(v), _p(gi), _p(gf), ld, ld, ld, ld, ld, _p(reqs), n_reqs, _p(state),
                  state[0].numel(), H, dim, vdim, float(q_scale), float(gate_cap), _p(out), H * vdim, int(from_nothing), _p(log_f_sum),
                  _p(end_slots), _p(end_state), end_state[0].numel() if end_state is not None else 0)
    check(load().pcb_mlstm(C.byref(a), _stream()), "pcb_mlstm")


def mlstm_chain(local: torch.Tensor, log_f_sum: torch.Tensor, start: torch.Tensor, state: torch.Tensor, chains: torch.Tensor, n_chains: int,
                H: int, dim: int, vdim: int) -> None:
    """``local``, ``start`` fp32 [segments, mlstm_state_floats]; ``log_f_sum`` fp32 [segments, H]; ``state`` fp32 [slots,
    mlstm_state_floats]; ``chains`` int32 {slot, first position, first segment, segments} x n_chains."""
    for t, nm in ((local, "local"), (log_f_sum, "log_f_sum"), (start, "start"), (state, "state")):
        _want(t, torch.float32, "mlstm_chain " + nm)
    _want(chains, torch.int32, "mlstm_chain chains")
    rec = mlstm_state_floats(H, dim, vdim)
    assert local.shape[-1] == rec == start.shape[-1] == state[0].numel() and local.shape[0] == start.shape[0]
    assert log_f_sum.numel() >= local.shape[0] * H and chains.numel() >= 4 * n_chains
    check(load().pcb_mlstm_chain(_p(local), _p(log_f_sum), _p(start), _p(state), rec, _p(chains), n_chains, H, dim, vdim, _stream()),
          "pcb_mlstm_chain")


def gla(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, ld: torch.Tensor, lds_: tuple, dcols: int, reqs: torch.Tensor, n_reqs: int,
        state: torch.Tensor, H: int, Hk: int, dim: int, vdim: int, q_scale: float, out: Optional[torch.Tensor], *,
        ld_coef: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None, ldvs: int = 0,
        ld_sum: Optional[torch.Tensor] = None) -> None:
    """Linear attention with a decay per token: ``q``, ``k`` (``Hk`` heads), ``v`` (``H`` heads) E rows with row strides
    ``lds_`` = (ldq, ldk, ldv, ldld); ``ld`` fp32 rows of log decays, ``dcols`` = ``dim`` (one per key channel) or 1 (one per head),
    times ``ld_coef`` [H] when given; ``v_scale`` fp32 rows (stride ``ldvs``) of one step size per head; ``state`` fp32
    [slots, H, dim, vdim]; ``out`` fp32 [rows, H * vdim] or None (states only; ``ld_sum`` fp32 [n_reqs, H * dcols] then receives
    the sums of the log decays)."""
    _want(reqs, torch.int32, "gla reqs"); _want(state, torch.float32, "gla state"); _want(out, torch.float32, "gla out")
    _want(ld_coef, torch.float32, "gla ld_coef"); _want(ld_sum, torch.float32, "gla ld_sum")
    assert q.dtype == k.dtype == v.dtype and q.is_cuda and ld.dtype == torch.float32 and ld.is_cuda
    assert reqs.numel() >= 4 * n_reqs and state.shape[-3:] == (H, dim, vdim) and dcols in (1, dim)
    assert out is None or out.shape[-1] == H * vdim
    assert v_scale is None or (v_scale.dtype == torch.float32 and ldvs >= H)
    assert ld_coef is None or ld_coef.numel() == H
    assert ld_sum is None or ld_sum.numel() >= n_reqs * H * dcols
    ldq, ldk, ldv, ldld = (int(x) for x in lds_)
    a = GlaArgs(C.sizeof(GlaArgs), _code(q), _p(q), _p(k), _p(v), ldq, ldk, ldv, _p(ld), ldld, int(dcols), _p(ld_coef), _p(v_scale),
                int(ldvs), _p(reqs), n_reqs, _p(state), H * dim * vdim, H, Hk, dim, vdim, float(q_scale), _p(out),
                H * vdim if out is not None else 0, _p(ld_sum))
    check(load().pcb_gla(C.byref(a), _stream()), "pcb_gla")
