"""TEST INFRASTRUCTURE - not part of the product.

ctypes front end of the CPU oracle (``fmha_oracle.c``).  It works on CPU torch tensors and is meant to be
imported by the tests, the smoke check and the benchmark's CPU-baseline leg only.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfmha_oracle.so")

FP8, FP16, BF16 = 1, 3, 4
NO_MASK, MASK_TOP_LEFT, MASK_BOTTOM_RIGHT, MASK_GENERIC = 0, 1, 2, 3
ROPE_NONE, ROPE_INTERLEAVED, ROPE_HALF_ROTATED = 0, 1, 2
KV_BATCH, KV_GROUP, KV_BLOCK_TABLE, KV_PAGE_LIST = 0, 1, 2, 3

_i32p = ctypes.c_void_p


class _Problem(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32),
        ("batch", ctypes.c_int32), ("hq", ctypes.c_int32), ("hk", ctypes.c_int32),
        ("d", ctypes.c_int32), ("dv", ctypes.c_int32),
        ("seqstart_q", _i32p),
        ("sq", ctypes.c_int32),
        ("kv_mode", ctypes.c_int32),
        ("sk", ctypes.c_int32),
        ("seqstart_k", _i32p),
        ("seqlen_k", _i32p),
        ("block_table", _i32p),
        ("block_table_stride", ctypes.c_int32),
        ("page_size", ctypes.c_int32),
        ("kv_indptr", _i32p),
        ("kv_page_indices", _i32p),
        ("kv_last_page_lens", _i32p),
        ("cache_batch_idx", _i32p),
        ("scale", ctypes.c_float),
        ("mask_type", ctypes.c_int32),
        ("window_left", ctypes.c_int64), ("window_right", ctypes.c_int64),
        ("bias_type", ctypes.c_int32),
        ("bias", ctypes.c_void_p),
        ("bias_batch_stride", ctypes.c_int64), ("bias_head_stride", ctypes.c_int64), ("bias_row_stride", ctypes.c_int64),
        ("logits_soft_cap", ctypes.c_float),
        ("kv_dtype", ctypes.c_int32), ("k_descale", ctypes.c_float), ("v_descale", ctypes.c_float),
        ("o_scale", ctypes.c_float),
    ]


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.fck_orc_visible.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_int, ctypes.c_int]
        _lib.fck_orc_fmha_fwd.argtypes = [ctypes.c_void_p] * 6
        _lib.fck_orc_fmha_splitkv.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        _lib.fck_orc_splitkv_combine.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int] * 6 + [ctypes.c_float]
        _lib.fck_orc_rope.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                      ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        _lib.fck_orc_appendkv.argtypes = ([ctypes.c_void_p] * 9 + [ctypes.c_int] * 3 + [ctypes.c_void_p, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_void_p, ctypes.c_int64] + [ctypes.c_int] * 7
                                         + [ctypes.c_float] * 2)
        _lib.fck_orc_f32_to_fp8.restype = ctypes.c_uint8
        _lib.fck_orc_f32_to_fp8.argtypes = [ctypes.c_float]
        _lib.fck_orc_gather_paged.argtypes = [ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 5 + [ctypes.c_void_p]
    return _lib


def fp8_to_f32(byte: int) -> float:
    lib().fck_orc_fp8_to_f32.restype = ctypes.c_float
    lib().fck_orc_fp8_to_f32.argtypes = [ctypes.c_uint8]
    return lib().fck_orc_fp8_to_f32(byte)


def num_threads():
    return lib().fck_orc_num_threads()


def dtype_id(t):
    if t == torch.bfloat16:
        return BF16
    if t == torch.float16:
        return FP16
    if t == torch.float8_e4m3fn:   # the all-fp8 roles: Q, K, V, P and O
        return FP8
    raise TypeError(f"oracle supports fp16 / bf16 / fp8 (e4m3) only, got {t}")


def _ptr(t):
    if t is None:
        return None
    assert t.device.type == "cpu" and t.is_contiguous(), "oracle takes contiguous CPU tensors"
    return ctypes.c_void_p(t.data_ptr())


def _i32(t):
    if t is None:
        return None
    assert t.dtype == torch.int32
    return _ptr(t)


def _problem(q, k, v, *, seqstart_q=None, seqstart_k=None, seqlen_k=None, block_table=None, page_size=0,
             kv_indptr=None, kv_page_indices=None, kv_last_page_lens=None, cache_batch_idx=None, scale=None,
             mask_type=NO_MASK, window=(-1, -1), batch=None, bias=None, alibi_slopes=None, logits_soft_cap=0.0,
             k_descale=1.0, v_descale=1.0, o_scale=1.0):
    """bias: data dtype, [1|B, 1|Hq, sq, sk] (batch mode) or [1|Hq, total_q, max_sk] (group mode), last dim contiguous;
    alibi_slopes: fp32 [Hq] or [B, Hq]; logits_soft_cap > 0: s = cap * tanh(scale * qk / cap)."""
    p = _Problem()
    p.dtype = dtype_id(q.dtype)
    p.hq, p.d = q.shape[-2], q.shape[-1]
    p.hk, p.dv = k.shape[-2], v.shape[-1]
    if seqstart_q is not None:
        p.batch = seqstart_q.numel() - 1
        p.sq = 0
    else:
        p.batch, p.sq = q.shape[0], q.shape[1]
    if batch is not None:
        p.batch = batch
    if kv_indptr is not None:
        p.kv_mode = KV_PAGE_LIST
        p.page_size = k.shape[1]
    elif block_table is not None:
        p.kv_mode = KV_BLOCK_TABLE
        p.page_size = k.shape[1]
        p.block_table_stride = block_table.shape[1]
    elif seqstart_k is not None:
        p.kv_mode = KV_GROUP
    else:
        p.kv_mode = KV_BATCH
        p.sk = k.shape[1]
    if page_size:
        assert page_size == p.page_size
    p.seqstart_q = _i32(seqstart_q)
    p.seqstart_k = _i32(seqstart_k)
    p.seqlen_k = _i32(seqlen_k)
    p.block_table = _i32(block_table)
    p.kv_indptr = _i32(kv_indptr)
    p.kv_page_indices = _i32(kv_page_indices)
    p.kv_last_page_lens = _i32(kv_last_page_lens)
    p.cache_batch_idx = _i32(cache_batch_idx)
    p.scale = float(scale if scale is not None else q.shape[-1] ** -0.5)
    p.mask_type = int(mask_type)
    p.window_left, p.window_right = int(window[0]), int(window[1])
    p.logits_soft_cap = float(logits_soft_cap)
    if k.dtype == torch.float8_e4m3fn:   # fp8 K/V with static scales
        assert v.dtype == torch.float8_e4m3fn
        p.kv_dtype, p.k_descale, p.v_descale = FP8, float(k_descale), float(v_descale)
    if q.dtype == torch.float8_e4m3fn:   # fp8 Q, P and O as well: O = saturate(o_scale * o)
        assert k.dtype == torch.float8_e4m3fn, "fp8 queries come with an fp8 K/V"
        p.o_scale = float(o_scale)
    assert bias is None or alibi_slopes is None, "one bias kind at a time"
    if bias is not None:
        want = torch.float32 if q.dtype == torch.float8_e4m3fn else q.dtype   # BiasDataType of the fp8 roles is float
        assert bias.dtype == want and bias.device.type == "cpu" and bias.stride(-1) == 1
        group = seqstart_q is not None
        assert bias.dim() == (3 if group else 4)
        p.bias_type = 1
        p.bias = bias.data_ptr()
        p.bias_row_stride = bias.stride(-2)
        p.bias_head_stride = bias.stride(-3) if bias.shape[-3] > 1 else 0
        p.bias_batch_stride = 0 if group or bias.shape[0] == 1 else bias.stride(0)
        p._keep = bias
    elif alibi_slopes is not None:
        assert alibi_slopes.dtype == torch.float32 and alibi_slopes.is_contiguous() and alibi_slopes.shape[-1] == p.hq
        p.bias_type = 2
        p.bias = alibi_slopes.data_ptr()
        p.bias_batch_stride = p.hq if alibi_slopes.dim() == 2 else 0
        p._keep = alibi_slopes
    return p


def fmha_fwd(q, k, v, return_lse=False, **kw):
    """Attention over any of the supported K/V addressings; returns O (and fp32 LSE)."""
    p = _problem(q, k, v, **kw)
    o = torch.empty(*q.shape[:-1], v.shape[-1], dtype=q.dtype)
    lse = None
    if return_lse:
        if kw.get("seqstart_q") is not None:
            lse = torch.empty(p.hq, q.shape[0], dtype=torch.float32)
        else:
            lse = torch.empty(p.batch, p.hq, p.sq, dtype=torch.float32)
    rc = lib().fck_orc_fmha_fwd(ctypes.byref(p), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse))
    assert rc == 0, rc
    return (o, lse) if return_lse else o


def fmha_splitkv(q, k, v, num_splits, **kw):
    """Per-split partial results: (o_acc fp32 [Bs,Hq,ns,Sq,Dv], lse_acc fp32 [Bs,Hq,ns,Sq])."""
    p = _problem(q, k, v, **kw)
    if kw.get("seqstart_q") is not None:
        bs, sq = 1, q.shape[0]
    else:
        bs, sq = p.batch, p.sq
    o_acc = torch.zeros(bs, p.hq, num_splits, sq, p.dv, dtype=torch.float32)
    lse_acc = torch.full((bs, p.hq, num_splits, sq), float("-inf"), dtype=torch.float32)
    rc = lib().fck_orc_fmha_splitkv(ctypes.byref(p), _ptr(q), _ptr(k), _ptr(v), num_splits, _ptr(o_acc), _ptr(lse_acc))
    assert rc == 0, rc
    return o_acc, lse_acc


def splitkv_combine(lse_acc, o_acc, dtype, seqstart_q=None, batch=None, return_lse=False, o_scale=1.0):
    bs, hq, ns, sq, dv = o_acc.shape
    if seqstart_q is not None:
        o = torch.empty(sq, hq, dv, dtype=dtype)
        nb = seqstart_q.numel() - 1
    else:
        o = torch.empty(bs, sq, hq, dv, dtype=dtype)
        nb = bs
    lse = torch.empty(bs, hq, sq, dtype=torch.float32) if return_lse else None
    rc = lib().fck_orc_splitkv_combine(_ptr(lse_acc), _ptr(o_acc), _ptr(o), _ptr(lse), _i32(seqstart_q), nb, sq, hq, dv,
                                       ns, dtype_id(dtype), float(o_scale))
    assert rc == 0, rc
    return (o, lse) if return_lse else o


def rope(x, pos, cos, sin, rope_mode=ROPE_HALF_ROTATED):
    """x [rows, heads, d] -> rotated copy; row r uses table row pos[r]."""
    out = x.clone().contiguous()
    rows, heads, d = out.shape
    rc = lib().fck_orc_rope(_ptr(out), rows, heads, d, _i32(pos), _ptr(cos), _ptr(sin), cos.shape[1] * 2, rope_mode,
                            dtype_id(x.dtype))
    assert rc == 0, rc
    return out


def f32_to_fp8(x: float) -> int:
    return lib().fck_orc_f32_to_fp8(x)


def appendkv(q, k_cache, v_cache, knew, vnew, seqlen_k, cu_seqlens_knew, cos=None, sin=None,
             rope_mode=ROPE_NONE, has_mask=True, block_table=None, cache_batch_idx=None, k_descale=1.0, v_descale=1.0):
    """In place on q, k_cache, v_cache (CPU tensors).  torch.float8_e4m3fn caches are written quantised with the static
    scales k_descale / v_descale."""
    kv_dtype = FP8 if k_cache.dtype == torch.float8_e4m3fn else 0
    batch = seqlen_k.numel()
    hk, d = knew.shape[-2], knew.shape[-1]
    dv = vnew.shape[-1]
    hq = q.shape[-2] if q is not None else 0
    rotary_dim = cos.shape[1] * 2 if cos is not None else 0
    if block_table is not None:
        page, stride, cbs = k_cache.shape[1], block_table.shape[1], 0
    else:
        page, stride, cbs = 0, 0, k_cache.shape[1]
    rc = lib().fck_orc_appendkv(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(knew), _ptr(vnew), _i32(seqlen_k),
                                _i32(cu_seqlens_knew), _ptr(cos), _ptr(sin), rotary_dim, rope_mode, int(has_mask),
                                _i32(block_table), stride, page, _i32(cache_batch_idx), cbs, batch, hq, hk, d, dv,
                                dtype_id(knew.dtype), kv_dtype, float(k_descale), float(v_descale))
    assert rc == 0, rc


def gather_paged(cache, pages, n):
    """First n logical rows of one sequence from a paged cache [num_pages, P, Hk, D]."""
    _, page, hk, d = cache.shape
    out = torch.empty(n, hk, d, dtype=cache.dtype)
    rc = lib().fck_orc_gather_paged(_ptr(cache), _i32(pages), page, n, hk, d, cache.element_size(), _ptr(out))
    assert rc == 0, rc
    return out


def visible(mask_type, window, sq, sk, i, j):
    return bool(lib().fck_orc_visible(mask_type, window[0], window[1], sq, sk, i, j))
