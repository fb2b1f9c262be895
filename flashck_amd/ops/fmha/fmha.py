"""Functional FMHA operators: the `flash_ck.ops.fmha` surface FlashCK declares but leaves empty
(flash_ck/utils/utils.py:49-58; tests/pytorch/fmha/test_{fmha_fwd,fmha_fwd_var_len,fmha_fwd_append_kv,
batch_prefill}.py are 0-byte files), backed by the gfx950 kernels through the C ABI.

The wrappers follow flash_ck/ops/norm/layer_norm.py:61-116 for validation (TypeError / ValueError before any
launch).  Unlike that operator there is no PyTorch fallback: a missing library or a rejected call raises.

Tensor conventions (T = torch.float16 | torch.bfloat16, contiguous, on the GPU):
    q, o         [B, sq, Hq, D]  or packed [total_q, Hq, D] with cu_seqlens_q (int32 [B+1])
    k, v         [B, sk, Hk, D]  or packed [total_k, Hk, D] with cu_seqlens_k
    k/v_cache    paged [num_pages, page_size, Hk, D] with block_table int32 [B, max_pages_per_seq]
    seqlen_k     int32 [B] valid keys per sequence
"""
import ctypes
import math
from typing import Optional, Tuple

import torch

from ... import _lib
from ...utils import FlashCKOperationType, flags, register_flashck_functions, tuning

__all__ = [
    "MASK_NONE", "MASK_TOP_LEFT", "MASK_BOTTOM_RIGHT", "MASK_GENERIC", "ROPE_NONE", "ROPE_INTERLEAVED",
    "ROPE_HALF_ROTATED", "fmha_fwd", "fmha_fwd_varlen", "fmha_fwd_splitkv", "fmha_fwd_splitkv_combine",
    "fmha_fwd_splitkv_fused", "fused_splitkv_fits",
    "fmha_fwd_appendkv", "fmha_batch_prefill", "fmha_fwd_pagedkv", "fmha_decode_paged", "fmha_decode_step",
    "tune_decode_num_splits", "tune_prefill_variant", "DecodeWorkspace", "num_splits_heuristic", "splitkv_workspace", "validate_paged", "fused_reset",
]

# GenericAttentionMaskEnum / RopeEnum, core/profiling/attention/fmha_library.h:81-87,195-200
MASK_NONE, MASK_TOP_LEFT, MASK_BOTTOM_RIGHT, MASK_GENERIC = 0, 1, 2, 3
ROPE_NONE, ROPE_INTERLEAVED, ROPE_HALF_ROTATED = 0, 1, 2

# flashck::DataType, core/utils/dtype.h:16-28.  float8_e4m3fn queries select the all-fp8 roles (Q, K, V, P and O in e4m3,
# FmhaFwdTypeConfig<fp8_t>, core/module/kernels/attention_kernels/fmha_common_jinja.h:157-171).
_DTYPE_ID = {torch.float8_e4m3fn: 1, torch.float16: 3, torch.bfloat16: 4}


# Host-side tests of the validation code switch this off (and replace _call); nothing else may.
_REQUIRE_GPU_TENSORS = True


def _dtype_id(t: torch.Tensor) -> int:
    if t.dtype not in _DTYPE_ID:
        raise TypeError(f"FMHA supports torch.float16, torch.bfloat16 and torch.float8_e4m3fn, got {t.dtype}")
    return _DTYPE_ID[t.dtype]


def _check_tensor(name, t, dtype=None, ndim=None, optional=False):
    if t is None:
        if optional:
            return
        raise TypeError(f"{name} must be a torch.Tensor, got None")
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"Expected {name} to be a torch.Tensor, got {type(t)}")
    if _REQUIRE_GPU_TENSORS and not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got device {t.device})")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must have dtype {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() not in (ndim if isinstance(ndim, tuple) else (ndim,)):
        raise ValueError(f"{name} must have {ndim} dimensions, got shape {tuple(t.shape)}")


def _check_shape(name, t, shape, like):
    """A caller-supplied buffer (workspace or output) must be exactly what the kernel is about to write: the C ABI
    only sees a pointer, so a wrong size here would be an out-of-bounds write on the GPU."""
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    if t.device != like.device:
        raise ValueError(f"{name} is on {t.device}, the inputs are on {like.device}")


def _out(name, out, shape, dtype, like):
    """`out` validated against (shape, dtype, device of `like`), or a new tensor when it is None."""
    if out is None:
        return torch.empty(*shape, dtype=dtype, device=like.device)
    _check_tensor(name, out, dtype=dtype)
    _check_shape(name, out, shape, like)
    return out


def _check_kv(q, k, v, ndim):
    """k and v against q: same rank, k's head dim is q's, v agrees with k on everything but the head dim."""
    if k.dim() != ndim or v.dim() != ndim:
        raise ValueError(f"k {tuple(k.shape)} / v {tuple(v.shape)} must have {ndim} dimensions")
    if k.shape[-1] != q.shape[-1]:
        raise ValueError(f"k head dim {k.shape[-1]} != q head dim {q.shape[-1]}")
    if v.shape[:-1] != k.shape[:-1]:
        raise ValueError(f"v {tuple(v.shape)} does not match k {tuple(k.shape)}")
    if k.shape[-2] <= 0 or q.shape[-2] % k.shape[-2]:
        raise ValueError(f"q heads {q.shape[-2]} must be a multiple of kv heads {k.shape[-2]}")


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _call(name, *args):
    lib = _lib.load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.fck_last_error().decode()
        if rc == -2:
            raise NotImplementedError(f"{name}: {msg}")
        if rc == -1:
            raise ValueError(f"{name}: {msg}")
        raise RuntimeError(f"{name} failed ({rc}): {msg}")


def _scale(scale, d):
    # scale == 0 selects 1/sqrt(head_dim), as the FlashCK harness does (fmha_fwd_split_kv_jinja.h:60-62)
    return float(scale) if scale else 1.0 / math.sqrt(d)


def _window(window):
    wl, wr = window
    return int(wl), int(wr)


def _attrs(q, bias, alibi_slopes, logits_soft_cap, group, batch, rows, min_cols, kv_fp8=False, k_descale=1.0, v_descale=1.0,
           decode_variant=0, prefill_variant=0, max_seqlen_k=0, o_scale=1.0):
    """fck_fmha_attrs for a call, or None when no score modifier is asked for.

    o_scale (float8_e4m3fn queries on the dense / paged / page-list prefill calls): the output is
    saturate(o_scale * o) in e4m3.
    bias (elementwise, BiasEnum ELEMENTWISE_BIAS): q's dtype (float32 for float8_e4m3fn queries), last dim contiguous; batch mode [1|B, 1|Hq, sq, >= sk],
    group mode [1|Hq, total_q, >= max sk]; size-1 dims are shared (the reference's rank 0 / 1 / 2).
    alibi_slopes (ALIBI): fp32 [Hq] or [B, Hq].  logits_soft_cap > 0: s = cap * tanh(scale * qk / cap).
    Returns (pointer argument, object to keep alive until the call has been made)."""
    cap = float(logits_soft_cap)
    if not (cap >= 0.0) or math.isinf(cap):
        raise ValueError("logits_soft_cap must be finite and >= 0")
    if int(decode_variant) not in (0, 1, 2, 3, 4):
        raise ValueError("decode_variant must be 0 (library's choice), 1 (one KV head per workgroup), 2 (head pairs), or 3 / 4 (the same "
                         "with splits of equal size in keys)")
    if int(prefill_variant) not in (0, 1, 2, 3, 4):
        raise ValueError("prefill_variant must be 0 (library's choice) or 1..4 (see fck_fmha_attrs.prefill_variant)")
    if bias is None and alibi_slopes is None and cap == 0.0 and not kv_fp8 and not decode_variant and not prefill_variant:
        return None, None
    if bias is not None and alibi_slopes is not None:
        raise ValueError("bias and alibi_slopes are exclusive (one BiasEnum per call)")
    a = _lib.Attrs()
    a.size = ctypes.sizeof(_lib.Attrs)
    a.logits_soft_cap = cap
    a.decode_variant = int(decode_variant)
    a.max_seqlen_k = max(int(max_seqlen_k), 0)
    a.prefill_variant = int(prefill_variant)
    if kv_fp8:
        if not (float(k_descale) > 0.0 and float(v_descale) > 0.0 and math.isfinite(k_descale) and math.isfinite(v_descale)):
            raise ValueError("k_descale and v_descale must be positive and finite")
        a.kv_dtype, a.k_descale, a.v_descale = 1, float(k_descale), float(v_descale)  # flashck::DataType FLOAT8
    if not (float(o_scale) > 0.0 and math.isfinite(o_scale)):
        raise ValueError("o_scale must be positive and finite")
    a.o_scale = float(o_scale)
    Hq = q.shape[-2]
    if bias is not None:
        if not isinstance(bias, torch.Tensor):
            raise TypeError(f"Expected bias to be a torch.Tensor, got {type(bias)}")
        if _REQUIRE_GPU_TENSORS and not bias.is_cuda:
            raise ValueError(f"bias must live on the GPU (got device {bias.device})")
        want = torch.float32 if q.dtype == torch.float8_e4m3fn else q.dtype   # BiasDataType of the e4m3 roles is float
        if bias.dtype != want:
            raise TypeError(f"bias must have dtype {want} for {q.dtype} queries, got {bias.dtype}")
        if bias.dim() != (3 if group else 4) or bias.stride(-1) != 1:
            raise ValueError(f"bias must be {'[1|Hq, total_q, sk]' if group else '[1|B, 1|Hq, sq, sk]'} with a contiguous last dim, "
                             f"got shape {tuple(bias.shape)} strides {bias.stride()}")
        if bias.shape[-3] not in (1, Hq) or (not group and bias.shape[0] not in (1, batch)):
            raise ValueError(f"bias {tuple(bias.shape)}: head dim must be 1 or {Hq}" + ("" if group else f", batch dim 1 or {batch}"))
        if bias.shape[-2] != rows or bias.shape[-1] < min_cols:
            raise ValueError(f"bias {tuple(bias.shape)} must have {rows} rows and at least {min_cols} columns")
        a.bias_type = 1
        a.bias_cols = bias.shape[-1]
        a.bias = bias.data_ptr()
        a.bias_row_stride = bias.stride(-2)
        a.bias_head_stride = bias.stride(-3) if bias.shape[-3] > 1 else 0
        a.bias_batch_stride = 0 if group or bias.shape[0] == 1 else bias.stride(0)
    elif alibi_slopes is not None:
        _check_tensor("alibi_slopes", alibi_slopes, dtype=torch.float32, ndim=(1, 2))
        if alibi_slopes.shape[-1] != Hq or (alibi_slopes.dim() == 2 and alibi_slopes.shape[0] != batch):
            raise ValueError(f"alibi_slopes must be [{Hq}] or [{batch}, {Hq}], got {tuple(alibi_slopes.shape)}")
        a.bias_type = 2
        a.bias = alibi_slopes.data_ptr()
        a.bias_batch_stride = Hq if alibi_slopes.dim() == 2 else 0
    return ctypes.byref(a), (a, bias, alibi_slopes)


def validate_paged(*, seqlen_k=None, block_table=None, kv_indptr=None, kv_page_indices=None, kv_last_page_lens=None,
                   num_total_pages: int, page_size: int, out=None, check: bool = False):
    """Debug aid: checks on the GPU what the paged kernels trust - key counts against what the block-table row / page
    list can address, page ids against the pool - without allocating when `out` (int32[4] on the device) is given.
    Returns the counters tensor [sequences with a bad length, page ids out of range, malformed page lists, first
    offending sequence or -1]; nothing is read back unless check=True, which synchronises and raises ValueError when a
    counter is non-zero.  The operators call it with check=True before every paged launch while the flag
    FC_DEBUG_KERNEL_INSTANCE is on (core/utils/flags.cc:169)."""
    paged = block_table is not None
    ref = block_table if paged else kv_indptr
    _check_tensor("block_table" if paged else "kv_indptr", ref, dtype=torch.int32, ndim=2 if paged else 1)
    if paged:
        _check_tensor("seqlen_k", seqlen_k, dtype=torch.int32, ndim=1)
        if kv_indptr is not None or kv_page_indices is not None:
            raise ValueError("give a block table or a page list, not both")
        B, stride = block_table.shape
        if seqlen_k.numel() != B:
            raise ValueError(f"seqlen_k has {seqlen_k.numel()} entries, the block table {B} rows")
    else:
        _check_tensor("kv_page_indices", kv_page_indices, dtype=torch.int32, ndim=1)
        _check_tensor("kv_last_page_lens", kv_last_page_lens, dtype=torch.int32, ndim=1, optional=True)
        B, stride = kv_indptr.numel() - 1, 0
    counts = _out("out", out, (4,), torch.int32, ref)
    _call("fck_fmha_validate_paged", _ptr(seqlen_k), _ptr(block_table), stride, _ptr(kv_indptr), _ptr(kv_page_indices),
          _ptr(kv_last_page_lens), B, int(num_total_pages), int(page_size), _ptr(counts), _stream())
    if check:
        bad_len, bad_page, bad_list, first = counts.tolist()
        if bad_len or bad_page or bad_list:
            raise ValueError(f"paged-cache arguments are inconsistent: {bad_len} sequence(s) longer than their table can address, "
                             f"{bad_page} page id(s) outside the pool of {num_total_pages}, {bad_list} malformed page list(s); "
                             f"first offending sequence: {first}")
    return counts


def _debug_validate(**kw):
    if flags.flag("FC_DEBUG_KERNEL_INSTANCE"):
        validate_paged(check=True, **kw)


def fused_reset() -> None:
    """Zero the arrival tickets of fmha_fwd_splitkv_fused on the current device and forget which stream owns which slice
    of the library's array (after a fused launch that did not run to completion, or to serve other streams; only while
    no fused call is in flight; see fck_fmha_fused_reset)."""
    _call("fck_fmha_fused_reset", _stream())


def num_splits_heuristic(batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k, head_dim, num_cu=0) -> int:
    """Split count chosen from the CU count and the KV length."""
    return int(_lib.load().fck_fmha_num_splits_heuristic(batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k,
                                                         head_dim, num_cu))


def splitkv_workspace(shape_batch, q_num_heads, shape_seqlen_q, v_head_dim, num_splits, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """(o_acc fp32 [Bs,Hq,ns,Sq,Dv], lse_acc fp32 [Bs,Hq,ns,Sq]) - fmha_fwd_split_kv_jinja.h:543-547."""
    o_acc = torch.empty(shape_batch, q_num_heads, num_splits, shape_seqlen_q, v_head_dim, dtype=torch.float32, device=device)
    lse_acc = torch.empty(shape_batch, q_num_heads, num_splits, shape_seqlen_q, dtype=torch.float32, device=device)
    return o_acc, lse_acc


def fmha_fwd(q, k, v, scale: float = 0.0, mask_type: int = MASK_NONE, window: Tuple[int, int] = (-1, -1),
             seqlen_k: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None, *, bias=None, alibi_slopes=None,
             logits_soft_cap: float = 0.0, k_descale: float = 1.0, v_descale: float = 1.0, o_scale: float = 1.0) -> torch.Tensor:
    """Dense attention, batch mode: q [B,sq,Hq,D], k/v [B,sk,Hk,D] -> o [B,sq,Hq,D].
    bias / alibi_slopes / logits_soft_cap: see _attrs.  float8_e4m3fn tensors: the all-fp8 roles, with k = k_descale *
    stored, v = v_descale * stored, o = saturate(o_scale * result)."""
    _check_tensor("q", q, ndim=4)
    _check_tensor("k", k, dtype=q.dtype, ndim=4)
    _check_tensor("v", v, dtype=q.dtype, ndim=4)
    _check_tensor("seqlen_k", seqlen_k, dtype=torch.int32, ndim=1, optional=True)
    B, sq, Hq, D = q.shape
    _check_kv(q, k, v, 4)
    if k.shape[0] != B:
        raise ValueError(f"k {tuple(k.shape)} / v {tuple(v.shape)} do not match q {tuple(q.shape)}")
    if q.numel() == 0:
        raise ValueError("Input tensor cannot be empty")
    if seqlen_k is not None and seqlen_k.numel() != B:
        raise ValueError(f"seqlen_k must have {B} entries, got {seqlen_k.numel()}")
    sk, Hk, Dv = k.shape[1], k.shape[2], v.shape[3]
    o = _out("out", out, (B, sq, Hq, Dv), q.dtype, q)
    wl, wr = _window(window)
    at, keep = _attrs(q, bias, alibi_slopes, logits_soft_cap, False, B, sq, sk, q.dtype == torch.float8_e4m3fn, k_descale, v_descale,
                      o_scale=o_scale)
    if at is None:
        _call("fck_fmha_fwd", _ptr(q), _ptr(k), _ptr(v), None, _ptr(o), None, None, _ptr(seqlen_k), B, sq, sk, Hq, Hk, D, Dv,
              sq, _scale(scale, D), wl, wr, mask_type, _dtype_id(q), _stream())
    else:
        _call("fck_fmha_fwd_attrs", _ptr(q), _ptr(k), _ptr(v), None, _ptr(o), None, None, _ptr(seqlen_k), B, sq, sk, Hq, Hk, D, Dv,
              sq, _scale(scale, D), wl, wr, mask_type, _dtype_id(q), at, _stream())
    del keep
    return o


def fmha_fwd_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q: int, scale: float = 0.0,
                    mask_type: int = MASK_NONE, window=(-1, -1), seqlen_k=None, out=None, *, bias=None, alibi_slopes=None,
                    logits_soft_cap: float = 0.0, k_descale: float = 1.0, v_descale: float = 1.0, o_scale: float = 1.0) -> torch.Tensor:
    """Dense attention, group mode: q [total_q,Hq,D], k/v [total_k,Hk,D] packed by cu_seqlens.
    bias / alibi_slopes / logits_soft_cap: see _attrs; float8_e4m3fn tensors and their scales: see fmha_fwd.

    seqlen_k (int32 [B], optional): logical key counts when the packed K/V slots hold padding behind the keys."""
    _check_tensor("q", q, ndim=3)
    _check_tensor("k", k, dtype=q.dtype, ndim=3)
    _check_tensor("v", v, dtype=q.dtype, ndim=3)
    _check_tensor("cu_seqlens_q", cu_seqlens_q, dtype=torch.int32, ndim=1)
    _check_tensor("cu_seqlens_k", cu_seqlens_k, dtype=torch.int32, ndim=1)
    if cu_seqlens_q.numel() != cu_seqlens_k.numel() or cu_seqlens_q.numel() < 2:
        raise ValueError("cu_seqlens_q and cu_seqlens_k must both have batch + 1 entries")
    B = cu_seqlens_q.numel() - 1
    tq, Hq, D = q.shape
    _check_kv(q, k, v, 3)
    _check_tensor("seqlen_k", seqlen_k, dtype=torch.int32, ndim=1, optional=True)
    if seqlen_k is not None and seqlen_k.numel() != B:
        raise ValueError(f"seqlen_k must have {B} entries, got {seqlen_k.numel()}")
    Hk, Dv = k.shape[1], v.shape[2]
    o = _out("out", out, (tq, Hq, Dv), q.dtype, q)
    wl, wr = _window(window)
    at, keep = _attrs(q, bias, alibi_slopes, logits_soft_cap, True, B, tq, 1, q.dtype == torch.float8_e4m3fn, k_descale, v_descale,
                      o_scale=o_scale)
    if at is None:
        _call("fck_fmha_fwd", _ptr(q), _ptr(k), _ptr(v), None, _ptr(o), _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), _ptr(seqlen_k), B, tq,
              k.shape[0], Hq, Hk, D, Dv, max_seqlen_q, _scale(scale, D), wl, wr, mask_type, _dtype_id(q), _stream())
    else:
        _call("fck_fmha_fwd_attrs", _ptr(q), _ptr(k), _ptr(v), None, _ptr(o), _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), _ptr(seqlen_k),
              B, tq, k.shape[0], Hq, Hk, D, Dv, max_seqlen_q, _scale(scale, D), wl, wr, mask_type, _dtype_id(q), at, _stream())
    del keep
    return o


def fmha_fwd_splitkv(q, k, v, num_splits: int, *, seqlen_k=None, block_table=None, cache_batch_idx=None,
                     cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q: int = 0, scale: float = 0.0,
                     mask_type: int = MASK_NONE, window=(-1, -1), o_acc=None, lse_acc=None, bias=None, alibi_slopes=None,
                     logits_soft_cap: float = 0.0, k_descale: float = 1.0, v_descale: float = 1.0, decode_variant: int = 0,
                     max_seqlen_k: int = 0):
    """Split-KV forward: returns the per-split partials (o_acc, lse_acc), to be merged by fmha_fwd_splitkv_combine.
    decode_variant: 0 = the library picks the kernel variant, 1 / 2 force it (what the tuner records, see
    tune_decode_num_splits); 3 / 4 = 1 / 2 with splits of equal size in keys (chunks of ceil(max_seqlen_k / num_splits)
    keys, the same for every sequence: even work items for a ragged batch; max_seqlen_k = 0 takes the block table's
    capacity).
    bias / alibi_slopes / logits_soft_cap: see _attrs.  k and v may be torch.float8_e4m3fn (a quantised cache with the
    static per-tensor scales k_descale, v_descale: value = descale * stored); q and the output keep q's dtype.

    k/v are a paged cache when block_table is given, packed when cu_seqlens_k is given, else [B*, sk, Hk, D].
    """
    group = cu_seqlens_q is not None
    _check_tensor("q", q, ndim=3 if group else 4)
    kv_fp8 = isinstance(k, torch.Tensor) and k.dtype == torch.float8_e4m3fn
    _check_tensor("k", k, dtype=torch.float8_e4m3fn if kv_fp8 else q.dtype)
    _check_tensor("v", v, dtype=torch.float8_e4m3fn if kv_fp8 else q.dtype)
    for name, t in (("seqlen_k", seqlen_k), ("block_table", block_table), ("cache_batch_idx", cache_batch_idx),
                    ("cu_seqlens_q", cu_seqlens_q), ("cu_seqlens_k", cu_seqlens_k)):
        _check_tensor(name, t, dtype=torch.int32, optional=True)
    if int(num_splits) < 1:
        raise ValueError("num_splits must be >= 1")
    Hq, D = q.shape[-2], q.shape[-1]
    _check_kv(q, k, v, 3 if (cu_seqlens_k is not None and block_table is None) else 4)
    Hk, Dv = k.shape[-2], v.shape[-1]
    if group:
        B, sq, bs = cu_seqlens_q.numel() - 1, q.shape[0], 1
        if max_seqlen_q <= 0:
            raise ValueError("group mode needs max_seqlen_q")
    else:
        B, sq, bs = q.shape[0], q.shape[1], q.shape[0]
        max_seqlen_q = sq
    if seqlen_k is not None and seqlen_k.numel() != B:
        raise ValueError(f"seqlen_k must have {B} entries, got {seqlen_k.numel()}")
    if block_table is not None:
        if seqlen_k is None:
            raise ValueError("a paged cache needs seqlen_k")
        if block_table.dim() != 2 or block_table.shape[0] != B:
            raise ValueError(f"block_table must be [batch, max_pages_per_seq], got {tuple(block_table.shape)}")
        page, sk, max_blocks = k.shape[1], 0, block_table.numel()
        _debug_validate(seqlen_k=seqlen_k, block_table=block_table, num_total_pages=k.shape[0], page_size=page)
    else:
        page, max_blocks = 0, 0
        sk = k.shape[0] if cu_seqlens_k is not None else k.shape[1]
    if (o_acc is None) != (lse_acc is None):
        raise ValueError("o_acc and lse_acc must be given together")
    if o_acc is None:
        o_acc, lse_acc = splitkv_workspace(bs, Hq, sq, Dv, num_splits, q.device)
    else:
        # the kernel writes with the strides of THIS split count
        _check_tensor("o_acc", o_acc, dtype=torch.float32)
        _check_tensor("lse_acc", lse_acc, dtype=torch.float32)
        _check_shape("o_acc", o_acc, (bs, Hq, int(num_splits), sq, Dv), q)
        _check_shape("lse_acc", lse_acc, (bs, Hq, int(num_splits), sq), q)
    wl, wr = _window(window)
    at, keep = _attrs(q, bias, alibi_slopes, logits_soft_cap, group, B, sq, 1 if (group or block_table is not None) else sk,
                      kv_fp8, k_descale, v_descale, decode_variant, max_seqlen_k=max_seqlen_k)
    if at is None:
        _call("fck_fmha_fwd_splitkv", _ptr(q), _ptr(k), _ptr(v), None, _ptr(lse_acc), _ptr(o_acc), _ptr(cu_seqlens_q),
              _ptr(cu_seqlens_k), _ptr(seqlen_k), _ptr(block_table), _ptr(cache_batch_idx), B, sq, sk, Hq, Hk, D, Dv,
              max_seqlen_q, int(num_splits), max_blocks, page, _scale(scale, D), wl, wr, mask_type, _dtype_id(q), _stream())
    else:
        _call("fck_fmha_fwd_splitkv_attrs", _ptr(q), _ptr(k), _ptr(v), None, _ptr(lse_acc), _ptr(o_acc), _ptr(cu_seqlens_q),
              _ptr(cu_seqlens_k), _ptr(seqlen_k), _ptr(block_table), _ptr(cache_batch_idx), B, sq, sk, Hq, Hk, D, Dv,
              max_seqlen_q, int(num_splits), max_blocks, page, _scale(scale, D), wl, wr, mask_type, _dtype_id(q), at, _stream())
    del keep
    return o_acc, lse_acc


# limits of the fused entry point's fixed device array (fmha_c_api.h, fck_fmha_fwd_splitkv_fused)
_FUSED_MAX_PARTIAL_FLOATS = 4 << 20
_FUSED_MAX_TICKETS = 16384
_FUSED_MAX_AUTO_SPLITS = 128


def fused_splitkv_fits(shape_batch, batch, q_num_heads, kv_num_heads, shape_seqlen_q, max_seqlen_q, v_head_dim, num_splits) -> bool:
    """Whether fmha_fwd_splitkv_fused can hold this problem's partial results (num_splits = 0: worst case of the
    library's own choice)."""
    ns = num_splits if num_splits > 0 else _FUSED_MAX_AUTO_SPLITS
    rows = max_seqlen_q * (q_num_heads // max(kv_num_heads, 1))
    m_tiles = 1 if rows <= 32 else (rows + 31) // 32
    return (shape_batch * q_num_heads * ns * shape_seqlen_q * (v_head_dim + 1) <= _FUSED_MAX_PARTIAL_FLOATS
            and batch * kv_num_heads * m_tiles <= _FUSED_MAX_TICKETS)


def fmha_fwd_splitkv_fused(q, k, v, num_splits: int = 0, *, seqlen_k=None, block_table=None, cache_batch_idx=None,
                           cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q: int = 0, scale: float = 0.0,
                           mask_type: int = MASK_NONE, window=(-1, -1), out=None) -> torch.Tensor:
    """Split-KV forward + LSE combine in one launch that allocates nothing on the GPU side: the partial results live in
    a fixed device array of the library (limits: see fused_splitkv_fits; beyond them NotImplementedError).

    num_splits = 0 lets the library take its heuristic split count for the CU count and the longest possible KV length.
    Each stream owns a slice of that array from its first call on; at most 4 streams per GPU (then NotImplementedError
    until fused_reset()).
    Arguments as fmha_fwd_splitkv; returns o [B,sq,Hq,Dv] (or [total_q,Hq,Dv] in group mode).
    """
    group = cu_seqlens_q is not None
    _check_tensor("q", q, ndim=3 if group else 4)
    _check_tensor("k", k, dtype=q.dtype)
    _check_tensor("v", v, dtype=q.dtype)
    for name, t in (("seqlen_k", seqlen_k), ("block_table", block_table), ("cache_batch_idx", cache_batch_idx),
                    ("cu_seqlens_q", cu_seqlens_q), ("cu_seqlens_k", cu_seqlens_k)):
        _check_tensor(name, t, dtype=torch.int32, optional=True)
    if int(num_splits) < 0:
        raise ValueError("num_splits must be >= 0")
    Hq, D = q.shape[-2], q.shape[-1]
    _check_kv(q, k, v, 3 if (cu_seqlens_k is not None and block_table is None) else 4)
    Hk, Dv = k.shape[-2], v.shape[-1]
    if group:
        B, sq = cu_seqlens_q.numel() - 1, q.shape[0]
        if max_seqlen_q <= 0:
            raise ValueError("group mode needs max_seqlen_q")
    else:
        B, sq = q.shape[0], q.shape[1]
        max_seqlen_q = sq
    if seqlen_k is not None and seqlen_k.numel() != B:
        raise ValueError(f"seqlen_k must have {B} entries, got {seqlen_k.numel()}")
    if block_table is not None:
        if seqlen_k is None:
            raise ValueError("a paged cache needs seqlen_k")
        if block_table.dim() != 2 or block_table.shape[0] != B:
            raise ValueError(f"block_table must be [batch, max_pages_per_seq], got {tuple(block_table.shape)}")
        page, sk, max_blocks = k.shape[1], 0, block_table.numel()
        _debug_validate(seqlen_k=seqlen_k, block_table=block_table, num_total_pages=k.shape[0], page_size=page)
    else:
        page, max_blocks = 0, 0
        sk = k.shape[0] if cu_seqlens_k is not None else k.shape[1]
    o = _out("out", out, (*q.shape[:-1], Dv), q.dtype, q)
    wl, wr = _window(window)
    _call("fck_fmha_fwd_splitkv_fused", _ptr(q), _ptr(k), _ptr(v), None, _ptr(o), _ptr(cu_seqlens_q), _ptr(cu_seqlens_k),
          _ptr(seqlen_k), _ptr(block_table), _ptr(cache_batch_idx), B, sq, sk, Hq, Hk, D, Dv, max_seqlen_q, int(num_splits),
          max_blocks, page, _scale(scale, D), wl, wr, mask_type, _dtype_id(q), _stream())
    return o


def fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype, cu_seqlens_q=None, max_seqlen_q: int = 0, out=None) -> torch.Tensor:
    """LSE combine of split-KV partials -> o [B,sq,Hq,Dv] (or [total_q,Hq,Dv] in group mode)."""
    if dtype not in _DTYPE_ID:
        raise TypeError(f"FMHA supports torch.float16, torch.bfloat16 and torch.float8_e4m3fn, got {dtype}")
    _check_tensor("lse_acc", lse_acc, dtype=torch.float32, ndim=4)
    _check_tensor("o_acc", o_acc, dtype=torch.float32, ndim=5)
    _check_tensor("cu_seqlens_q", cu_seqlens_q, dtype=torch.int32, optional=True)
    bs, Hq, ns, sq, Dv = o_acc.shape
    if tuple(lse_acc.shape) != (bs, Hq, ns, sq):
        raise ValueError(f"lse_acc {tuple(lse_acc.shape)} does not match o_acc {tuple(o_acc.shape)}")
    if lse_acc.device != o_acc.device:
        raise ValueError(f"lse_acc is on {lse_acc.device}, o_acc on {o_acc.device}")
    if cu_seqlens_q is not None:
        if bs != 1:
            raise ValueError(f"group mode partials have shape batch 1, got {bs}")
        B = cu_seqlens_q.numel() - 1
        o = _out("out", out, (sq, Hq, Dv), dtype, o_acc)
    else:
        B = bs
        o = _out("out", out, (bs, sq, Hq, Dv), dtype, o_acc)
    _call("fck_fmha_fwd_splitkv_combine", _ptr(lse_acc), _ptr(o_acc), _ptr(o), _ptr(cu_seqlens_q), B, sq, Hq, Dv,
          max_seqlen_q or sq, ns, _DTYPE_ID[dtype], _stream())
    return o


def fmha_fwd_appendkv(q, k_cache, v_cache, knew, vnew, seqlen_k, *, cu_seqlens_knew=None, max_seqlen_knew: int = 0,
                      rotary_cos=None, rotary_sin=None, rope_mode: int = ROPE_NONE, has_mask: bool = True,
                      block_table=None, cache_batch_idx=None, k_descale: float = 1.0, v_descale: float = 1.0) -> None:
    """Rotate knew (and q, in place) and append knew/vnew to the cache behind seqlen_k[b] tokens; in place.

    knew/vnew/q are packed [total_new, H, D] with cu_seqlens_knew, or [B, n, H, D] with n new tokens everywhere.
    seqlen_k is NOT advanced: the caller adds the new counts, as with the ck_tile kernel.
    torch.float8_e4m3fn caches are written quantised with the static scales: cache = fp8(x / descale), saturating.
    """
    packed = cu_seqlens_knew is not None
    _check_tensor("knew", knew, ndim=3 if packed else 4)
    _check_tensor("vnew", vnew, dtype=knew.dtype, ndim=3 if packed else 4)
    _check_tensor("q", q, dtype=knew.dtype, ndim=3 if packed else 4, optional=True)
    kv_fp8 = isinstance(k_cache, torch.Tensor) and k_cache.dtype == torch.float8_e4m3fn
    _check_tensor("k_cache", k_cache, dtype=torch.float8_e4m3fn if kv_fp8 else knew.dtype, ndim=4)
    _check_tensor("v_cache", v_cache, dtype=torch.float8_e4m3fn if kv_fp8 else knew.dtype, ndim=4)
    _check_tensor("seqlen_k", seqlen_k, dtype=torch.int32, ndim=1)
    for name, t in (("cu_seqlens_knew", cu_seqlens_knew), ("block_table", block_table), ("cache_batch_idx", cache_batch_idx)):
        _check_tensor(name, t, dtype=torch.int32, optional=True)
    _check_tensor("rotary_cos", rotary_cos, dtype=knew.dtype, ndim=2, optional=True)
    _check_tensor("rotary_sin", rotary_sin, dtype=knew.dtype, ndim=2, optional=True)
    B = seqlen_k.numel()
    Hk, D, Dv = knew.shape[-2], knew.shape[-1], vnew.shape[-1]
    Hq = q.shape[-2] if q is not None else 0
    if k_cache.shape[2:] != (Hk, D) or v_cache.shape[2:] != (Hk, Dv) or v_cache.shape[:2] != k_cache.shape[:2]:
        raise ValueError(f"k_cache {tuple(k_cache.shape)} / v_cache {tuple(v_cache.shape)} do not match knew "
                         f"{tuple(knew.shape)} / vnew {tuple(vnew.shape)}")
    if vnew.shape[:-1] != knew.shape[:-1]:
        raise ValueError(f"vnew {tuple(vnew.shape)} does not match knew {tuple(knew.shape)}")
    if q is not None and (q.shape[-1] != D or q.shape[:-2] != knew.shape[:-2] or Hq % Hk):
        raise ValueError(f"q {tuple(q.shape)} does not match knew {tuple(knew.shape)}")
    if packed and cu_seqlens_knew.numel() != B + 1:
        raise ValueError(f"cu_seqlens_knew must have {B + 1} entries, got {cu_seqlens_knew.numel()}")
    if not packed and knew.shape[0] != B:
        raise ValueError(f"knew batch {knew.shape[0]} != number of sequences {B}")
    if block_table is not None and (block_table.dim() != 2 or block_table.shape[0] != B):
        raise ValueError(f"block_table must be [batch, max_pages_per_seq] with batch {B}, got {tuple(block_table.shape)}")
    if rope_mode != ROPE_NONE and rotary_cos is not None and rotary_sin is not None and rotary_cos.shape != rotary_sin.shape:
        raise ValueError("rotary_cos and rotary_sin must have the same shape")
    if packed:
        if max_seqlen_knew <= 0:
            raise ValueError("packed new tokens need max_seqlen_knew")
        n = max_seqlen_knew
    else:
        n = knew.shape[1]
    if rope_mode != ROPE_NONE:
        if rotary_cos is None or rotary_sin is None:
            raise ValueError("rope_mode != ROPE_NONE needs rotary_cos and rotary_sin")
        rotary_dim = rotary_cos.shape[1] * 2
    else:
        rotary_dim = 0
    if block_table is not None:
        stride, page, rows = block_table.shape[1], k_cache.shape[1], 0
        if flags.flag("FC_DEBUG_KERNEL_INSTANCE"):  # the table must hold the sequences WITH their new tokens
            grown = seqlen_k + ((cu_seqlens_knew[1:] - cu_seqlens_knew[:-1]) if packed else n)
            validate_paged(seqlen_k=grown.to(torch.int32), block_table=block_table, num_total_pages=k_cache.shape[0],
                           page_size=page, check=True)
    else:
        stride, page, rows = 0, 0, k_cache.shape[1]
    args = (_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(knew), _ptr(vnew), _ptr(seqlen_k), _ptr(cu_seqlens_knew), n,
            _ptr(rotary_cos), _ptr(rotary_sin), rotary_dim, rope_mode, int(bool(has_mask)), _ptr(block_table), stride, page,
            _ptr(cache_batch_idx), rows, B, Hq, Hk, D, Dv, _dtype_id(knew))
    if kv_fp8:
        if not (float(k_descale) > 0.0 and float(v_descale) > 0.0 and math.isfinite(k_descale) and math.isfinite(v_descale)):
            raise ValueError("k_descale and v_descale must be positive and finite")
        at = _lib.Attrs()
        at.size = ctypes.sizeof(_lib.Attrs)
        at.kv_dtype, at.k_descale, at.v_descale = 1, float(k_descale), float(v_descale)  # flashck::DataType FLOAT8
        _call("fck_fmha_fwd_appendkv_attrs", *args, ctypes.byref(at), _stream())
    else:
        _call("fck_fmha_fwd_appendkv", *args, _stream())


def _usable_prefill_variant(variant, head_dim, v_head_dim, max_seqlen_q, page_size):
    """A cached tile variant is a hint (the problem class is coarser than the variant's preconditions): variants 2..4
    need the ping-pong kernel, i.e. equal head dims of 64 or 128, query runs longer than 128 and pages a multiple of 64."""
    variant = int(variant)
    if variant in (2, 3, 4):
        ok = head_dim == v_head_dim and head_dim in (64, 128) and max_seqlen_q > 128 and page_size % 64 == 0
        return variant if ok else 0
    return variant if variant == 1 else 0


def tune_prefill_variant(q, k_cache, v_cache, cu_seqlens_q, kv_indptr, kv_page_indices, kv_last_page_lens=None, *, max_seqlen_q: int,
                         variants=(1, 2, 3, 4), cache=None, **kwargs) -> dict:
    """Time fmha_batch_prefill with each tile variant on these tensors and record the fastest for the problem class (see
    utils/tuning.py); later calls on problems of that class with prefill_variant = 0 use it.  Returns the record."""
    tq, Hq, D = q.shape
    _, page, Hk, Dv = v_cache.shape
    mask_type = kwargs.get("mask_type", MASK_BOTTOM_RIGHT)
    problem = tuning.prefill_problem(Hq, Hk, D, max_seqlen_q, tq, page, "fp16" if q.dtype == torch.float16 else "bf16", mask_type)
    out = torch.empty(tq, Hq, Dv, dtype=q.dtype, device=q.device)

    def run(variant):
        fmha_batch_prefill(q, k_cache, v_cache, cu_seqlens_q, kv_indptr, kv_page_indices, kv_last_page_lens, max_seqlen_q=max_seqlen_q,
                           out=out, prefill_variant=variant, **kwargs)
        return _lib.load().fck_fmha_last_kernel().decode()

    return tuning.tune_prefill_variant(run, tuning.gpu_timer, variants, problem, cache=cache)


def fmha_batch_prefill(q, k_cache, v_cache, cu_seqlens_q, kv_indptr, kv_page_indices, kv_last_page_lens=None, *,
                       max_seqlen_q: int, scale: float = 0.0, mask_type: int = MASK_BOTTOM_RIGHT, window=(-1, 0),
                       out=None, bias=None, alibi_slopes=None, logits_soft_cap: float = 0.0, k_descale: float = 1.0,
                       v_descale: float = 1.0, prefill_variant: int = 0, o_scale: float = 1.0) -> torch.Tensor:
    """Varlen prefill over a page list: q [total_q,Hq,D]; sequence b owns pages
    kv_page_indices[kv_indptr[b]:kv_indptr[b+1]] of the cache [num_pages, page_size, Hk, D].  The caches may be
    torch.float8_e4m3fn with the static scales k_descale / v_descale (value = descale * stored); with float8_e4m3fn
    queries as well (the all-fp8 roles) the output is float8_e4m3fn, saturate(o_scale * result)."""
    _check_tensor("q", q, ndim=3)
    kv_fp8 = isinstance(k_cache, torch.Tensor) and k_cache.dtype == torch.float8_e4m3fn
    _check_tensor("k_cache", k_cache, dtype=torch.float8_e4m3fn if kv_fp8 else q.dtype, ndim=4)
    _check_tensor("v_cache", v_cache, dtype=torch.float8_e4m3fn if kv_fp8 else q.dtype, ndim=4)
    for name, t in (("cu_seqlens_q", cu_seqlens_q), ("kv_indptr", kv_indptr), ("kv_page_indices", kv_page_indices)):
        _check_tensor(name, t, dtype=torch.int32, ndim=1)
    _check_tensor("kv_last_page_lens", kv_last_page_lens, dtype=torch.int32, ndim=1, optional=True)
    B = cu_seqlens_q.numel() - 1
    if kv_indptr.numel() != B + 1:
        raise ValueError("kv_indptr must have batch + 1 entries")
    tq, Hq, D = q.shape
    _check_kv(q, k_cache, v_cache, 4)
    if kv_last_page_lens is not None and kv_last_page_lens.numel() != B:
        raise ValueError(f"kv_last_page_lens must have {B} entries, got {kv_last_page_lens.numel()}")
    num_pages, page, Hk, Dv = v_cache.shape
    o = _out("out", out, (tq, Hq, Dv), q.dtype, q)
    wl, wr = _window(window)
    _debug_validate(kv_indptr=kv_indptr, kv_page_indices=kv_page_indices, kv_last_page_lens=kv_last_page_lens,
                    num_total_pages=num_pages, page_size=page)
    plain = bias is None and alibi_slopes is None and not logits_soft_cap and not kv_fp8
    if not prefill_variant and plain:   # a tuned tile variant for this class of problems, if one is recorded and fits
        prefill_variant = _usable_prefill_variant(tuning.choose_prefill_variant(tuning.prefill_problem(
            Hq, Hk, D, max_seqlen_q, tq, page, "fp16" if q.dtype == torch.float16 else "bf16", mask_type)), D, Dv, max_seqlen_q, page)
    at, keep = _attrs(q, bias, alibi_slopes, logits_soft_cap, True, B, tq, 1, kv_fp8, k_descale, v_descale,
                      prefill_variant=prefill_variant, o_scale=o_scale)
    if at is None:
        _call("fck_fmha_batch_prefill", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(o), _ptr(cu_seqlens_q), _ptr(kv_indptr),
              _ptr(kv_page_indices), _ptr(kv_last_page_lens), num_pages, page, B, Hq, Hk, D, Dv, max_seqlen_q,
              _scale(scale, D), wl, wr, mask_type, _dtype_id(q), _stream())
    else:
        _call("fck_fmha_batch_prefill_attrs", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(o), _ptr(cu_seqlens_q), _ptr(kv_indptr),
              _ptr(kv_page_indices), _ptr(kv_last_page_lens), num_pages, page, B, Hq, Hk, D, Dv, max_seqlen_q,
              _scale(scale, D), wl, wr, mask_type, _dtype_id(q), at, _stream())
    del keep
    return o


def fmha_fwd_pagedkv(q, k_cache, v_cache, seqlen_k, block_table, *, cu_seqlens_q=None, max_seqlen_q: int = 0,
                     scale: float = 0.0, mask_type: int = MASK_BOTTOM_RIGHT, window=(-1, 0), out=None, bias=None,
                     alibi_slopes=None, logits_soft_cap: float = 0.0, k_descale: float = 1.0, v_descale: float = 1.0,
                     prefill_variant: int = 0, o_scale: float = 1.0) -> torch.Tensor:
    """Prefill over a block table (no splits): q [B,sq,Hq,D] or packed [total_q,Hq,D].  The caches may be
    torch.float8_e4m3fn with the static scales k_descale / v_descale (value = descale * stored); float8_e4m3fn queries
    and o_scale: see fmha_batch_prefill."""
    group = cu_seqlens_q is not None
    _check_tensor("q", q, ndim=3 if group else 4)
    kv_fp8 = isinstance(k_cache, torch.Tensor) and k_cache.dtype == torch.float8_e4m3fn
    _check_tensor("k_cache", k_cache, dtype=torch.float8_e4m3fn if kv_fp8 else q.dtype, ndim=4)
    _check_tensor("v_cache", v_cache, dtype=torch.float8_e4m3fn if kv_fp8 else q.dtype, ndim=4)
    _check_tensor("seqlen_k", seqlen_k, dtype=torch.int32, ndim=1)
    _check_tensor("block_table", block_table, dtype=torch.int32, ndim=2)
    _check_tensor("cu_seqlens_q", cu_seqlens_q, dtype=torch.int32, ndim=1, optional=True)
    B = seqlen_k.numel()
    Hq, D = q.shape[-2], q.shape[-1]
    _check_kv(q, k_cache, v_cache, 4)
    if block_table.shape[0] != B:
        raise ValueError(f"block_table must be [batch, max_pages_per_seq] with batch {B}, got {tuple(block_table.shape)}")
    if (cu_seqlens_q.numel() - 1 if group else q.shape[0]) != B:
        raise ValueError("seqlen_k must have one entry per sequence of q")
    _, page, Hk, Dv = v_cache.shape
    sq = 0 if group else q.shape[1]
    if group and max_seqlen_q <= 0:
        raise ValueError("group mode needs max_seqlen_q")
    o = _out("out", out, (*q.shape[:-1], Dv), q.dtype, q)
    wl, wr = _window(window)
    _debug_validate(seqlen_k=seqlen_k, block_table=block_table, num_total_pages=k_cache.shape[0], page_size=page)
    at, keep = _attrs(q, bias, alibi_slopes, logits_soft_cap, group, B, q.shape[0] if group else sq, 1, kv_fp8, k_descale, v_descale,
                      prefill_variant=prefill_variant, o_scale=o_scale)
    if at is None:
        _call("fck_fmha_fwd_pagedkv", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(o), _ptr(cu_seqlens_q), _ptr(seqlen_k),
              _ptr(block_table), block_table.shape[1], page, B, sq, Hq, Hk, D, Dv, max_seqlen_q or sq, _scale(scale, D), wl, wr,
              mask_type, _dtype_id(q), _stream())
    else:
        _call("fck_fmha_fwd_pagedkv_attrs", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(o), _ptr(cu_seqlens_q), _ptr(seqlen_k),
              _ptr(block_table), block_table.shape[1], page, B, sq, Hq, Hk, D, Dv, max_seqlen_q or sq, _scale(scale, D), wl, wr,
              mask_type, _dtype_id(q), at, _stream())
    del keep
    return o


def _auto_num_splits(batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k, head_dim, page_size, dtype):
    """(split count, kernel variant): the tuned pair recorded for this class of problems if there is one, else the
    heuristic split count and variant 0 (the library's choice)."""
    return tuning.choose_splitkv(
        lambda: num_splits_heuristic(batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k, head_dim),
        batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k, head_dim, page_size,
        "fp16" if dtype == torch.float16 else "bf16")


def _usable_variant(variant, q_num_heads, kv_num_heads, rows, head_dim, v_head_dim, plain=True, page_size=128):
    """A kernel variant from the tuning cache is a hint: the record's problem class is coarser than what the variant
    needs (query counts are bucketed, v_head_dim is not part of the key), so its preconditions are checked again for
    this call, and 0 (the library's choice) is returned when one fails.  Head pairs (2) need an even number of KV heads,
    equal head dims of 64 or 128 and at most 16 packed query rows (queries x heads per KV head); a record is only served to
    the kind of call it was measured with (plain: no score modifier, 16-bit cache); one head per workgroup (1) fits
    every call.  Variants 3 / 4 (splits of equal size) are 1 / 2 for plain calls with at most 16 packed rows, head dim 64
    or 128 and pages a multiple of 32 keys."""
    variant = int(variant)
    g = q_num_heads // max(kv_num_heads, 1)
    small = plain and head_dim == v_head_dim and head_dim in (64, 128) and rows * g <= 16
    if variant in (2, 4):
        return variant if small and kv_num_heads % 2 == 0 and (variant == 2 or page_size % 32 == 0) else 0
    if variant == 3:
        return 3 if small and page_size % 32 == 0 else 0
    return variant if variant == 1 else 0


def fmha_decode_paged(q, k_cache, v_cache, seqlen_k, block_table, *, num_splits: int = 0, max_seqlen_k: int = 0,
                      cu_seqlens_q=None, max_seqlen_q: int = 0, scale: float = 0.0, mask_type: int = MASK_NONE,
                      window=(-1, -1), workspace=None, out=None, fused: bool = False, bias=None, alibi_slopes=None,
                      logits_soft_cap: float = 0.0, k_descale: float = 1.0, v_descale: float = 1.0,
                      decode_variant: int = 0) -> torch.Tensor:
    """Paged decode = split-KV forward + LSE combine; num_splits = 0 asks the tuning cache, then the heuristic (needs
    max_seqlen_k); a cached record also brings the kernel variant it was measured with.  bias / alibi_slopes /
    logits_soft_cap / fp8 caches with k_descale, v_descale: as fmha_fwd_splitkv (not with fused = True).

    fused = True runs both in one launch that allocates nothing (fmha_fwd_splitkv_fused; the partial results then live
    in the library's fixed device array, `workspace` is not used, and problems beyond its limits raise)."""
    group = cu_seqlens_q is not None
    _check_tensor("q", q, ndim=3 if group else 4)
    kv_fp8 = isinstance(k_cache, torch.Tensor) and k_cache.dtype == torch.float8_e4m3fn
    _check_tensor("k_cache", k_cache, dtype=torch.float8_e4m3fn if kv_fp8 else q.dtype, ndim=4)
    _check_tensor("v_cache", v_cache, dtype=torch.float8_e4m3fn if kv_fp8 else q.dtype, ndim=4)
    _check_tensor("seqlen_k", seqlen_k, dtype=torch.int32, ndim=1)
    _check_tensor("block_table", block_table, dtype=torch.int32, ndim=2)
    Hq, D = q.shape[-2], q.shape[-1]
    Hk = k_cache.shape[2]
    B = seqlen_k.numel()
    sq = max_seqlen_q if group else q.shape[1]
    plain = bias is None and alibi_slopes is None and not logits_soft_cap and not kv_fp8
    if workspace is not None and num_splits <= 0:
        # the partials are laid out for one split count: with a caller-owned workspace that count is the workspace's
        num_splits = int(workspace[0].shape[2]) if workspace[0].dim() == 5 else 0
        if num_splits <= 0:
            raise ValueError("workspace must be (o_acc [Bs,Hq,ns,Sq,Dv], lse_acc [Bs,Hq,ns,Sq])")
    if num_splits <= 0:
        if max_seqlen_k <= 0:
            max_seqlen_k = block_table.shape[1] * k_cache.shape[1]
        num_splits, cached_variant = _auto_num_splits(B, Hq, Hk, sq, max_seqlen_k, D, k_cache.shape[1], q.dtype)
        if not decode_variant:
            decode_variant = _usable_variant(cached_variant, Hq, Hk, sq, D, v_cache.shape[3], plain, k_cache.shape[1])
    if fused:
        if not plain or decode_variant:
            raise NotImplementedError("the fused launch takes no bias / soft cap / fp8 cache / kernel variant")
        return fmha_fwd_splitkv_fused(q, k_cache, v_cache, num_splits, seqlen_k=seqlen_k, block_table=block_table,
                                      cu_seqlens_q=cu_seqlens_q, max_seqlen_q=max_seqlen_q, scale=scale,
                                      mask_type=mask_type, window=window, out=out)
    o_acc, lse_acc = workspace if workspace is not None else (None, None)
    o_acc, lse_acc = fmha_fwd_splitkv(q, k_cache, v_cache, num_splits, seqlen_k=seqlen_k, block_table=block_table,
                                      cu_seqlens_q=cu_seqlens_q, max_seqlen_q=max_seqlen_q, scale=scale,
                                      mask_type=mask_type, window=window, o_acc=o_acc, lse_acc=lse_acc, bias=bias,
                                      alibi_slopes=alibi_slopes, logits_soft_cap=logits_soft_cap, k_descale=k_descale,
                                      v_descale=v_descale, decode_variant=decode_variant, max_seqlen_k=max_seqlen_k)
    return fmha_fwd_splitkv_combine(lse_acc, o_acc, q.dtype, cu_seqlens_q=cu_seqlens_q, max_seqlen_q=max_seqlen_q, out=out)


def tune_decode_num_splits(q, k_cache, v_cache, seqlen_k, block_table, *, max_seqlen_k: int,
                           candidates=(1, 2, 4, 8, 16, 32, 64), variants=(0,), cache=None, **kwargs) -> dict:
    """Time `fmha_decode_paged` with each candidate (split count, kernel variant) on these tensors and record the
    fastest for the problem class (see utils/tuning.py); later calls with num_splits = 0 on problems of that class use
    both.  variants: 0 = the library's own choice, 1 = one KV head per workgroup, 2 = head pairs (skipped where the
    problem cannot take it).  cache: the tuning.TuningCache to record into (default: the process-wide one).  Returns
    the record ({"num_splits", "variant", "kernel", "latency_us", "tried_us", ...})."""
    Hq, D = q.shape[-2], q.shape[-1]
    Hk, page = k_cache.shape[2], k_cache.shape[1]
    B = seqlen_k.numel()
    sq = kwargs.get("max_seqlen_q", 0) or (q.shape[1] if q.dim() == 4 else 1)
    problem = tuning.splitkv_problem(B, Hq, Hk, sq, max_seqlen_k, D, page, "fp16" if q.dtype == torch.float16 else "bf16")
    ws = {}

    def run(ns, variant=0):
        if ns not in ws:
            shape_batch, shape_sq = (1, q.shape[0]) if q.dim() == 3 else (q.shape[0], q.shape[1])
            ws[ns] = splitkv_workspace(shape_batch, Hq, shape_sq, v_cache.shape[3], ns, q.device)
        fmha_decode_paged(q, k_cache, v_cache, seqlen_k, block_table, num_splits=ns, max_seqlen_k=max_seqlen_k,
                          workspace=ws[ns], decode_variant=variant, **kwargs)
        return _lib.load().fck_fmha_last_kernel().decode()

    return tuning.tune_num_splits(run, tuning.gpu_timer, candidates, problem, cache=cache, variants=variants)


class DecodeWorkspace:
    """Buffers a decode step needs besides its inputs and outputs, kept between steps.

    Holds the split-KV partials (o_acc, lse_acc) and the advanced key counts.  Buffers are only reallocated when a
    step needs a larger one, so a serving loop with a fixed batch allocates on its first step only.
    """

    def __init__(self):
        self._o_acc = None
        self._lse_acc = None
        self._seqlen = None
        self._counts = None

    @staticmethod
    def _fit(buf, numel, dtype, device):
        if buf is None or buf.numel() < numel or buf.dtype != dtype or buf.device != device:
            buf = torch.empty(numel, dtype=dtype, device=device)
        return buf

    def partials(self, shape_batch, q_num_heads, num_splits, shape_seqlen_q, v_head_dim, device):
        n_lse = shape_batch * q_num_heads * num_splits * shape_seqlen_q
        self._o_acc = self._fit(self._o_acc, n_lse * v_head_dim, torch.float32, device)
        self._lse_acc = self._fit(self._lse_acc, n_lse, torch.float32, device)
        o_acc = self._o_acc[:n_lse * v_head_dim].view(shape_batch, q_num_heads, num_splits, shape_seqlen_q, v_head_dim)
        lse_acc = self._lse_acc[:n_lse].view(shape_batch, q_num_heads, num_splits, shape_seqlen_q)
        return o_acc, lse_acc

    def lengths(self, batch, device):
        self._seqlen = self._fit(self._seqlen, batch, torch.int32, device)
        self._counts = self._fit(self._counts, batch, torch.int32, device)
        return self._seqlen[:batch], self._counts[:batch]


def fmha_decode_step(q, knew, vnew, k_cache, v_cache, seqlen_k, block_table, *, cu_seqlens_knew=None,
                     max_seqlen_knew: int = 0, rotary_cos=None, rotary_sin=None, rope_mode: int = ROPE_NONE,
                     num_splits: int = 0, max_seqlen_k: int = 0, scale: float = 0.0, window_left: int = -1,
                     workspace: Optional[DecodeWorkspace] = None, out=None, k_descale: float = 1.0, v_descale: float = 1.0):
    """One serving step over a paged cache: append the new tokens, then attend from them.

    The caller side of the split-KV path, FmhaKind::FwdAppendKV -> FwdSplitKV -> FwdSplitKVCombine
    (core/profiling/attention/fmha_library.h:17-25), with the argument set of AttentionLayer
    (core/module/layers/attention_layers/attention_layer.h:13-35):
      1. knew is rotated and knew/vnew are written behind the seqlen_k[b] tokens of each sequence; q is rotated in
         place at the same positions;
      2. the split count comes from the CU count and the longest possible KV length unless num_splits is given;
      3. split-KV forward over the seqlen_k[b] + n_b keys now in the cache - query i of a sequence sees keys up to
         its own position (bottom-right causal; window_left >= 0 adds a sliding window) - and the LSE combine.
    q/knew/vnew are [B, n, H, D] (n new tokens everywhere) or packed [total_new, H, D] with cu_seqlens_knew and
    max_seqlen_knew.  Nothing is read back from the GPU, so a step only enqueues work on the current stream.
    With torch.float8_e4m3fn caches the new rows are quantised on their way in and dequantised by the attention
    kernel, both with the static scales k_descale / v_descale.

    Returns (o, seqlen_k_new): o has q's shape (with Dv); seqlen_k_new = seqlen_k + n_b lives in the workspace and is
    overwritten by the next step; seqlen_k itself is not modified.
    """
    packed = cu_seqlens_knew is not None
    ws = workspace if workspace is not None else DecodeWorkspace()
    B = seqlen_k.numel()
    Hq, D = q.shape[-2], q.shape[-1]
    Hk, Dv = k_cache.shape[2], v_cache.shape[3]
    page = k_cache.shape[1]
    if packed:
        if max_seqlen_knew <= 0:
            raise ValueError("packed new tokens need max_seqlen_knew")
        n = int(max_seqlen_knew)
    else:
        if q.dim() != 4:
            raise ValueError(f"q must be [B, n, Hq, D] without cu_seqlens_knew, got shape {tuple(q.shape)}")
        n = q.shape[1]
    fmha_fwd_appendkv(q, k_cache, v_cache, knew, vnew, seqlen_k, cu_seqlens_knew=cu_seqlens_knew, max_seqlen_knew=n,
                      rotary_cos=rotary_cos, rotary_sin=rotary_sin, rope_mode=rope_mode, has_mask=True,
                      block_table=block_table, k_descale=k_descale, v_descale=v_descale)
    kv_fp8 = k_cache.dtype == torch.float8_e4m3fn
    seqlen_new, counts = ws.lengths(B, seqlen_k.device)
    if packed:
        torch.sub(cu_seqlens_knew[1:], cu_seqlens_knew[:-1], out=counts)
        torch.add(seqlen_k, counts, out=seqlen_new)
    else:
        torch.add(seqlen_k, n, out=seqlen_new)
    if num_splits <= 0:
        if max_seqlen_k <= 0:
            max_seqlen_k = block_table.shape[1] * page  # what the block table can address
        num_splits, decode_variant = _auto_num_splits(B, Hq, Hk, n, max_seqlen_k, D, page, q.dtype)
        decode_variant = _usable_variant(decode_variant, Hq, Hk, n, D, Dv, plain=not kv_fp8, page_size=page)
    else:
        decode_variant = 0
    # a lone new token sees every key: no mask needed unless a sliding window is asked for
    if n == 1 and window_left < 0:
        mask_type, window = MASK_NONE, (-1, -1)
    else:
        mask_type, window = MASK_BOTTOM_RIGHT, (int(window_left), 0)
    shape_batch, shape_sq = (1, q.shape[0]) if packed else (B, n)
    o_acc, lse_acc = ws.partials(shape_batch, Hq, num_splits, shape_sq, Dv, q.device)
    fmha_fwd_splitkv(q, k_cache, v_cache, num_splits, seqlen_k=seqlen_new, block_table=block_table,
                     cu_seqlens_q=cu_seqlens_knew, max_seqlen_q=n if packed else 0, scale=scale, mask_type=mask_type,
                     window=window, o_acc=o_acc, lse_acc=lse_acc, decode_variant=decode_variant, k_descale=k_descale,
                     v_descale=v_descale, max_seqlen_k=max_seqlen_k)
    o = fmha_fwd_splitkv_combine(lse_acc, o_acc, q.dtype, cu_seqlens_q=cu_seqlens_knew, max_seqlen_q=n if packed else 0,
                                 out=out)
    return o, seqlen_new


register_flashck_functions(FlashCKOperationType.FMHA.value, {
    "forward": fmha_fwd,
    "forward_varlen": fmha_fwd_varlen,
    "forward_splitkv": fmha_fwd_splitkv,
    "forward_splitkv_combine": fmha_fwd_splitkv_combine,
    "forward_appendkv": fmha_fwd_appendkv,
    "batch_prefill": fmha_batch_prefill,
    "forward_pagedkv": fmha_fwd_pagedkv,
    "decode_paged": fmha_decode_paged,
    "decode_step": fmha_decode_step,
})
