"""Attention modules: stateless parameter holders over `flashck_amd.ops.fmha`.

`Attention` takes the constructor arguments of AttentionLayer<T>
(core/module/layers/attention_layers/attention_layer.h:13-35: head counts, head dims, scale, window, mask) and its call
arguments (q, k, v, seqstart_q, seqstart_k, seqlen_k); the module style follows flash_ck/nn/norm/layer_norm.py:19-110
(validation in the constructor, `extra_repr`, no fallback path here).  `PagedAttention` is the serving-side caller of
the same kernels: prefill over a paged cache and the append -> split-KV -> combine decode step, with the workspace kept
between steps.
"""
import math
from typing import Optional, Tuple

import torch

from ..ops.fmha import fmha


def _check_heads(q_num_heads, kv_num_heads, qk_head_dim, v_head_dim):
    for name, v in (("q_num_heads", q_num_heads), ("kv_num_heads", kv_num_heads), ("qk_head_dim", qk_head_dim),
                    ("v_head_dim", v_head_dim)):
        if not isinstance(v, int) or v <= 0:
            raise ValueError(f"{name} must be a positive int, got {v!r}")
    if q_num_heads % kv_num_heads != 0:
        raise ValueError(f"q_num_heads ({q_num_heads}) must be a multiple of kv_num_heads ({kv_num_heads})")


class Attention(torch.nn.Module):
    """Dense attention, batch mode ([B, s, H, D] tensors) or group mode (packed tensors with seqstart_q/seqstart_k)."""

    def __init__(self, q_num_heads: int, kv_num_heads: int, qk_head_dim: int, v_head_dim: Optional[int] = None,
                 scale: float = 0.0, window_size: Tuple[int, int] = (-1, -1), mask_type: int = fmha.MASK_NONE):
        super().__init__()
        v_head_dim = qk_head_dim if v_head_dim is None else v_head_dim
        _check_heads(q_num_heads, kv_num_heads, qk_head_dim, v_head_dim)
        if mask_type not in (fmha.MASK_NONE, fmha.MASK_TOP_LEFT, fmha.MASK_BOTTOM_RIGHT, fmha.MASK_GENERIC):
            raise ValueError(f"unknown mask_type {mask_type}")
        self.q_num_heads, self.kv_num_heads = q_num_heads, kv_num_heads
        self.qk_head_dim, self.v_head_dim = qk_head_dim, v_head_dim
        self.scale = float(scale)  # 0 selects 1/sqrt(qk_head_dim)
        self.window_size = (int(window_size[0]), int(window_size[1]))
        self.mask_type = mask_type

    def _check(self, q, k, v):
        if q.shape[-2] != self.q_num_heads or q.shape[-1] != self.qk_head_dim:
            raise ValueError(f"q has heads x dim {tuple(q.shape[-2:])}, module expects ({self.q_num_heads}, {self.qk_head_dim})")
        if k.shape[-2] != self.kv_num_heads or k.shape[-1] != self.qk_head_dim:
            raise ValueError(f"k has heads x dim {tuple(k.shape[-2:])}, module expects ({self.kv_num_heads}, {self.qk_head_dim})")
        if v.shape[-2] != self.kv_num_heads or v.shape[-1] != self.v_head_dim:
            raise ValueError(f"v has heads x dim {tuple(v.shape[-2:])}, module expects ({self.kv_num_heads}, {self.v_head_dim})")

    def forward(self, q, k, v, seqstart_q=None, seqstart_k=None, seqlen_k=None, max_seqlen_q: int = 0):
        self._check(q, k, v)
        if (seqstart_q is None) != (seqstart_k is None):
            raise ValueError("group mode needs both seqstart_q and seqstart_k")
        if seqstart_q is not None:
            if max_seqlen_q <= 0:
                raise ValueError("group mode needs max_seqlen_q")
            return fmha.fmha_fwd_varlen(q, k, v, seqstart_q, seqstart_k, max_seqlen_q, scale=self.scale,
                                        mask_type=self.mask_type, window=self.window_size)
        return fmha.fmha_fwd(q, k, v, scale=self.scale, mask_type=self.mask_type, window=self.window_size,
                             seqlen_k=seqlen_k)

    def extra_repr(self) -> str:
        return (f"q_num_heads={self.q_num_heads}, kv_num_heads={self.kv_num_heads}, qk_head_dim={self.qk_head_dim}, "
                f"v_head_dim={self.v_head_dim}, scale={self.scale}, window_size={self.window_size}, mask_type={self.mask_type}")


class PagedAttention(torch.nn.Module):
    """Causal attention over a paged KV cache [num_pages, page_size, Hk, D]: `prefill` for whole prompts already in the
    cache, `decode_step` for appending new tokens and attending from them.  The caches may be torch.float8_e4m3fn with the
    static per-tensor scales k_descale / v_descale (value = descale * stored; the reference's is_static_quant,
    core/profiling/attention/fmha_fwd_split_kv/fmha_fwd_split_kv_problem.h:79): decode_step then quantises what it
    appends and both calls dequantise what they read."""

    def __init__(self, q_num_heads: int, kv_num_heads: int, qk_head_dim: int, v_head_dim: Optional[int] = None,
                 scale: float = 0.0, window_left: int = -1, rope_mode: int = fmha.ROPE_NONE, num_splits: int = 0,
                 k_descale: float = 1.0, v_descale: float = 1.0):
        super().__init__()
        v_head_dim = qk_head_dim if v_head_dim is None else v_head_dim
        _check_heads(q_num_heads, kv_num_heads, qk_head_dim, v_head_dim)
        if rope_mode not in (fmha.ROPE_NONE, fmha.ROPE_INTERLEAVED, fmha.ROPE_HALF_ROTATED):
            raise ValueError(f"unknown rope_mode {rope_mode}")
        if num_splits < 0:
            raise ValueError("num_splits must be >= 0 (0 = choose from the CU count and the KV length)")
        self.q_num_heads, self.kv_num_heads = q_num_heads, kv_num_heads
        self.qk_head_dim, self.v_head_dim = qk_head_dim, v_head_dim
        self.scale = float(scale)
        self.window_left = int(window_left)
        self.rope_mode = rope_mode
        self.num_splits = int(num_splits)
        if not (k_descale > 0.0 and v_descale > 0.0 and math.isfinite(k_descale) and math.isfinite(v_descale)):
            raise ValueError("k_descale and v_descale must be positive and finite")
        self.k_descale, self.v_descale = float(k_descale), float(v_descale)
        self.workspace = fmha.DecodeWorkspace()

    def _check_cache(self, q, k_cache, v_cache):
        if q.shape[-2] != self.q_num_heads or q.shape[-1] != self.qk_head_dim:
            raise ValueError(f"q has heads x dim {tuple(q.shape[-2:])}, module expects ({self.q_num_heads}, {self.qk_head_dim})")
        if k_cache.dim() != 4 or k_cache.shape[2] != self.kv_num_heads or k_cache.shape[3] != self.qk_head_dim:
            raise ValueError(f"k_cache must be [pages, page_size, {self.kv_num_heads}, {self.qk_head_dim}], got {tuple(k_cache.shape)}")
        if v_cache.dim() != 4 or v_cache.shape[2] != self.kv_num_heads or v_cache.shape[3] != self.v_head_dim:
            raise ValueError(f"v_cache must be [pages, page_size, {self.kv_num_heads}, {self.v_head_dim}], got {tuple(v_cache.shape)}")

    def prefill(self, q, k_cache, v_cache, cu_seqlens_q, *, kv_indptr=None, kv_page_indices=None, kv_last_page_lens=None,
                seqlen_k=None, block_table=None, max_seqlen_q: int = 0):
        """Varlen causal attention of packed prompts q [total_q, Hq, D]; K/V addressed by a page list
        (kv_indptr / kv_page_indices / kv_last_page_lens) or by a block table with seqlen_k."""
        self._check_cache(q, k_cache, v_cache)
        window = (self.window_left, 0)
        if kv_indptr is not None:
            return fmha.fmha_batch_prefill(q, k_cache, v_cache, cu_seqlens_q, kv_indptr, kv_page_indices, kv_last_page_lens,
                                           max_seqlen_q=max_seqlen_q, scale=self.scale, mask_type=fmha.MASK_BOTTOM_RIGHT,
                                           window=window, k_descale=self.k_descale, v_descale=self.v_descale)
        if block_table is None or seqlen_k is None:
            raise ValueError("prefill needs either kv_indptr/kv_page_indices or block_table/seqlen_k")
        return fmha.fmha_fwd_pagedkv(q, k_cache, v_cache, seqlen_k, block_table, cu_seqlens_q=cu_seqlens_q,
                                     max_seqlen_q=max_seqlen_q, scale=self.scale, mask_type=fmha.MASK_BOTTOM_RIGHT,
                                     window=window, k_descale=self.k_descale, v_descale=self.v_descale)

    def decode_step(self, q, knew, vnew, k_cache, v_cache, seqlen_k, block_table, *, cu_seqlens_knew=None,
                    max_seqlen_knew: int = 0, rotary_cos=None, rotary_sin=None, max_seqlen_k: int = 0, out=None):
        """Append knew/vnew behind seqlen_k[b] tokens (rotating knew and q), attend from the new tokens.
        Returns (o, seqlen_k_new); see `fmha_decode_step`."""
        self._check_cache(q, k_cache, v_cache)
        return fmha.fmha_decode_step(q, knew, vnew, k_cache, v_cache, seqlen_k, block_table,
                                     cu_seqlens_knew=cu_seqlens_knew, max_seqlen_knew=max_seqlen_knew,
                                     rotary_cos=rotary_cos, rotary_sin=rotary_sin, rope_mode=self.rope_mode,
                                     num_splits=self.num_splits, max_seqlen_k=max_seqlen_k, scale=self.scale,
                                     window_left=self.window_left, workspace=self.workspace, out=out,
                                     k_descale=self.k_descale, v_descale=self.v_descale)

    def extra_repr(self) -> str:
        return (f"q_num_heads={self.q_num_heads}, kv_num_heads={self.kv_num_heads}, qk_head_dim={self.qk_head_dim}, "
                f"v_head_dim={self.v_head_dim}, scale={self.scale}, window_left={self.window_left}, "
                f"rope_mode={self.rope_mode}, num_splits={self.num_splits}, k_descale={self.k_descale}, v_descale={self.v_descale}")
