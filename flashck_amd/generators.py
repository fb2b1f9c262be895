"""Seeded synthetic inputs for the FMHA operators.

Counterpart of the data generators in FlashCK's profiler harness (seeded sequence lengths, `iota_shuffle`
block tables, rotary tables: core/module/kernels/attention_kernels/fmha_common_jinja.h:191-229,259-343,460-470 and
fmha_fwd_split_kv_jinja.h:549-557).  Everything is drawn on the CPU from ``torch.Generator().manual_seed(seed)``
in fp32 and rounded once to the data type, so a CPU checker and the GPU see the same bits.  The default base seed is
FlashCK's FC_TUNING_SEED = 42 (core/utils/flags.cc:225); workload k uses 42 + k.
"""
import math
from typing import List, Optional, Sequence

import torch

BASE_SEED = 42


def _gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def randn(shape, dtype, g):
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


def rotary_tables(max_pos: int, rotary_dim: int, dtype, base: float = 10000.0):
    """cos/sin [max_pos, rotary_dim/2] in `dtype`; angle(pos, i) = pos * base^(-2i/rotary_dim), evaluated in fp64."""
    i = torch.arange(rotary_dim // 2, dtype=torch.float64)
    inv = base ** (-2.0 * i / rotary_dim)
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    return torch.cos(ang).to(dtype).contiguous(), torch.sin(ang).to(dtype).contiguous()


def paged_layout(lens: Sequence[int], page_size: int, g, slack: float = 0.10, capacity: Optional[Sequence[int]] = None,
                 shuffle: bool = True):
    """Shuffled block table: sequence b takes consecutive entries of a random permutation of the pool.

    Returns (block_table int32 [B, max_pages], num_pool_pages).  `capacity` (>= lens) reserves pages for growth.
    """
    cap = list(capacity) if capacity is not None else list(lens)
    pages = [max(1, -(-c // page_size)) for c in cap]
    total = sum(pages)
    pool = int(math.ceil(total * (1.0 + slack)))
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    if not shuffle:
        perm = torch.arange(pool, dtype=torch.int32)
    table = torch.zeros(len(lens), max(pages), dtype=torch.int32)
    at = 0
    for b, n in enumerate(pages):
        table[b, :n] = perm[at:at + n]
        at += n
    return table, pool


def scatter_to_pages(rows: List[torch.Tensor], table: torch.Tensor, pool: int, page_size: int, fill=float("nan")):
    """rows[b]: [L_b, Hk, D] -> cache [pool, page_size, Hk, D]; every slot not written holds `fill`."""
    hk, d = rows[0].shape[1], rows[0].shape[2]
    cache = torch.full((pool, page_size, hk, d), fill, dtype=rows[0].dtype)
    flat = cache.view(pool * page_size, hk, d)
    for b, r in enumerate(rows):
        n = r.shape[0]
        if n == 0:
            continue
        t = torch.arange(n)
        phys = table[b, t // page_size].to(torch.int64) * page_size + t % page_size
        flat[phys] = r
    return cache


def paged_kv(lens, hk, d, dtype, g, page_size=128, slack=0.10, capacity=None, shuffle=True, dv=None):
    """Random K/V for sequences of the given lengths, stored in a shuffled paged cache with NaN in unused slots
    (dv: head dim of V when it differs from K's)."""
    table, pool = paged_layout(lens, page_size, g, slack, capacity, shuffle)
    k_rows = [randn((n, hk, d), dtype, g) for n in lens]
    v_rows = [randn((n, hk, dv or d), dtype, g) for n in lens]
    k_cache = scatter_to_pages(k_rows, table, pool, page_size)
    v_cache = scatter_to_pages(v_rows, table, pool, page_size)
    return dict(k_cache=k_cache, v_cache=v_cache, block_table=table, k_rows=k_rows, v_rows=v_rows,
                seqlen_k=torch.tensor(list(lens), dtype=torch.int32), page_size=page_size)


def randint_list(lo, hi_inclusive, n, g):
    return torch.randint(lo, hi_inclusive + 1, (n,), generator=g).tolist()


# ---------------------------------------------------------------------------------------------------------------
# The five benchmark workloads (sizes can be scaled down for CPU-checked tests through the keyword arguments).
# ---------------------------------------------------------------------------------------------------------------

def workload_dense_fp16(seed=BASE_SEED + 1, batch=2, seqlen=128, heads=8, head_dim=64):
    """1: FMHA forward, non-causal, fp16, contiguous BSHD."""
    g = _gen(seed)
    q = randn((batch, seqlen, heads, head_dim), torch.float16, g)
    k = randn((batch, seqlen, heads, head_dim), torch.float16, g)
    v = randn((batch, seqlen, heads, head_dim), torch.float16, g)
    return dict(q=q, k=k, v=v, scale=1.0 / math.sqrt(head_dim))


def workload_paged_decode(seed=BASE_SEED + 2, batch=32, hq=32, hk=8, head_dim=128, min_len=512, max_len=4096,
                          page_size=128, dtype=torch.bfloat16):
    """2: paged-KV decode, GQA, q_len = 1, KV lengths ~ U[min_len, max_len], pool with 10 % slack."""
    g = _gen(seed)
    lens = randint_list(min_len, max_len, batch, g)
    kv = paged_kv(lens, hk, head_dim, dtype, g, page_size)
    kv["q"] = randn((batch, 1, hq, head_dim), dtype, g)
    kv["scale"] = 1.0 / math.sqrt(head_dim)
    kv["lens"] = lens
    return kv


def workload_splitkv_decode(seed=BASE_SEED + 3, batch=4, hq=64, hk=8, head_dim=128, kv_len=32768, page_size=128,
                            num_splits=8, dtype=torch.bfloat16, shuffle=True):
    """3: split-KV long-context decode, fixed KV length, shuffled pages, num_splits partials + combine."""
    g = _gen(seed)
    lens = [kv_len] * batch
    kv = paged_kv(lens, hk, head_dim, dtype, g, page_size, shuffle=shuffle)
    kv["q"] = randn((batch, 1, hq, head_dim), dtype, g)
    kv["scale"] = 1.0 / math.sqrt(head_dim)
    kv["num_splits"] = num_splits
    kv["lens"] = lens
    return kv


def workload_appendkv_decode(seed=BASE_SEED + 4, batch=16, hq=32, hk=8, head_dim=128, min_len=1024, max_len=8192,
                             max_new=16, page_size=128, dtype=torch.bfloat16, rope_base=10000.0):
    """4: appendKV + RoPE (1..max_new new tokens per sequence at absolute positions) into shuffled pages."""
    g = _gen(seed)
    lens = randint_list(min_len, max_len, batch, g)
    new = randint_list(1, max_new, batch, g)
    cap = [l + n for l, n in zip(lens, new)]
    kv = paged_kv(lens, hk, head_dim, dtype, g, page_size, capacity=cap)
    total_new = sum(new)
    cu = torch.zeros(batch + 1, dtype=torch.int32)
    cu[1:] = torch.tensor(new).cumsum(0)
    cos, sin = rotary_tables(max(cap) + 1, head_dim, dtype, rope_base)
    kv.update(q=randn((total_new, hq, head_dim), dtype, g), knew=randn((total_new, hk, head_dim), dtype, g),
              vnew=randn((total_new, hk, head_dim), dtype, g), cu_seqlens_knew=cu, new=new, lens=lens,
              rotary_cos=cos, rotary_sin=sin, max_new=max(new), scale=1.0 / math.sqrt(head_dim))
    return kv


def workload_varlen_prefill(seed=BASE_SEED + 5, batch=16, hq=32, hk=8, head_dim=128, min_len=128, max_len=8192,
                            page_size=128, dtype=torch.bfloat16, lens=None, v_head_dim=None):
    """5: varlen causal batch prefill, sq = sk = L_b packed by cu_seqlens, K/V in a shuffled paged cache.
    `lens` fixes the lengths instead of drawing them; `v_head_dim` is the head dim of V when it differs from Q / K's."""
    g = _gen(seed)
    lens = list(lens) if lens is not None else randint_list(min_len, max_len, batch, g)
    batch = len(lens)
    kv = paged_kv(lens, hk, head_dim, dtype, g, page_size, dv=v_head_dim)
    cu = torch.zeros(batch + 1, dtype=torch.int32)
    cu[1:] = torch.tensor(lens).cumsum(0)
    total = int(cu[-1])
    pages = [-(-l // page_size) for l in lens]
    indptr = torch.zeros(batch + 1, dtype=torch.int32)
    indptr[1:] = torch.tensor(pages).cumsum(0)
    indices = torch.cat([kv["block_table"][b, :pages[b]] for b in range(batch)]).contiguous()
    last = torch.tensor([l - (p - 1) * page_size for l, p in zip(lens, pages)], dtype=torch.int32)
    kv.update(q=randn((total, hq, head_dim), dtype, g), cu_seqlens_q=cu, kv_indptr=indptr, kv_page_indices=indices,
              kv_last_page_lens=last, lens=lens, max_seqlen_q=max(lens), scale=1.0 / math.sqrt(head_dim))
    return kv


# ---------------------------------------------------------------------------------------------------------------
# algorithmic work of a call (what the roofline figures are computed from)
# ---------------------------------------------------------------------------------------------------------------

def decode_bytes(lens, q_lens, hq, hk, d, dv, page_size, elem=2, kv_elem=None):
    """K and V once, Q in, O out, block-table entries and sequence lengths; fp32 workspace traffic excluded.
    kv_elem: bytes per K/V element when the cache type differs from the Q/O type (1 for an fp8 cache)."""
    kv = sum(lens) * hk * (d + dv) * (elem if kv_elem is None else kv_elem)
    qo = sum(q_lens) * hq * (d + dv) * elem
    idx = 4 * (sum(-(-l // page_size) for l in lens) + len(lens))
    return kv + qo + idx


def decode_flops(lens, q_lens, hq, d, dv):
    return 2 * sum(q * l for q, l in zip(q_lens, lens)) * hq * (d + dv)


def causal_pairs(sq, sk):
    """Visible (query, key) pairs under the bottom-right causal rule j <= i + sk - sq."""
    return sum(max(0, min(sk, i + 1 + sk - sq)) for i in range(sq))


def prefill_flops(lens, hq, d, dv, causal=True):
    pairs = sum(causal_pairs(l, l) if causal else l * l for l in lens)
    return 2 * hq * (d + dv) * pairs


def prefill_bytes(lens, hq, hk, d, dv, elem=2):
    return sum(lens) * (hq * (d + dv) + hk * (d + dv)) * elem
