"""Host model of every K/V load the split-KV decode kernel issues (splitkv_decode.hip): which cache element lane l of
load instruction u of tile c of wave w reads, for one KV head per workgroup and for head pairs, for padded head dims,
on the uniform-page path (one first row per tile) and on the per-row lookup path, including the clamps (rows past the
last key repeat it, claims past the last tile re-read it).

Asserted for every workgroup of a set of workloads (the GPU tests' shapes, scaled):
  * every load lies inside the cache it reads (no request can fault) and reads a row the sequence owns (a row of one of
    its pages, a key below its length): a load of a foreign or unused slot could not fault, but it would be wrong;
  * the lanes of one instruction cover whole 16-byte pieces of the head group's part of a token row, each exactly once
    per key of the tile, so the staged tile is complete;
  * the pieces a padded head dim does not have are never loaded.
The formulas restate the kernel's address arithmetic (src_off, tile_row0, ld_key, ld_piece, claim); the GPU parity tests
cover the data path end to end.
"""
import numpy as np
import pytest
import torch

from flashck_amd import generators as gen


def shape(D, HG):
    TK = 32 // HG
    LPR = D // 8
    LPT = LPR * HG
    KPI = 64 // LPT
    return dict(TK=TK, LPR=LPR, LPT=LPT, KPI=KPI, VN=TK // KPI)


class Cache:
    def __init__(self, lens, hk, d, dv, page, seed=3):
        g = torch.Generator().manual_seed(seed)
        self.table, self.pool = gen.paged_layout(lens, page, g)
        self.table = self.table.numpy().astype(np.int64)
        self.lens, self.hk, self.d, self.dv, self.page = list(lens), hk, d, dv, page
        self.k_elems = self.pool * page * hk * d
        self.v_elems = self.pool * page * hk * dv

    def row(self, b, key):
        return self.table[b, key // self.page] * self.page + key % self.page


def workgroup_loads(cache, D, HG, NW, num_splits, b, hgrp, split, uniform):
    """yields (operand, element offsets [64 lanes], valid mask, keys [64]) for every load instruction of the workgroup"""
    S = shape(D, HG)
    pad = cache.d != D or cache.dv != D
    sk = cache.lens[b]
    per = max(1, -(-sk // num_splits))
    k0 = min(per * split, sk)
    k1 = min(k0 + per, sk)
    t_begin, t_end = k0 // S["TK"], -(-k1 // S["TK"])
    n_tiles = t_end - t_begin
    if n_tiles <= 0 or sk == 0:
        return
    lane = np.arange(64)
    ld_key, ld_piece = lane // S["LPT"], lane % S["LPT"]
    hkv0 = hgrp * HG
    last_key = sk - 1
    for wave in range(NW):
        # the wave claims tiles wave, wave + NW, ... and two more past the end of its share (requested, clamped, unused)
        claims = list(range(wave, n_tiles, NW))
        if not claims:
            continue
        for c in claims:
            kb = (t_begin + c) * S["TK"]
            for u in range(S["VN"]):
                key = np.minimum(kb + u * S["KPI"] + ld_key, last_key)
                if uniform:
                    # one first row per tile; rows past the last key repeat it
                    row0 = cache.row(b, kb)
                    kl = np.minimum(u * S["KPI"] + ld_key, last_key - kb)
                    rows = row0 + kl
                    assert kb // cache.page == (kb + S["TK"] - 1) // cache.page, "a tile straddles a page"
                else:
                    rows = np.array([cache.row(b, int(k)) for k in key])
                for name, dim in (("k", cache.d), ("v", cache.dv)):
                    off = (rows * cache.hk + hkv0) * dim + ld_piece * 8
                    valid = (ld_piece * 8 < dim) if pad else np.ones(64, bool)
                    yield name, off, valid, key, rows


def check(cache, D, HG, NW, num_splits, uniform):
    S = shape(D, HG)
    ng = cache.hk // HG
    loads = 0
    for b in range(len(cache.lens)):
        own_rows = set()
        for key in range(cache.lens[b]):
            own_rows.add(int(cache.row(b, key)))
        for hgrp in range(ng):
            for split in range(num_splits):
                seen = {"k": {}, "v": {}}
                for name, off, valid, key, rows in workgroup_loads(cache, D, HG, NW, num_splits, b, hgrp, split, uniform):
                    dim = cache.d if name == "k" else cache.dv
                    total = cache.k_elems if name == "k" else cache.v_elems
                    o = off[valid]
                    assert o.min() >= 0 and o.max() + 8 <= total, "load outside the cache"
                    assert set(rows[valid].tolist()) <= own_rows, "load of a row the sequence does not own"
                    assert (key < cache.lens[b]).all()
                    # a piece stays inside its head's row: [head * dim, (head + 1) * dim) for one of the group's heads
                    inner = o % (cache.hk * dim) - hgrp * HG * dim
                    assert (inner >= 0).all() and (inner + 8 <= HG * dim).all()
                    for k_, o_ in zip(key[valid], o):
                        seen[name].setdefault(int(k_), set()).add(int(o_))
                    loads += 1
                # every key of the split was staged completely (all pieces of the head group's part of its row)
                sk = cache.lens[b]
                per = max(1, -(-sk // num_splits))
                k0, k1 = min(per * split, sk), min(min(per * split, sk) + per, sk)
                for name, dim in (("k", cache.d), ("v", cache.dv)):
                    for key in range(k0, k1):
                        assert len(seen[name].get(key, ())) == HG * dim // 8, (name, key)
    return loads


CASES = [
    # D, HG, NW, (d, dv), page, lens, num_splits, uniform
    (128, 1, 8, (128, 128), 128, [1, 33, 129, 700], 3, True),
    (128, 2, 8, (128, 128), 128, [1, 33, 129, 700], 2, True),
    (64, 2, 8, (64, 64), 64, [16, 257, 90], 4, True),
    (256, 1, 4, (256, 256), 32, [5, 300], 2, True),
    (128, 1, 8, (128, 128), 48, [1, 47, 49, 200], 3, False),     # page size not a multiple of the tile: per-row lookups
    (128, 1, 8, (96, 96), 32, [40, 333], 2, True),                # padded head dims
    (256, 1, 4, (192, 128), 64, [70, 260], 3, True),
    (64, 1, 8, (8, 40), 16, [3, 100], 2, False),
    (128, 1, 8, (128, 64), 128, [500], 8, True),                  # more splits than tiles in some ranges
]


@pytest.mark.parametrize("D,HG,NW,dims,page,lens,ns,uniform", CASES)
def test_every_load_reads_a_row_the_sequence_owns(D, HG, NW, dims, page, lens, ns, uniform):
    cache = Cache(lens, 4, dims[0], dims[1], page)
    assert check(cache, D, HG, NW, ns, uniform) > 0


def test_the_model_has_teeth():
    """A row stride taken from the padded head dim instead of the stored one walks out of the cache and into foreign rows."""
    cache = Cache([40, 333], 4, 96, 96, 32)
    assert check(cache, 128, 1, 8, 2, True) > 0
    cache.d = 128   # the mistake: addresses computed with the kernel's D while the cache rows are 96 elements wide
    with pytest.raises(AssertionError):
        check(cache, 128, 1, 8, 2, True)
