"""Host model of every global -> LDS request the two direct-to-LDS prefill kernels issue (prefill_pingpong.hip at head
dims 64 / 128, prefill_dma.hip at head dim 256): 64-bit tile base + 32-bit per-lane byte offset, the row clamp on the
last tile of a sequence and the re-requests past the last tile.

For every workload the GPU tests run through these kernels (and for config 5 at full size) it asserts, for every
workgroup, wave, instruction and lane:
  * 0 <= address and address + 16 <= bytes of the pool (no request can fault);
  * the 32-bit quantities the kernels compute (row * row_stride + chunk, table[pi] * page_size, the byte offset) do not
    overflow;
  * the LDS destination lies inside the ring the request names;
  * the swizzle applied on the global side is the inverse of the one the LDS reads apply, i.e. every (row, chunk) of a
    tile lands exactly once where its reader expects it.
The formulas restate the kernels' address arithmetic; they are kept in step with it by name (cp_row, cp_k, cp_v, room,
row0, tile) - a change there must be made here, and the GPU parity tests then cover the data path end to end.
"""
import numpy as np
import pytest
import torch

from flashck_amd import generators as gen

BM, BN, RING, XCD = 256, 64, 4, 8
PAGE_CACHE = 4096          # kPrefillPageCache


def k_swz(D, row):
    return (row & 15) if D >= 128 else (((row & 7) + ((row >> 3) & 1)) & 7)


def v_swz(D, row, lc):
    return (((row & 3) << 1) ^ (((lc >> 1) & 1) << 3)) if D >= 128 else ((row & 3) << 1)


def copy_lanes(D):
    """(cp_row, cp_k, cp_v, lds_off) for every (wave, u, lane): what lane l of instruction u of wave w fetches."""
    ROWB, TILEB = D * 2, BN * D * 2
    LD = TILEB // 1024 // 8
    wave, u, lane = np.meshgrid(np.arange(8), np.arange(LD), np.arange(64), indexing="ij")
    off = (wave + 8 * u) * 1024 + lane * 16
    row = off // ROWB
    pc = (off % ROWB) >> 4
    cp_k = (pc ^ np.vectorize(lambda r: k_swz(D, r))(row)) * 8
    t = pc ^ ((row & 3) << 1)
    cp_v = np.where(D >= 128, t ^ (((t >> 1) & 1) << 3), t) * 8
    return row.ravel(), cp_k.ravel(), cp_v.ravel(), off.ravel()


@pytest.mark.parametrize("D", [64, 128])
def test_global_side_swizzle_is_the_inverse_of_the_read_side(D):
    """Every (row, logical chunk) of a tile is fetched exactly once, into the LDS place its reader computes."""
    CH = D // 8
    row, cp_k, cp_v, off = copy_lanes(D)
    assert sorted(off.tolist()) == list(range(0, BN * D * 2, 16)), "the 8 waves fill the tile exactly once"
    # K reader: row r, logical chunk lc at physical chunk lc ^ k_swz(r)
    placed = {(int(r), int(c) // 8): int(o) for r, c, o in zip(row, cp_k, off)}
    assert len(placed) == BN * CH
    for r in range(BN):
        for lc in range(CH):
            assert placed[(r, lc)] == r * D * 2 + ((lc ^ k_swz(D, r)) << 4)
    # V reader: row r, logical chunk lc at physical chunk lc ^ v_swz(r, lc)
    placed = {(int(r), int(c) // 8): int(o) for r, c, o in zip(row, cp_v, off)}
    assert len(placed) == BN * CH
    for r in range(BN):
        for lc in range(CH):
            assert placed[(r, lc)] == r * D * 2 + ((lc ^ v_swz(D, r, lc)) << 4)


class Pool:
    def __init__(self, w, D):
        self.D = D
        self.hk = w["k_cache"].shape[2]
        self.page = w["k_cache"].shape[1]
        self.pool_bytes = w["k_cache"].numel() * 2
        self.row_stride = self.hk * D          # elements
        self.hq = w["q"].shape[-2]
        self.lens = list(w["lens"])
        self.indptr = w["kv_indptr"].tolist()
        self.indices = w["kv_page_indices"].numpy().astype(np.int64)
        assert BN * self.row_stride * 2 < 2 ** 31, "64 cache rows must span < 2 GiB (guarded in fmha_api.cpp)"
        assert int(self.indices.max() + 1) * self.page < 2 ** 31, "first rows are kept as int32"

    def first_rows(self, b, t_begin, n):
        """row_lds[i]: first cache row of tile t_begin + i of sequence b (uniform pages: a tile never straddles a page)."""
        kb = (t_begin + np.arange(n, dtype=np.int64)) * BN
        pi = kb // self.page
        table = self.indices[self.indptr[b]:self.indptr[b + 1]]
        assert pi.max(initial=0) < len(table), "tile past the sequence's page list"
        return table[pi] * self.page + (kb - pi * self.page)


def check_requests(pool, b, hkv, t_begin, tiles, lanes):
    """Every request for local tiles `tiles` (numpy array, may repeat) of sequence b, KV head hkv."""
    if len(tiles) == 0:
        return 0
    cp_row, cp_k, cp_v, _ = lanes
    sk = pool.lens[b]
    n_all = (sk + BN - 1) // BN - t_begin
    assert tiles.min() >= 0 and tiles.max() < n_all, "request for a tile the sequence does not have"
    row0 = pool.first_rows(b, t_begin, int(tiles.max()) + 1)[tiles]
    room = sk - 1 - (t_begin + tiles) * BN
    assert room.min() >= 0
    tb = (row0 * pool.row_stride + hkv * pool.D) * 2                      # 64-bit scalar base, bytes
    for cp_c in (cp_k, cp_v):
        # whole tiles share one offset pattern; the (at most one) ragged tile gets its own
        lo_whole = int((cp_row * pool.row_stride + cp_c).min()) * 2
        hi_whole = int((cp_row * pool.row_stride + cp_c).max()) * 2
        assert hi_whole < 2 ** 32
        whole = room >= BN - 1
        if whole.any():
            assert (tb[whole] + lo_whole).min() >= 0 and (tb[whole] + hi_whole + 16).max() <= pool.pool_bytes
        for tbi, rm in zip(tb[~whole], room[~whole]):
            off = (np.minimum(cp_row, rm) * pool.row_stride + cp_c) * 2
            assert off.max() < 2 ** 32 and tbi + off.min() >= 0 and tbi + off.max() + 16 <= pool.pool_bytes
    return len(tiles)


def causal_range(sq, sk, m0):
    """tiles [t_begin, t_end) a 256-row workgroup at row m0 (negative for a ragged first tile: row tiles are aligned to
    the end of the sequence) walks under the bottom-right causal mask"""
    last_row = min(m0 + BM, sq) - 1
    hi = min(sk, last_row + 1 + sk - sq)
    return 0, max(0, (hi + BN - 1) // BN)


def pingpong_workgroups(pool):
    """(b, hkv, t_begin, n) of every workgroup of the ping-pong kernel's 1-D grid, in grid order"""
    g = pool.hq // pool.hk
    groups = len(pool.lens) * pool.hk
    gx = (groups + XCD - 1) // XCD
    m_tiles = (max(pool.lens) + BM - 1) // BM
    for bid in range(XCD * m_tiles * gx * g):
        xcd, slot = bid % XCD, bid // XCD
        gk, mt = (slot // g) % gx, m_tiles - 1 - slot // (g * gx)
        gid = gk * XCD + xcd
        if gid >= groups:
            continue
        b, hkv = gid // pool.hk, gid % pool.hk
        tiles_b = (pool.lens[b] + BM - 1) // BM
        if mt >= tiles_b:
            continue
        t_begin, t_end = causal_range(pool.lens[b], pool.lens[b], mt * BM - (tiles_b * BM - pool.lens[b]))
        yield b, hkv, t_begin, t_end - t_begin


def run_pingpong(pool, lanes):
    total = 0
    for b, hkv, t_begin, n in pingpong_workgroups(pool):
        if n <= 0:
            continue
        # prologue requests tiles 0, 1, 2; iteration i requests K_{i+3} and V_{i+2}; past the end: the last tile again
        want = np.concatenate([np.arange(3), np.arange(n - 1) + 3, np.arange(2), np.arange(n - 1) + 2])
        total += check_requests(pool, b, hkv, t_begin, np.minimum(want, n - 1), lanes)
    return total


WORKLOADS = {
    # the GPU tests that run this kernel: tests/test_gpu_prefill.py and tests/test_gpu_prefill_grid.py, then config 5
    "midsize_every_row_d128": dict(lens=[5000, 300], hq=2, hk=1, head_dim=128),
    "midsize_every_row_d64": dict(lens=[5000, 300], hq=2, hk=1, head_dim=64),
    "small_page64": dict(seed=50 + 128 + 64, batch=5, hq=4, hk=2, head_dim=128, min_len=1, max_len=400, page_size=64),
    "small_page128_d64": dict(seed=50 + 64 + 128, batch=5, hq=4, hk=2, head_dim=64, min_len=1, max_len=400, page_size=128),
    "ragged": dict(lens=[1, 63, 64, 65, 255, 256, 257, 511, 513, 1024, 1500], hq=4, hk=2, head_dim=128),
    "config5_d128": dict(head_dim=128),
}


@pytest.mark.parametrize("name", list(WORKLOADS))
def test_every_request_stays_inside_the_pool(name):
    kw = dict(WORKLOADS[name])
    # the address arithmetic does not depend on the tensor contents: build the page layout only
    w = layout_only(**kw)
    pool = Pool(w, kw.get("head_dim", 128))
    lanes = copy_lanes(pool.D)
    assert run_pingpong(pool, lanes) > 0


def layout_only(seed=gen.BASE_SEED + 5, batch=16, hq=32, hk=8, head_dim=128, min_len=128, max_len=8192, page_size=128,
                lens=None):
    """workload_varlen_prefill's page layout without the tensor data (same generator order for the lengths and pages)"""
    g = torch.Generator().manual_seed(seed)
    lens = list(lens) if lens is not None else gen.randint_list(min_len, max_len, batch, g)
    table, pool = gen.paged_layout(lens, page_size, g)
    pages = [-(-l // page_size) for l in lens]
    indptr = torch.zeros(len(lens) + 1, dtype=torch.int32)
    indptr[1:] = torch.tensor(pages).cumsum(0)
    indices = torch.cat([table[b, :pages[b]] for b in range(len(lens))]).contiguous()
    return dict(k_cache=torch.empty(pool, page_size, hk, head_dim, dtype=torch.bfloat16, device="meta"),
                q=torch.empty(sum(lens), hq, head_dim, dtype=torch.bfloat16, device="meta"), lens=lens, kv_indptr=indptr,
                kv_page_indices=indices)


def test_the_model_rejects_wrong_address_arithmetic():
    """Teeth: a row stride taken from the query heads instead of the KV heads, or a page id used as a row, sends
    requests outside the pool and is caught."""
    w = layout_only(lens=[700, 300], hq=8, hk=2, head_dim=128)
    lanes = copy_lanes(128)
    pool = Pool(w, 128)
    assert run_pingpong(pool, lanes) > 0
    pool.row_stride = pool.hq * pool.D          # the mistake
    with pytest.raises(AssertionError):
        run_pingpong(pool, lanes)
    pool = Pool(w, 128)
    pool.page = pool.page * 2                    # first row = page id * wrong page size
    with pytest.raises(AssertionError):
        run_pingpong(pool, lanes)


# ---------------------------------------------------------------------------------------------------------------------
# prefill_dma.hip (head dim 256): 4 waves, 128-row workgroups, two buffers per operand; wave w fills the 1 KiB blocks
# w, w+4, ... of a tile (two rows each), so three offset registers serve all 16 instructions of a tile and the 8u rows
# of block u go into the scalar base when every row of the tile exists.
# ---------------------------------------------------------------------------------------------------------------------
DMA_BM, DMA_D, DMA_LD = 128, 256, 64 * 512 // 1024 // 4


def dma_lanes():
    """(cp_row0, cp_pc, cp_kc0, cp_kc1, cp_vc) for every (wave, lane) of the 4-wave kernel"""
    wave, lane = np.meshgrid(np.arange(4), np.arange(64), indexing="ij")
    cp_row0 = wave * 2 + (lane >> 5)
    cp_pc = lane & 31
    cp_kc0 = (cp_pc ^ (cp_row0 & 15)) * 8
    cp_kc1 = (cp_pc ^ ((cp_row0 + 8) & 15)) * 8
    t = cp_pc ^ ((cp_row0 & 3) << 1)
    cp_vc = (t ^ (((t >> 1) & 1) << 3)) * 8
    return wave.ravel(), lane.ravel(), cp_row0.ravel(), cp_kc0.ravel(), cp_kc1.ravel(), cp_vc.ravel()


def test_dma_kernel_swizzle_is_the_inverse_of_the_read_side():
    """The three offset registers are enough: block w + 4u holds rows cp_row0 + 8u, whose K swizzle alternates with the
    parity of u and whose V swizzle does not depend on u; every (row, chunk) lands once where its reader looks."""
    D, CH = DMA_D, DMA_D // 8
    wave, lane, cp_row0, kc0, kc1, vc = dma_lanes()
    k_placed, v_placed, offs = {}, {}, []
    for u in range(DMA_LD):
        lds_off = (wave + 4 * u) * 1024 + lane * 16
        row = cp_row0 + 8 * u
        assert (lds_off // 512 == row).all() and ((lds_off % 512) >> 4 == (lane & 31)).all()
        kc = kc1 if u & 1 else kc0
        for r, ck, cv, o in zip(row, kc, vc, lds_off):
            k_placed[(int(r), int(ck) // 8)] = int(o)
            v_placed[(int(r), int(cv) // 8)] = int(o)
        offs += lds_off.tolist()
    assert sorted(offs) == list(range(0, BN * D * 2, 16)), "the 4 waves fill the tile exactly once"
    assert len(k_placed) == BN * CH and len(v_placed) == BN * CH
    for r in range(BN):
        for lc in range(CH):
            assert k_placed[(r, lc)] == r * 512 + ((lc ^ k_swz(D, r)) << 4)
            assert v_placed[(r, lc)] == r * 512 + ((lc ^ v_swz(D, r, lc)) << 4)


def dma_workgroups(pool):
    """(b, hkv, t_begin, n) of every workgroup of the DMA kernel's 1-D grid (128-row tiles aligned to the sequence end)"""
    g = pool.hq // pool.hk
    groups = len(pool.lens) * pool.hk
    gx = (groups + XCD - 1) // XCD
    m_tiles = (max(pool.lens) + DMA_BM - 1) // DMA_BM
    for bid in range(XCD * m_tiles * gx * g):
        xcd, slot = bid % XCD, bid // XCD
        gk, mt = (slot // g) % gx, m_tiles - 1 - slot // (g * gx)
        gid = gk * XCD + xcd
        if gid >= groups:
            continue
        b, hkv = gid // pool.hk, gid % pool.hk
        sq = pool.lens[b]
        tiles_b = (sq + DMA_BM - 1) // DMA_BM
        if mt >= tiles_b:
            continue
        m0 = mt * DMA_BM - (tiles_b * DMA_BM - sq)
        last_row = min(m0 + DMA_BM, sq) - 1
        yield b, hkv, 0, max(0, (min(sq, last_row + 1) + BN - 1) // BN)


def run_dma(pool):
    wave, lane, cp_row0, kc0, kc1, vc = dma_lanes()
    total = 0
    for b, hkv, t_begin, n in dma_workgroups(pool):
        if n <= 0:
            continue
        sk = pool.lens[b]
        tiles = np.arange(n)                                    # request(0), then request(i + 1) while i + 1 < n
        row0 = pool.first_rows(b, t_begin, n)
        room = sk - 1 - (t_begin + tiles) * BN
        assert room.min() >= 0
        tile_off = row0 * pool.row_stride + hkv * pool.D        # elements
        for u in range(DMA_LD):
            for chunk in ((kc1 if u & 1 else kc0), vc):
                # whole tiles: rows 8u.. go into the scalar base, the lane offset is cp_row0 * row_stride + chunk
                off_whole = (cp_row0 * pool.row_stride + chunk) * 2
                assert off_whole.max() < 2 ** 32
                whole = room >= BN - 1
                if whole.any():
                    tb = (tile_off[whole] + 8 * u * pool.row_stride) * 2
                    assert tb.min() + off_whole.min() >= 0 and tb.max() + off_whole.max() + 16 <= pool.pool_bytes
                for t_off, rm in zip(tile_off[~whole], room[~whole]):
                    off = (np.minimum(cp_row0 + 8 * u, rm) * pool.row_stride + chunk) * 2
                    assert off.max() < 2 ** 32 and t_off * 2 + off.min() >= 0 and t_off * 2 + off.max() + 16 <= pool.pool_bytes
        total += n
    return total


DMA_WORKLOADS = {
    "midsize_every_row_d256": dict(lens=[5000, 300], hq=2, hk=1, head_dim=256),
    "small_page64_d256": dict(seed=50 + 256 + 64, batch=5, hq=4, hk=2, head_dim=256, min_len=1, max_len=400, page_size=64),
    "ragged_d256": dict(lens=[1, 63, 64, 65, 127, 128, 129, 255, 257, 513, 1024, 1500], hq=4, hk=2, head_dim=256),
    "config5_d256": dict(head_dim=256),
}


@pytest.mark.parametrize("name", list(DMA_WORKLOADS))
def test_every_request_of_the_dma_kernel_stays_inside_the_pool(name):
    kw = dict(DMA_WORKLOADS[name])
    pool = Pool(layout_only(**kw), 256)
    assert run_dma(pool) > 0


def test_the_dma_model_rejects_wrong_address_arithmetic():
    pool = Pool(layout_only(lens=[700, 300], hq=8, hk=2, head_dim=256), 256)
    assert run_dma(pool) > 0
    pool.row_stride = pool.hq * pool.D          # the mistake: query heads instead of KV heads
    with pytest.raises(AssertionError):
        run_dma(pool)
