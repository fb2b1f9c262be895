"""The decode step (append -> split count -> split-KV -> combine) and the nn modules on the GPU, against the oracle."""
import pytest
import torch

from flashck_amd import generators as gen
import helpers
from helpers import assert_bits_equal, assert_close, dev

pytestmark = pytest.mark.gpu


def _expected(orc, w, rope_mode, window_left=-1):
    q, kc, vc = w["q"].clone(), w["k_cache"].clone(), w["v_cache"].clone()
    orc.appendkv(q, kc, vc, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], cos=w["rotary_cos"],
                 sin=w["rotary_sin"], rope_mode=rope_mode, has_mask=True, block_table=w["block_table"])
    sl = (w["seqlen_k"] + torch.tensor(w["new"], dtype=torch.int32)).contiguous()
    o = orc.fmha_fwd(q, kc, vc, seqstart_q=w["cu_seqlens_knew"], seqlen_k=sl, block_table=w["block_table"],
                     scale=w["scale"], mask_type=2, window=(window_left, 0))
    return o, q, kc, vc, sl


@pytest.mark.parametrize("num_splits", [0, 4])
def test_decode_step_packed(fmha, orc, num_splits):
    w = gen.workload_appendkv_decode(seed=71, batch=6, hq=8, hk=2, head_dim=128, min_len=0, max_len=700, max_new=9,
                                     page_size=64)
    ws = fmha.DecodeWorkspace()
    q, kc, vc = dev(w["q"].clone()), dev(w["k_cache"].clone()), dev(w["v_cache"].clone())
    sl = dev(w["seqlen_k"])
    ro, rq, rkc, rvc, rsl = _expected(orc, w, 2)
    for step in range(2):  # the second step reuses the workspace; inputs are restored so the result must repeat
        q.copy_(w["q"])
        kc.copy_(w["k_cache"])
        vc.copy_(w["v_cache"])
        o, sl_new = fmha.fmha_decode_step(q, dev(w["knew"]), dev(w["vnew"]), kc, vc, sl, dev(w["block_table"]),
                                          cu_seqlens_knew=dev(w["cu_seqlens_knew"]), max_seqlen_knew=w["max_new"],
                                          rotary_cos=dev(w["rotary_cos"]), rotary_sin=dev(w["rotary_sin"]), rope_mode=2,
                                          num_splits=num_splits, scale=w["scale"], workspace=ws)
        assert_bits_equal(q, rq, "rotated q")
        assert_bits_equal(kc, rkc, "k cache")
        assert_bits_equal(vc, rvc, "v cache")
        assert torch.equal(sl_new.cpu(), rsl)
        assert torch.equal(sl.cpu(), w["seqlen_k"])
        assert_close(o, ro, 2e-2, f"decode step {step}")


def test_paged_attention_module(fmha, orc):
    from flashck_amd.nn import PagedAttention
    # single new token per sequence, batch form, fp16
    g = torch.Generator().manual_seed(72)
    B, hq, hk, d, page = 5, 8, 4, 64, 16
    lens = [0, 15, 16, 333, 64]
    kv = gen.paged_kv(lens, hk, d, torch.float16, g, page, capacity=[l + 1 for l in lens])
    q = gen.randn((B, 1, hq, d), torch.float16, g)
    knew, vnew = gen.randn((B, 1, hk, d), torch.float16, g), gen.randn((B, 1, hk, d), torch.float16, g)
    m = PagedAttention(hq, hk, d)
    kc, vc = dev(kv["k_cache"].clone()), dev(kv["v_cache"].clone())
    o, sl_new = m.decode_step(dev(q), dev(knew), dev(vnew), kc, vc, dev(kv["seqlen_k"]), dev(kv["block_table"]))
    rkc, rvc = kv["k_cache"].clone(), kv["v_cache"].clone()
    cu = torch.arange(B + 1, dtype=torch.int32)
    orc.appendkv(None, rkc, rvc, knew.view(B, hk, d), vnew.view(B, hk, d), kv["seqlen_k"], cu, block_table=kv["block_table"])
    assert_bits_equal(kc, rkc, "k cache")
    assert_bits_equal(vc, rvc, "v cache")
    ro = orc.fmha_fwd(q, rkc, rvc, seqlen_k=(kv["seqlen_k"] + 1).contiguous(), block_table=kv["block_table"])
    assert_close(o, ro, 1e-2, "module decode step")
    assert torch.equal(sl_new.cpu(), kv["seqlen_k"] + 1)


def test_attention_module_dense(fmha, orc):
    from flashck_amd.nn import Attention
    w = gen.workload_dense_fp16()
    m = Attention(w["q"].shape[2], w["k"].shape[2], w["q"].shape[3], scale=w["scale"])
    o = m(dev(w["q"]), dev(w["k"]), dev(w["v"]))
    ro = orc.fmha_fwd(w["q"], w["k"], w["v"], scale=w["scale"])
    assert_close(o, ro, 1e-2, "Attention module, config 1")


def test_tuned_split_count_is_recorded_and_used(fmha, orc, tmp_path):
    import flashck_amd
    from flashck_amd.utils import tuning
    saved = {n: flashck_amd.get_flag_value(n) for n in ("FC_TUNING_DB_DIR", "FC_TUNING_NUM_COLD_ITERATION",
                                                          "FC_TUNING_NUM_REPEATS", "FC_TUNING_MODE")}
    old_default = tuning._default
    try:
        flashck_amd.set_flag_value("FC_TUNING_DB_DIR", str(tmp_path))
        flashck_amd.set_flag_value("FC_TUNING_NUM_COLD_ITERATION", "2")
        flashck_amd.set_flag_value("FC_TUNING_NUM_REPEATS", "5")
        flashck_amd.set_flag_value("FC_TUNING_MODE", "2")
        tuning._default = None
        w = gen.workload_paged_decode(seed=73, batch=4, hq=16, hk=4, head_dim=128, min_len=900, max_len=2000, page_size=64)
        q, kc, vc = dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"])
        sl, bt = dev(w["seqlen_k"]), dev(w["block_table"])
        rec = fmha.tune_decode_num_splits(q, kc, vc, sl, bt, max_seqlen_k=2048, candidates=(1, 2, 4, 8), scale=w["scale"])
        assert rec["num_splits"] in (1, 2, 4, 8) and set(rec["tried_us"]) == {"1", "2", "4", "8"}
        assert (tmp_path / tuning.FILE_NAME).exists()
        prob = tuning.splitkv_problem(4, 16, 4, 1, 2048, 128, 64, "bf16")
        assert tuning.default_cache().query(tuning.SPLITKV, prob)["num_splits"] == rec["num_splits"]
        o = fmha.fmha_decode_paged(q, kc, vc, sl, bt, max_seqlen_k=2048, scale=w["scale"])  # num_splits = 0: the record
        ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqlen_k=w["seqlen_k"], block_table=w["block_table"],
                          scale=w["scale"])
        assert_close(o, ro, 2e-2, "decode with the tuned split count")
    finally:
        for n, v in saved.items():
            flashck_amd.set_flag_value(n, v)
        tuning._default = old_default


def test_decode_kernel_variant_is_tunable(fmha, orc, tmp_path):
    """The two split-KV kernel variants (one KV head per workgroup, head pairs) forced through the attribute both match
    the oracle; the tuner measures (split count, variant) pairs and a later num_splits = 0 call runs the recorded pair."""
    import flashck_amd
    from flashck_amd import _lib
    from flashck_amd.utils import tuning
    w = gen.workload_paged_decode(seed=76, batch=6, hq=16, hk=4, head_dim=128, min_len=300, max_len=1500, page_size=128)
    q, kc, vc = dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"])
    sl, bt = dev(w["seqlen_k"]), dev(w["block_table"])
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqlen_k=w["seqlen_k"], block_table=w["block_table"], scale=w["scale"])
    outs = {}
    for variant in (1, 2):
        outs[variant] = fmha.fmha_decode_paged(q, kc, vc, sl, bt, num_splits=2, scale=w["scale"], decode_variant=variant)
        assert_close(outs[variant], ro, 2e-2, f"variant {variant}")
    with pytest.raises(ValueError):   # head pairs need an even number of KV heads
        odd = gen.workload_paged_decode(seed=77, batch=2, hq=6, hk=3, head_dim=128, min_len=50, max_len=100, page_size=128)
        fmha.fmha_decode_paged(dev(odd["q"]), dev(odd["k_cache"]), dev(odd["v_cache"]), dev(odd["seqlen_k"]), dev(odd["block_table"]),
                               num_splits=2, decode_variant=2)
    saved = {n: flashck_amd.get_flag_value(n) for n in ("FC_TUNING_DB_DIR", "FC_TUNING_NUM_COLD_ITERATION",
                                                          "FC_TUNING_NUM_REPEATS", "FC_TUNING_MODE")}
    old_default = tuning._default
    try:
        flashck_amd.set_flag_value("FC_TUNING_DB_DIR", str(tmp_path))
        flashck_amd.set_flag_value("FC_TUNING_NUM_COLD_ITERATION", "2")
        flashck_amd.set_flag_value("FC_TUNING_NUM_REPEATS", "5")
        flashck_amd.set_flag_value("FC_TUNING_MODE", "2")
        tuning._default = None
        rec = fmha.tune_decode_num_splits(q, kc, vc, sl, bt, max_seqlen_k=2048, candidates=(2, 4), variants=(1, 2), scale=w["scale"])
        assert rec["variant"] in (1, 2) and set(rec["tried_us"]) == {"2/v1", "2/v2", "4/v1", "4/v2"}
        assert rec["kernel"].startswith("splitkv_decode_kernel")
        o = fmha.fmha_decode_paged(q, kc, vc, sl, bt, max_seqlen_k=2048, scale=w["scale"])   # num_splits = 0: the recorded pair
        assert_close(o, ro, 2e-2, "decode with the tuned pair")
    finally:
        for n, v in saved.items():
            flashck_amd.set_flag_value(n, v)
        tuning._default = old_default


def test_page_size_one(fmha, orc):
    """A page list with one token per page (the layout some serving stacks use): prefill and decode."""
    w = gen.workload_varlen_prefill(seed=74, batch=4, hq=4, hk=2, head_dim=128, min_len=3, max_len=300, page_size=1)
    o = fmha.fmha_batch_prefill(dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"]), dev(w["cu_seqlens_q"]), dev(w["kv_indptr"]),
                                dev(w["kv_page_indices"]), dev(w["kv_last_page_lens"]), max_seqlen_q=w["max_seqlen_q"],
                                scale=w["scale"])
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"],
                      kv_page_indices=w["kv_page_indices"], kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"],
                      mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "prefill, page size 1")
    d = gen.workload_paged_decode(seed=75, batch=3, hq=8, hk=2, head_dim=128, min_len=1, max_len=500, page_size=1)
    od = fmha.fmha_decode_paged(dev(d["q"]), dev(d["k_cache"]), dev(d["v_cache"]), dev(d["seqlen_k"]), dev(d["block_table"]),
                                num_splits=3, scale=d["scale"])
    rd = orc.fmha_fwd(d["q"], d["k_cache"], d["v_cache"], seqlen_k=d["seqlen_k"], block_table=d["block_table"], scale=d["scale"])
    assert_close(od, rd, 2e-2, "decode, page size 1")


@pytest.mark.parametrize("fused", [False, True])
def test_decode_captured_in_a_graph(fmha, orc, fused):
    """A decode launch sequence (appendKV + split-KV + combine, or appendKV + the fused launch) captured into a HIP
    graph after one eager warm-up call, then replayed three times with new inputs written into the captured buffers and
    eager work and synchronisations between the replays; every replay is checked against the oracle.  The operators
    enqueue kernels only (no memset, no allocation), so the capture holds nothing else."""
    B, hq, hk, d, page = 4, 16, 4, 128, 64
    g = torch.Generator().manual_seed(83)
    lens = [100, 1, 333, 64]
    kv = gen.paged_kv(lens, hk, d, torch.bfloat16, g, page, capacity=[l + 8 for l in lens])
    cos, sin = gen.rotary_tables(400, d, torch.bfloat16, 10000.0)
    kc, vc, bt = dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["block_table"])
    sl = dev(kv["seqlen_k"].clone())           # advanced in place by the captured graph's caller between replays
    sl_after = torch.empty_like(sl)
    q, knew, vnew = (torch.empty(B, 1, h, d, dtype=torch.bfloat16, device=helpers.DEVICE) for h in (hq, hk, hk))
    out = torch.empty(B, 1, hq, d, dtype=torch.bfloat16, device=helpers.DEVICE)
    ws = fmha.splitkv_workspace(B, hq, 1, d, 3, helpers.DEVICE)
    dcos, dsin = dev(cos), dev(sin)

    def enqueue():
        fmha.fmha_fwd_appendkv(q, kc, vc, knew, vnew, sl, rotary_cos=dcos, rotary_sin=dsin, rope_mode=fmha.ROPE_HALF_ROTATED,
                               block_table=bt)
        torch.add(sl, 1, out=sl_after)
        fmha.fmha_decode_paged(q, kc, vc, sl_after, bt, num_splits=3, workspace=None if fused else ws, out=out, fused=fused)

    def new_inputs():
        hq_, hk_ = gen.randn((B, 1, hq, d), torch.bfloat16, g), gen.randn((B, 1, hk, d), torch.bfloat16, g)
        return hq_, hk_, gen.randn((B, 1, hk, d), torch.bfloat16, g)

    # CPU mirror of the cache and the lengths
    rkc, rvc, rsl = kv["k_cache"].clone(), kv["v_cache"].clone(), kv["seqlen_k"].clone()
    cu = torch.arange(0, B + 1, dtype=torch.int32)

    def expect(hq_, hk_, hv_):
        rq = hq_.clone().view(B, hq, d)
        orc.appendkv(rq, rkc, rvc, hk_.view(B, hk, d), hv_.view(B, hk, d), rsl, cu, cos=cos, sin=sin, rope_mode=2, has_mask=True,
                     block_table=kv["block_table"])
        rsl.add_(1)
        return orc.fmha_fwd(rq.view(B, 1, hq, d), rkc, rvc, seqlen_k=rsl, block_table=kv["block_table"])

    # eager warm-up call (first use of every kernel: opts in to its LDS size), on a scratch copy of the state
    a, b_, c = new_inputs()
    q.copy_(a); knew.copy_(b_); vnew.copy_(c)
    keep = (kc.clone(), vc.clone())
    enqueue()
    torch.cuda.synchronize()
    kc.copy_(keep[0]); vc.copy_(keep[1])

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    kc.copy_(keep[0]); vc.copy_(keep[1])   # whatever the capture did to the cache is undone: replays start from the mirror's state
    for rep in range(3):
        a, b_, c = new_inputs()
        q.copy_(a); knew.copy_(b_); vnew.copy_(c)
        graph.replay()
        torch.cuda.synchronize()
        ro = expect(a, b_, c)
        assert_close(out, ro, 2e-2, f"replay {rep}")
        assert_bits_equal(kc, rkc, f"k cache after replay {rep}")
        sl.add_(1)                          # eager work between the replays
        assert torch.equal(sl.cpu(), rsl)
