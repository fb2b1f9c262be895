"""The C++ header API (include/flashck/fmha/fmha_fwd.h) with real device pointers: tests/cpp/fmha_header_gpu (built by
`__graft_entry__.build()` / `python -m flashck_amd.build`) runs dense forward, paged split-KV decode + combine and
page-list prefill through the typed header functions; the outputs are compared with the oracle."""
import os
import subprocess

import numpy as np
import pytest
import torch

from flashck_amd import generators as gen
from helpers import ATOL, assert_close

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "fmha_header_gpu")


def run(op, dtype, header, arrays, out_shape, tmp_path):
    assert os.path.exists(EXE), "tests/cpp/fmha_header_gpu is missing: run `python -m flashck_amd.build`"
    inp, out = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(inp, "wb") as f:
        f.write(np.array(list(header) + [0] * (16 - len(header)), dtype=np.int64).tobytes())
        for a in arrays:
            a = a.contiguous()
            f.write((a.view(torch.int16) if a.dtype in (torch.float16, torch.bfloat16) else a).numpy().tobytes())
    r = subprocess.run([EXE, "fp16" if dtype == torch.float16 else "bf16", op, inp, out], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    raw = np.fromfile(out, dtype=np.int16)
    return torch.from_numpy(raw).view(dtype).reshape(out_shape)


def test_dense_forward_through_the_header(orc, tmp_path):
    w = gen.workload_dense_fp16()
    q, k, v = w["q"], w["k"], w["v"]
    B, sq, Hq, D = q.shape
    for mask_type, window in ((0, (-1, -1)), (2, (-1, 0))):
        o = run("fwd", torch.float16, [B, sq, k.shape[1], Hq, k.shape[2], D, mask_type, window[0], window[1]], [q, k, v], q.shape, tmp_path)
        assert_close(o, orc.fmha_fwd(q, k, v, mask_type=mask_type, window=window), ATOL[torch.float16], f"mask {mask_type}")


@pytest.mark.parametrize("num_splits", [3, 0])
def test_paged_decode_through_the_header(orc, tmp_path, num_splits):
    w = gen.workload_paged_decode(seed=101, batch=3, hq=8, hk=2, head_dim=128, min_len=100, max_len=900, page_size=128)
    q, kc, vc, sl, bt = w["q"], w["k_cache"], w["v_cache"], w["seqlen_k"], w["block_table"]
    B, _, Hq, D = q.shape
    o = run("decode", torch.bfloat16, [B, Hq, kc.shape[2], D, kc.shape[0], kc.shape[1], bt.shape[1], num_splits], [q, kc, vc, sl, bt],
            (B, 1, Hq, D), tmp_path)
    assert_close(o, orc.fmha_fwd(q, kc, vc, seqlen_k=sl, block_table=bt, scale=w["scale"]), ATOL[torch.bfloat16], "decode")


def test_batch_prefill_through_the_header(orc, tmp_path):
    w = gen.workload_varlen_prefill(seed=102, batch=3, hq=4, hk=2, head_dim=128, min_len=10, max_len=400, page_size=64)
    q, kc, vc = w["q"], w["k_cache"], w["v_cache"]
    o = run("prefill", torch.bfloat16,
            [3, q.shape[0], 4, 2, 128, kc.shape[0], kc.shape[1], w["kv_page_indices"].numel(), w["max_seqlen_q"]],
            [q, kc, vc, w["cu_seqlens_q"], w["kv_indptr"], w["kv_page_indices"], w["kv_last_page_lens"]], q.shape, tmp_path)
    ro = orc.fmha_fwd(q, kc, vc, seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"], kv_page_indices=w["kv_page_indices"],
                      kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"], mask_type=2, window=(-1, 0))
    assert_close(o, ro, ATOL[torch.bfloat16], "prefill")
