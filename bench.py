#!/usr/bin/env python3
"""Benchmark of the FMHA hot path on one MI355X.

One "step" is one pass of the headline workload: split-KV long-context decode (batch 4, q_len 1, 64 query / 8 KV heads,
head_dim 128, 32768 keys per sequence in shuffled 128-token pages, num_splits 8) = one split-KV launch + one combine
launch.  `value` is algorithmic HBM bytes per step / wall time per step with every input resident in HBM; the KV pool is
rotated over several copies so no step finds its pages in the caches.  The JSON line also carries the roofline of the
dominant kernel (HIP events around every split-KV launch of the timed region), a CPU baseline (the oracle on a bounded
sample, same run, host cores of this box) and, under "extra", the other workloads: paged decode, appendKV, and varlen
causal prefill in TFLOP/s.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16

COUNTER_FILE = os.path.join(ROOT, "profiles", "splitkv_decode_cfg3.md")
# every source file that goes into the device code of the split-KV kernel
DECODE_SOURCES = [os.path.join(ROOT, "flashck_amd", "csrc", f) for f in ("splitkv_decode.hip", "common.hpp", "kernels.hpp", "gfx950_ops.hpp")]


def decode_source_hash():
    import hashlib
    h = hashlib.sha256()
    for path in DECODE_SOURCES:
        h.update(open(path, "rb").read())
    return h.hexdigest()


def measured_traffic(kernel):
    """HBM bytes one split-KV launch of the default workload moved when the hardware counters were last read, or None.

    The figure is not measured by this run: it comes from the `counters` line of profiles/splitkv_decode_cfg3.md (two
    `rocprofv3 --pmc` runs of this script, FETCH_SIZE and WRITE_SIZE in KiB per dispatch, each scaled by what the same
    counter reads for a plain device copy of known size).  It is only reported while it still describes the code that
    runs: same kernel variant and same source files (the kernel and the headers it is built from) as when the
    counters were read.
    """
    import re
    try:
        text = open(COUNTER_FILE).read()
        sha = decode_source_hash()
    except OSError:
        return None
    m = re.search(r'counters kernel="([^"]+)" source_sha256=([0-9a-f]+) fetch_kib=([0-9.]+) write_kib=([0-9.]+) '
                  r'fetch_scale=([0-9.]+) write_scale=([0-9.]+)', text)
    if not m or m.group(1) != kernel or m.group(2) != sha:
        return None
    return int(float(m.group(3)) * 1024 * float(m.group(5)) + float(m.group(4)) * 1024 * float(m.group(6)))


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="splitkv", choices=["splitkv", "paged_decode", "prefill", "prefill256", "copy"],
                    help="workload of the headline line (default: split-KV long-context decode)")
    ap.add_argument("--copies", type=int, default=4, help="KV pool copies rotated between steps")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--paged-splits", type=int, default=0, help="split count of the paged-decode workload (0: the library's heuristic)")
    ap.add_argument("--kv-fp8", action="store_true", help="split-KV workload with the cache stored as fp8 (e4m3, static scales)")
    ap.add_argument("--decode-path", default="two-launch", choices=["two-launch", "fused"],
                    help="two-launch: split-KV + combine kernels with a caller-owned workspace; fused: one launch "
                         "(--num-splits 0 lets the library choose the key ranges)")
    args = ap.parse_args()
    # the split-KV workload: 32768 keys per sequence, 8 splits, shuffled pages
    args.kv_len, args.num_splits, args.no_shuffle = 32768, 8, False
    return args


def time_steps(fn, steps, warmup, torch, kernel_events=False):
    """Runs fn(step, ev) warmup + steps times.  Returns (wall seconds for `steps`, avg ms per launch by HIP events).

    kernel_events = "region": one event pair on the launch stream brackets the whole timed region (for steps that are
    a single launch: the average it gives includes the gaps between launches).  kernel_events = True: the timed region
    carries no events; the same steps are then run once more with an event pair around the kernel of every step.
    """
    for i in range(warmup):
        fn(i, None)
    torch.cuda.synchronize()
    region = kernel_events == "region"
    if region:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if region:
        e0.record()
    for i in range(steps):
        fn(warmup + i, None)
    if region:
        e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kern_ms = None
    if region:
        kern_ms = e0.elapsed_time(e1) / steps
    elif kernel_events:
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for i in range(steps):
            fn(warmup + steps + i, evs[i])
        torch.cuda.synchronize()
        kern_ms = sum(a.elapsed_time(b) for a, b in evs) / steps
    return wall, kern_ms


def bench_decode(args, torch, fmha, gen, which):
    from flashck_amd import _lib
    if which == "splitkv":
        w = gen.workload_splitkv_decode(kv_len=args.kv_len, num_splits=args.num_splits, shuffle=not args.no_shuffle)
        ns = w["num_splits"]
        if getattr(args, "decode_path", "two-launch") == "fused":
            ns = args.num_splits
            name = (f"split-KV long-context decode: B=4 q=1 Hq64/Hk8 D128 L={args.kv_len} P=128, one fused launch, "
                    f"ns={ns if ns else 'library-chosen'} (bf16)")
        else:
            name = f"split-KV long-context decode: B=4 q=1 Hq64/Hk8 D128 L={args.kv_len} P=128 ns={ns} + combine (bf16)"
    else:
        w = gen.workload_paged_decode()
        if getattr(args, "decode_path", "two-launch") == "fused":
            ns = 0
            name = "paged-KV decode: B=32 q=1 Hq32/Hk8 D128 L~U[512,4096] P=128, one fused launch, library-chosen ranges (bf16)"
        else:
            ns = args.paged_splits or fmha.num_splits_heuristic(32, 32, 8, 1, max(w["lens"]), 128)
            name = f"paged-KV decode: B=32 q=1 Hq32/Hk8 D128 L~U[512,4096] P=128 ns={ns} + combine (bf16)"
            if getattr(args, "paged_variant", 0):
                name += f" [kernel variant {args.paged_variant}]"
    B, _, Hq, D = w["q"].shape
    Hk = w["k_cache"].shape[2]
    dev = "cuda"
    q = w["q"].to(dev)
    bt, sl = w["block_table"].to(dev), w["seqlen_k"].to(dev)
    all_fp8 = getattr(args, "all_fp8", False)  # Q, P and O in e4m3 as well (the query scale goes into the softmax scale)
    kv_fp8 = getattr(args, "kv_fp8", False) or all_fp8
    scales = {}
    if all_fp8:
        q = (w["q"].float() / 0.0625).to(torch.float8_e4m3fn).to(dev)  # cast on the host, as the tests do
        w["scale"] = w["scale"] * 0.0625
    if kv_fp8:
        # unit-variance data: a static scale of 1/16 keeps it well inside the e4m3 range (+-448)
        scales = dict(k_descale=0.0625, v_descale=0.0625)
        w["k_cache"] = (w["k_cache"].float() / 0.0625).to(torch.float8_e4m3fn)
        w["v_cache"] = (w["v_cache"].float() / 0.0625).to(torch.float8_e4m3fn)
        name = name.replace("(bf16)", "(e4m3 in and out, bf16 matrix instructions)") if all_fp8 else name + " [K/V cache fp8 e4m3]"
    pools = [(w["k_cache"].to(dev), w["v_cache"].to(dev))]
    for _ in range(args.copies - 1):
        pools.append((pools[0][0].clone(), pools[0][1].clone()))
    o_acc, lse_acc = fmha.splitkv_workspace(B, Hq, 1, D, max(ns, 1), dev)
    o = torch.empty(B, 1, Hq, D, dtype=q.dtype, device=dev)

    fused = getattr(args, "decode_path", "two-launch") == "fused"
    variant = getattr(args, "paged_variant", 0) if which == "paged_decode" else 0

    def step(i, ev):
        kc, vc = pools[i % len(pools)]
        if ev is not None:
            ev[0].record()
        if fused:
            fmha.fmha_fwd_splitkv_fused(q, kc, vc, ns, seqlen_k=sl, block_table=bt, scale=w["scale"], out=o)
        else:
            fmha.fmha_fwd_splitkv(q, kc, vc, ns, seqlen_k=sl, block_table=bt, scale=w["scale"], o_acc=o_acc, lse_acc=lse_acc,
                                  decode_variant=variant, max_seqlen_k=max(w["lens"]) if variant >= 3 else 0, **scales)
        if ev is not None:
            ev[1].record()
        if not fused:
            fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, q.dtype, out=o)

    wall, kern_ms = time_steps(step, args.steps, args.warmup, torch, kernel_events="region" if fused else True)
    kernel = _lib.load().fck_fmha_last_kernel().decode()  # the combine launch does not change it
    nbytes = gen.decode_bytes(w["lens"], [1] * B, Hq, Hk, D, D, 128, kv_elem=1 if kv_fp8 else None)
    flops = gen.decode_flops(w["lens"], [1] * B, Hq, D, D)
    ms = wall / args.steps * 1e3
    res = dict(name=name, ms_per_step=ms, bytes=nbytes, flops=flops, gbs=nbytes / (ms * 1e-3) / 1e9,
               kernel_ms=kern_ms, kernel_gbs=nbytes / (kern_ms * 1e-3) / 1e9, num_splits=ns, w=w, kernel=kernel)
    return res


def bench_prefill(args, torch, fmha, gen, d, steps, warmup, variant=0, alibi=False, kv_fp8=False, dv=None, all_fp8=False):
    """variant: tile variant (fck_fmha_attrs.prefill_variant); alibi: with per-head ALiBi slopes; kv_fp8: K/V cache as e4m3;
    all_fp8: Q, P and O in e4m3 as well; dv: head dim of V / O when it differs from d"""
    w = gen.workload_varlen_prefill(head_dim=d, v_head_dim=dv)
    dev = "cuda"
    kw = {}
    kv_fp8 = kv_fp8 or all_fp8
    if all_fp8:
        w["q"] = (w["q"].float() / 0.0625).to(torch.float8_e4m3fn)
        w["scale"] = w["scale"] * 0.0625
    if alibi:
        kw["alibi_slopes"] = (torch.arange(1, 33, dtype=torch.float32) / 256).to(dev)
    if kv_fp8:
        w["k_cache"] = (w["k_cache"].float() / 0.0625).to(torch.float8_e4m3fn)
        w["v_cache"] = (w["v_cache"].float() / 0.0625).to(torch.float8_e4m3fn)
        kw.update(k_descale=0.0625, v_descale=0.0625)
    a = [w[k].to(dev) for k in ("q", "k_cache", "v_cache", "cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    o = torch.empty(a[0].shape[0], a[0].shape[1], dv or d, dtype=a[0].dtype, device=dev)

    def step(i, ev):
        if ev is not None:
            ev[0].record()
        fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"], out=o, prefill_variant=variant, **kw)
        if ev is not None:
            ev[1].record()

    wall, kern_ms = time_steps(step, steps, warmup, torch, kernel_events=True)
    from flashck_amd import _lib
    kernel = _lib.load().fck_fmha_last_kernel().decode()
    flops = gen.prefill_flops(w["lens"], 32, d, dv or d)
    nbytes = gen.prefill_bytes(w["lens"], 32, 8, d, dv or d)
    ms = wall / steps * 1e3
    tag = (f" (v_head_dim {dv})" if dv else "") + (" + ALiBi" if alibi else "") + (" [K/V cache fp8 e4m3]" if kv_fp8 and not all_fp8 else "") + (f" [tile variant {variant}]" if variant else "")
    kind = "e4m3 in and out, bf16 matrix instructions" if all_fp8 else "bf16"
    return dict(name=f"varlen causal batch prefill: 16 seqs L~U[128,8192] Hq32/Hk8 D{d} paged P=128 ({kind})" + tag,
                ms_per_step=ms, flops=flops, bytes=nbytes, tflops=flops / (ms * 1e-3) / 1e12, kernel_ms=kern_ms,
                kernel_tflops=flops / (kern_ms * 1e-3) / 1e12, total_q=sum(w["lens"]), kernel=kernel)


def bench_appendkv(args, torch, fmha, gen, steps, warmup):
    w = gen.workload_appendkv_decode()
    dev = "cuda"
    q, kc, vc = w["q"].to(dev), w["k_cache"].to(dev), w["v_cache"].to(dev)
    knew, vnew, sl, cu = w["knew"].to(dev), w["vnew"].to(dev), w["seqlen_k"].to(dev), w["cu_seqlens_knew"].to(dev)
    cos, sin, bt = w["rotary_cos"].to(dev), w["rotary_sin"].to(dev), w["block_table"].to(dev)

    def step(i, ev):
        fmha.fmha_fwd_appendkv(q, kc, vc, knew, vnew, sl, cu_seqlens_knew=cu, max_seqlen_knew=w["max_new"], rotary_cos=cos,
                               rotary_sin=sin, rope_mode=fmha.ROPE_HALF_ROTATED, has_mask=True, block_table=bt)

    wall, _ = time_steps(step, steps, warmup, torch)
    tn = q.shape[0]
    nbytes = tn * (8 * 128 * 2 * 2) * 2 + tn * 32 * 128 * 2 * 2
    return dict(name="appendKV + RoPE: B=16, 1-16 new tokens, Hq32/Hk8 D128, shuffled 128-token pages (bf16)",
                us_per_call=wall / steps * 1e6, bytes=nbytes, new_tokens=tn)


def cpu_baseline_decode(w, ns, gen, min_seconds=10.0):
    """The oracle (a port of the reference's CPU host-reference attention) on the same workload: split-KV partials +
    combine over every sequence and head, repeated until at least `min_seconds` of CPU work have been timed."""
    from oracle import fmha_oracle as orc
    orc.build()
    q, bt, sl, lens = w["q"], w["block_table"], w["seqlen_k"], w["lens"]
    B, Hq, D, Hk = q.shape[0], q.shape[2], q.shape[3], w["k_cache"].shape[2]
    passes, t0 = 0, time.perf_counter()
    while True:
        o_acc, lse_acc = orc.fmha_splitkv(q, w["k_cache"], w["v_cache"], ns, seqlen_k=sl, block_table=bt, scale=w["scale"])
        orc.splitkv_combine(lse_acc, o_acc, q.dtype)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds or passes >= 1000:
            break
    nbytes = gen.decode_bytes(lens, [1] * B, Hq, Hk, D, D, 128) * passes
    return dict(value=nbytes / dt / 1e9, unit="GB/s", cores=orc.num_threads(), kind="port",
                sample=f"{passes} passes over the whole workload ({B} sequences, {Hq} heads, full KV lengths), "
                       f"split-KV partials + combine, {dt:.1f} s of CPU time on {orc.num_threads()} threads",
                seconds=dt, us_per_call=dt / passes * 1e6)


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this build has no multi-GPU path (asked for --gpus {args.gpus})", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    from flashck_amd import _lib, generators as gen
    from flashck_amd.ops import fmha
    _lib.load()  # raises when the HIP library is missing: there is no other compute path
    torch.cuda.set_device(0)

    extra = {}
    if args.workload == "copy":
        # calibration run for the hardware counters: a plain device copy of known size (512 MiB read + 512 MiB written)
        n = 512 << 20
        src = torch.full((n,), 1, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        wall, _ = time_steps(lambda i, ev: dst.copy_(src), args.steps, args.warmup, torch)
        print(json.dumps({"metric": "device copy (counter calibration)", "value": 2 * n / (wall / args.steps) / 1e9,
                          "unit": "GB/s", "bytes_read": n, "bytes_written": n, "steps": args.steps}))
        return
    if args.workload in ("splitkv", "paged_decode"):
        r = bench_decode(args, torch, fmha, gen, args.workload)
        value, unit, metric = r["gbs"], "GB/s", "paged-KV decode HBM GB/s (% of peak) + us/call; prefill TFLOP/s, MFMA util %"
        default_shape = (args.workload == "splitkv" and args.kv_len == 32768 and args.num_splits == 8 and not args.no_shuffle
                         and args.decode_path == "two-launch")
        traffic = measured_traffic(r["kernel"]) if default_shape else None  # counters were only read for that shape
        roof = dict(bound="hbm", kernel=r["kernel"], achieved=r["kernel_gbs"], peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=r["kernel_gbs"] / HBM_PEAK_GBS, traffic=traffic, bytes_per_launch=r["bytes"],
                    avg_launch_us=r["kernel_ms"] * 1e3)
        extra["pct_of_hbm_peak"] = 100.0 * value / HBM_PEAK_GBS
        extra["us_per_call"] = r["ms_per_step"] * 1e3
        cpu = None
        if not args.no_cpu:
            try:
                cpu = cpu_baseline_decode(r["w"], r["num_splits"], gen)
            except Exception as e:  # noqa: BLE001
                cpu = dict(error=f"{type(e).__name__}: {e}")
        ms, name = r["ms_per_step"], r["name"]
    else:
        d = 128 if args.workload == "prefill" else 256
        r = bench_prefill(args, torch, fmha, gen, d, args.steps, args.warmup)
        value, unit, metric = r["tflops"], "TFLOP/s", "varlen causal prefill TFLOP/s (MFMA util %)"
        roof = dict(bound="mfma", kernel=r["kernel"], achieved=r["kernel_tflops"], peak=MFMA_BF16_PEAK_TFLOPS,
                    unit="TFLOP/s", frac=r["kernel_tflops"] / MFMA_BF16_PEAK_TFLOPS, traffic=None,
                    flops_per_launch=r["flops"], avg_launch_us=r["kernel_ms"] * 1e3)
        cpu = None
        ms, name = r["ms_per_step"], r["name"]

    if not args.no_extra and args.workload == "splitkv":
        # secondary workloads: a failure in one of them is reported in its place and does not cost the headline line
        def secondary(name, fn):
            try:
                extra[name] = fn()
            except Exception as e:  # noqa: BLE001
                extra[name] = dict(error=f"{type(e).__name__}: {e}")
            torch.cuda.empty_cache()

        def paged():
            a2 = argparse.Namespace(**vars(args))
            a2.steps, a2.warmup = max(20, args.steps // 2), 10
            r2 = bench_decode(a2, torch, fmha, gen, "paged_decode")
            return dict(workload=r2["name"], us_per_call=r2["ms_per_step"] * 1e3, gbs=r2["gbs"],
                        pct_of_hbm_peak=100 * r2["gbs"] / HBM_PEAK_GBS, kernel_us=r2["kernel_ms"] * 1e3, bytes=r2["bytes"])

        def paged_tuned():
            # the library's tuning flow on this workload: measure (split count, kernel variant) pairs, run the winner
            import tempfile
            from flashck_amd.utils import tuning
            w = gen.workload_paged_decode()
            t = [w[k].to("cuda") for k in ("q", "k_cache", "v_cache", "seqlen_k", "block_table")]
            with tempfile.TemporaryDirectory() as tmp:
                rec = fmha.tune_decode_num_splits(*t, max_seqlen_k=max(w["lens"]), candidates=(1, 2, 3, 4, 6, 8, 12, 16), variants=(1, 2, 3, 4),
                                                  cache=tuning.TuningCache(directory=tmp), scale=w["scale"])
            del t
            a2 = argparse.Namespace(**vars(args))
            a2.steps, a2.warmup, a2.paged_splits, a2.paged_variant = max(20, args.steps // 2), 10, rec["num_splits"], rec["variant"]
            r2 = bench_decode(a2, torch, fmha, gen, "paged_decode")
            return dict(workload=r2["name"], us_per_call=r2["ms_per_step"] * 1e3, gbs=r2["gbs"],
                        pct_of_hbm_peak=100 * r2["gbs"] / HBM_PEAK_GBS, kernel_us=r2["kernel_ms"] * 1e3, kernel=r2["kernel"],
                        num_splits=rec["num_splits"], variant=rec["variant"], tried_us=rec["tried_us"])

        def append():
            r4 = bench_appendkv(args, torch, fmha, gen, 100, 10)
            return dict(workload=r4["name"], us_per_call=r4["us_per_call"], bytes=r4["bytes"], new_tokens=r4["new_tokens"])

        def prefill(d, **kw):
            r5 = bench_prefill(args, torch, fmha, gen, d, 10, 3, **kw)
            return dict(workload=r5["name"], ms_per_call=r5["ms_per_step"], tflops=r5["tflops"],
                        mfma_util_pct=100 * r5["tflops"] / MFMA_BF16_PEAK_TFLOPS, flops=r5["flops"], kernel_ms=r5["kernel_ms"],
                        kernel=r5["kernel"])

        def prefill_tuned():
            # every tile variant of the ping-pong kernel on this workload, then the fastest again as a line of its own
            tried = {}
            for v in (1, 2, 3, 4):
                r = bench_prefill(args, torch, fmha, gen, 128, 5, 2, variant=v)
                tried[f"v{v}"] = dict(ms=r["kernel_ms"], kernel=r["kernel"])
            best = min((1, 2, 3, 4), key=lambda v: tried[f"v{v}"]["ms"])
            out = prefill(128, variant=best)
            out.update(variant=best, tried_kernel_ms={k: t["ms"] for k, t in tried.items()})
            return out

        def splitkv_variant(path, ns, kv_fp8=False, all_fp8=False):
            a2 = argparse.Namespace(**vars(args))
            a2.steps, a2.warmup, a2.decode_path, a2.num_splits, a2.kv_fp8, a2.all_fp8 = max(20, args.steps // 2), 10, path, ns, kv_fp8, all_fp8
            r3 = bench_decode(a2, torch, fmha, gen, "splitkv")
            return dict(workload=r3["name"], us_per_call=r3["ms_per_step"] * 1e3, gbs=r3["gbs"],
                        pct_of_hbm_peak=100 * r3["gbs"] / HBM_PEAK_GBS, kernel_us=r3["kernel_ms"] * 1e3, num_splits=r3["num_splits"])

        # the same workload with the split count the library's heuristic picks, and as one fused launch
        ns_lib = fmha.num_splits_heuristic(4, 64, 8, 1, args.kv_len, 128)
        secondary("splitkv_library_splits", lambda: splitkv_variant("two-launch", ns_lib))
        secondary("splitkv_fused", lambda: splitkv_variant("fused", 0))
        secondary("splitkv_fp8_cache", lambda: splitkv_variant("two-launch", ns_lib, kv_fp8=True))
        secondary("splitkv_all_fp8", lambda: splitkv_variant("two-launch", ns_lib, all_fp8=True))
        secondary("paged_decode", paged)
        secondary("paged_decode_tuned", paged_tuned)
        secondary("appendkv", append)
        for d in (128, 256):
            secondary(f"prefill_d{d}", lambda d=d: prefill(d))
        secondary("prefill_d128_tuned", prefill_tuned)
        secondary("prefill_d128_alibi", lambda: prefill(128, alibi=True))
        secondary("prefill_d256_alibi", lambda: prefill(256, alibi=True))
        secondary("prefill_d128_fp8_cache", lambda: prefill(128, kv_fp8=True))
        secondary("prefill_d128_all_fp8", lambda: prefill(128, all_fp8=True))
        secondary("prefill_d192_dv128", lambda: prefill(192, dv=128))

    line = {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic", "config": {"workload": name, "kv_pool_copies_rotated": args.copies,
                                "library": os.path.relpath(_lib.LIB_PATH, ROOT)},
        "roofline": roof, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
