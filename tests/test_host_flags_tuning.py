"""Flags surface and the persisted tuning cache (host logic, no GPU)."""
import json
import os

import pytest

import flashck_amd
from flashck_amd.utils import flags, tuning

ENV = {"rocm_version": "7.0.test", "device_name": "gfx950-test"}


@pytest.fixture(autouse=True)
def restore_flags():
    saved = dict(flags._VALUES)
    yield
    flags._VALUES.clear()
    flags._VALUES.update(saved)


def test_flag_values_travel_as_strings():
    assert flashck_amd.get_flag_value("FC_TUNING_SEED") == "42"          # FC_TUNING_SEED default, flags.cc:225
    assert flashck_amd.get_flag_value("FC_TUNING_NUM_REPEATS") == "64"   # flags.cc:219
    assert flashck_amd.get_flag_value("FC_TUNING_FLUSH_CACHE") == "true"
    flashck_amd.set_flag_value("FC_TUNING_NUM_REPEATS", "7")
    assert flags.flag("FC_TUNING_NUM_REPEATS") == 7 and flashck_amd.get_flag_value("FC_TUNING_NUM_REPEATS") == "7"
    flashck_amd.set_flag_value("FC_TUNING_LOG", "TRUE")
    assert flags.flag("FC_TUNING_LOG") is True
    flashck_amd.set_flag_value("FC_TUNING_DB_DIR", "/tmp/x")
    assert flashck_amd.get_flag_value("FC_TUNING_DB_DIR") == "/tmp/x"


def test_flag_errors_follow_the_reference_messages():
    with pytest.raises(RuntimeError, match="Flag not found: FC_NOPE"):
        flashck_amd.get_flag_value("FC_NOPE")
    with pytest.raises(RuntimeError, match="Failed to set flag: FC_NOPE"):
        flashck_amd.set_flag_value("FC_NOPE", "1")
    with pytest.raises(RuntimeError, match="Failed to set flag: FC_TUNING_SEED"):
        flashck_amd.set_flag_value("FC_TUNING_SEED", "forty-two")
    with pytest.raises(RuntimeError, match="Failed to set flag: FC_TUNING_LOG"):
        flashck_amd.set_flag_value("FC_TUNING_LOG", "maybe")
    with pytest.raises(RuntimeError, match="Failed to set flag: FC_TUNING_GPU_TIMER"):  # read-only
        flashck_amd.set_flag_value("FC_TUNING_GPU_TIMER", "false")
    with pytest.raises(RuntimeError, match="Flag not found"):
        flashck_amd.print_flag_info("FC_NOPE")


def test_flag_printing(capsys):
    flashck_amd.print_all_flags()
    out = capsys.readouterr().out
    assert "=== FlashCK Flags ===" in out and "FC_TUNING_MODE" in out and "FC_TUNING_GPU_TIMER" in out
    flashck_amd.print_all_flags(writable_only=True)
    assert "FC_TUNING_GPU_TIMER" not in capsys.readouterr().out
    flashck_amd.print_flag_info("FC_TUNING_SEED")
    out = capsys.readouterr().out
    assert "Name: FC_TUNING_SEED" in out and "Type: int32_t" in out and "Default Value: 42" in out


def test_flags_start_from_the_environment():
    import subprocess
    import sys
    code = "import flashck_amd; print(flashck_amd.get_flag_value('FC_TUNING_MODE'), flashck_amd.get_flag_value('FC_TUNING_LOG'))"
    env = dict(os.environ, FC_TUNING_MODE="0", FC_TUNING_LOG="yes")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, cwd=os.path.dirname(os.path.dirname(__file__)))
    assert out.stdout.split() == ["0", "true"], out.stderr
    bad = subprocess.run([sys.executable, "-c", code], env=dict(os.environ, FC_TUNING_SEED="x"), capture_output=True, text=True,
                         cwd=os.path.dirname(os.path.dirname(__file__)))
    assert bad.returncode != 0 and "FC_TUNING_SEED" in bad.stderr


def test_problem_key_buckets():
    a = tuning.splitkv_problem(4, 64, 8, 1, 32768, 128, 128, "bf16")
    assert a == "dtype=bf16,hq=64,hk=8,d=128,page=128,b<=4,sq<=1,sk<=32768"
    assert tuning.splitkv_problem(3, 64, 8, 1, 20000, 128, 128, "bf16") == a          # same buckets
    assert tuning.splitkv_problem(5, 64, 8, 1, 32768, 128, 128, "bf16") != a          # next batch bucket
    assert tuning.splitkv_problem(4, 64, 8, 1, 32769, 128, 128, "bf16") != a
    assert tuning.splitkv_problem(4, 32, 8, 1, 32768, 128, 128, "bf16") != a          # head geometry is exact


def test_cache_round_trip_and_persistence(tmp_path):
    c = tuning.TuningCache(str(tmp_path), ENV)
    prob = tuning.splitkv_problem(4, 64, 8, 1, 32768, 128, 128)
    assert c.query(tuning.SPLITKV, prob) is None and len(c) == 0
    c.insert(tuning.SPLITKV, prob, {"num_splits": 8, "latency_us": 104.0})
    assert c.query(tuning.SPLITKV, prob)["num_splits"] == 8
    doc = json.load(open(tmp_path / tuning.FILE_NAME))
    assert doc["schema"] == 1 and len(doc["records"]) == 1
    key = next(iter(doc["records"]))
    assert key.startswith("fmha_fwd_splitkv|7.0.test|gfx950-test||dtype=bf16")
    # another process (a fresh object) sees the record; another device or ROCm version does not
    assert tuning.TuningCache(str(tmp_path), ENV).query(tuning.SPLITKV, prob)["latency_us"] == 104.0
    assert tuning.TuningCache(str(tmp_path), dict(ENV, device_name="other")).query(tuning.SPLITKV, prob) is None
    assert [f for f in os.listdir(tmp_path)] == [tuning.FILE_NAME]  # no temporary files left behind
    c.clear()
    assert tuning.TuningCache(str(tmp_path), ENV).query(tuning.SPLITKV, prob) is None


def test_cache_survives_a_corrupt_file_and_honours_flush(tmp_path):
    (tmp_path / tuning.FILE_NAME).write_text("{not json")
    c = tuning.TuningCache(str(tmp_path), ENV)
    assert len(c) == 0
    c.insert(tuning.SPLITKV, "p", {"num_splits": 2})
    assert tuning.TuningCache(str(tmp_path), ENV).query(tuning.SPLITKV, "p") == {"num_splits": 2}
    flags.set_flag_value("FC_FLUSH_PROFILING_DB", "true")
    assert tuning.TuningCache(str(tmp_path), ENV).query(tuning.SPLITKV, "p") is None


def test_memory_only_cache_without_a_directory():
    c = tuning.TuningCache("", ENV)
    c.insert(tuning.SPLITKV, "p", {"num_splits": 3})
    assert c.path() is None and c.query(tuning.SPLITKV, "p")["num_splits"] == 3


def test_choose_num_splits_modes(tmp_path):
    c = tuning.TuningCache(str(tmp_path), ENV)
    args = (4, 64, 8, 1, 32768, 128, 128, "bf16")
    calls = []

    def heuristic():
        calls.append(1)
        return 5

    assert tuning.choose_num_splits(heuristic, *args, cache=c) == 5 and len(calls) == 1       # empty cache
    c.insert(tuning.SPLITKV, tuning.splitkv_problem(*args), {"num_splits": 8})
    assert tuning.choose_num_splits(heuristic, *args, cache=c) == 8 and len(calls) == 1       # cached winner
    flags.set_flag_value("FC_TUNING_MODE", "0")
    assert tuning.choose_num_splits(heuristic, *args, cache=c) == 5                            # heuristic only
    flags.set_flag_value("FC_TUNING_MODE", "2")
    c.insert(tuning.SPLITKV, tuning.splitkv_problem(*args), {"num_splits": 4000})
    assert tuning.choose_num_splits(heuristic, *args, cache=c) == 5                            # out-of-range record ignored


def test_tune_num_splits_picks_the_fastest_and_respects_existing_records(tmp_path):
    c = tuning.TuningCache(str(tmp_path), ENV)
    cost = {1: 9e-4, 2: 5e-4, 4: 2e-4, 8: 1e-4, 16: 1.5e-4}
    ran = []

    def timer(fn, cold, repeats):
        fn()
        assert (cold, repeats) == (2, 3)
        return cost[ran[-1]]

    flags.set_flag_value("FC_TUNING_NUM_COLD_ITERATION", "2")
    flags.set_flag_value("FC_TUNING_NUM_REPEATS", "3")
    rec = tuning.tune_num_splits(ran.append, timer, [16, 1, 2, 4, 8, 8, 0, 500], "p", nbytes=537_000_000, cache=c)
    assert ran == [1, 2, 4, 8, 16]
    assert rec["num_splits"] == 8 and abs(rec["latency_us"] - 100.0) < 1e-9 and abs(rec["bandwidth_gbs"] - 5370.0) < 1e-6
    assert set(rec["tried_us"]) == {"1", "2", "4", "8", "16"}
    ran.clear()
    assert tuning.tune_num_splits(ran.append, timer, [1, 2], "p", cache=c)["num_splits"] == 8 and ran == []  # cached
    flags.set_flag_value("FC_FORCE_PROFILING", "true")
    assert tuning.tune_num_splits(ran.append, timer, [1, 2], "p", cache=c)["num_splits"] == 2 and ran == [1, 2]
    with pytest.raises(ValueError):
        tuning.tune_num_splits(ran.append, timer, [0, 129], "q", cache=c)


def test_tuner_records_the_kernel_variant_with_the_split_count(tmp_path):
    """Pairs (split count, variant) are measured, a pair the problem cannot take is skipped, and the record carries the
    winning variant and the kernel that ran; choose_splitkv hands both back."""
    c = tuning.TuningCache(str(tmp_path), ENV)
    cost = {(2, 1): 4e-4, (2, 2): 3e-4, (4, 1): 2e-4, (4, 2): None}   # (4, 2) is refused
    ran = []

    def run(ns, variant):
        if cost[(ns, variant)] is None:
            raise ValueError("variant 2 needs an even head count")
        ran.append((ns, variant))
        return f"kernel<v{variant}>"

    def timer(fn, cold, repeats):
        fn()
        return cost[ran[-1]]

    rec = tuning.tune_num_splits(run, timer, [2, 4], "p2", cache=c, variants=(1, 2))
    assert (rec["num_splits"], rec["variant"], rec["kernel"]) == (4, 1, "kernel<v1>")
    assert set(rec["tried_us"]) == {"2/v1", "2/v2", "4/v1"}
    args = (4, 16, 4, 1, 2048, 128, 64, "bf16")
    c.insert(tuning.SPLITKV, tuning.splitkv_problem(*args), rec)
    assert tuning.choose_splitkv(lambda: 7, *args, cache=c) == (4, 1)
    assert tuning.choose_splitkv(lambda: 7, 8, 16, 4, 1, 2048, 128, 64, "bf16", cache=c) == (7, 0)   # another class: heuristic


def test_cached_variant_is_only_a_hint():
    """The tuning key buckets the query count and does not hold v_head_dim, so a record for one call can be served to a
    call the recorded kernel variant cannot take; the Python layer re-checks the variant's preconditions."""
    from flashck_amd.ops.fmha import fmha as F
    assert F._usable_variant(2, 40, 8, 3, 128, 128) == 2     # 15 packed rows: head pairs fit
    assert F._usable_variant(2, 40, 8, 4, 128, 128) == 0     # same query bucket, 20 packed rows: back to the library's choice
    assert F._usable_variant(2, 32, 8, 1, 128, 64) == 0      # qk_head_dim != v_head_dim
    assert F._usable_variant(2, 32, 8, 1, 256, 256) == 0     # head pairs exist for 64 and 128
    assert F._usable_variant(2, 21, 7, 1, 128, 128) == 0     # odd number of KV heads
    assert F._usable_variant(2, 32, 8, 1, 128, 128, plain=False) == 0   # score modifier / fp8 cache
    assert F._usable_variant(1, 21, 7, 9, 256, 64) == 1      # one head per workgroup fits every call
    assert F._usable_variant(7, 32, 8, 1, 128, 128) == 0     # nonsense in the cache


def test_decode_step_drops_a_cached_variant_it_cannot_take(monkeypatch, tmp_path):
    """fmha_decode_step with num_splits = 0 and a cache record (3 splits, head pairs) made with 3 new tokens: a step with
    4 new tokens falls into the same class but packs 20 query rows per KV head; it must run with variant 0."""
    import torch
    from flashck_amd.ops.fmha import fmha as F
    c = tuning.TuningCache(str(tmp_path), ENV)
    flags.set_flag_value("FC_TUNING_MODE", "1")
    c.insert(tuning.SPLITKV, tuning.splitkv_problem(2, 40, 8, 3, 256, 128, 128, "bf16"), dict(num_splits=3, variant=2))
    monkeypatch.setattr(tuning, "default_cache", lambda: c)
    seen = []
    monkeypatch.setattr(F, "_REQUIRE_GPU_TENSORS", False)
    monkeypatch.setattr(F, "fmha_fwd_appendkv", lambda *a, **k: None)
    monkeypatch.setattr(F, "fmha_fwd_splitkv", lambda *a, **k: seen.append((a[3], k["decode_variant"])) or (k["o_acc"], k["lse_acc"]))
    monkeypatch.setattr(F, "fmha_fwd_splitkv_combine", lambda lse, o, dt, **k: torch.empty(0))
    for n, want in ((3, 2), (4, 0)):
        q = torch.zeros(2, n, 40, 128, dtype=torch.bfloat16)
        kn = torch.zeros(2, n, 8, 128, dtype=torch.bfloat16)
        kc = torch.zeros(4, 128, 8, 128, dtype=torch.bfloat16)
        F.fmha_decode_step(q, kn, kn, kc, kc, torch.tensor([5, 9], dtype=torch.int32), torch.tensor([[0, 1], [2, 3]], dtype=torch.int32))
        assert seen[-1] == (3, want), (n, seen[-1])


def test_prefill_variant_tuner_and_lookup(tmp_path):
    c = tuning.TuningCache(str(tmp_path), ENV)
    cost = {1: 3e-3, 2: 2.5e-3, 3: None, 4: 2.8e-3}   # variant 3 is refused
    ran = []

    def run(v):
        if cost[v] is None:
            raise ValueError("cannot take it")
        ran.append(v)
        return f"kernel<v{v}>"

    def timer(fn, cold, repeats):
        fn()
        return cost[ran[-1]]

    problem = tuning.prefill_problem(32, 8, 128, 8000, 66000, 128, "bf16", 2)
    assert tuning.choose_prefill_variant(problem, cache=c) == 0
    rec = tuning.tune_prefill_variant(run, timer, (1, 2, 3, 4), problem, flops=int(1.7e12), cache=c)
    assert rec["variant"] == 2 and rec["kernel"] == "kernel<v2>" and set(rec["tried_us"]) == {"v1", "v2", "v4"} and abs(rec["tflops"] - 680.0) < 1e-6
    assert tuning.choose_prefill_variant(problem, cache=c) == 2
    assert tuning.choose_prefill_variant(tuning.prefill_problem(32, 8, 128, 8000, 66000, 128, "bf16", 0), cache=c) == 0   # another mask: another class
    assert tuning.prefill_problem(32, 8, 128, 8192, 65536, 128) == tuning.prefill_problem(32, 8, 128, 5000, 40000, 128)  # buckets
    flags.set_flag_value("FC_TUNING_MODE", "0")
    assert tuning.choose_prefill_variant(problem, cache=c) == 0
    flags.set_flag_value("FC_TUNING_MODE", "2")
    from flashck_amd.ops.fmha import fmha as F
    assert F._usable_prefill_variant(3, 128, 128, 300, 128) == 3 and F._usable_prefill_variant(3, 128, 128, 300, 0) == 3
    assert F._usable_prefill_variant(3, 256, 256, 300, 128) == 0 and F._usable_prefill_variant(2, 128, 128, 128, 128) == 0
    assert F._usable_prefill_variant(4, 128, 128, 300, 48) == 0 and F._usable_prefill_variant(1, 256, 64, 1, 7) == 1
