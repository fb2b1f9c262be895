"""Persisted tuning choices: which launch parameter won for a class of problems on this machine.

What is kept from the reference's profiling engine is its cache, not its code generator: a record is found by
(rocm_version, device_name, setting, problem) exactly as ProfilingDB::Query does (core/profiling/profiling_db.cc:64-71)
and stores the winner with its measurements (instance name, split_k, latency, tflops, bandwidth in that table; here
the choice - for split-KV the number of splits - with latency and bandwidth).  The store is one JSON file under
FC_TUNING_DB_DIR, rewritten atomically; with no directory set the cache lives in memory only.

FC_TUNING_MODE: 0 = always the built-in heuristic, 2 (default) = a cached choice when there is one, else the heuristic,
1 = as 2, and `tune_num_splits` re-measures even when a record exists if FC_FORCE_PROFILING is set.
"""
import json
import os
import tempfile
import threading
from typing import Callable, Dict, Iterable, Optional

from . import flags

__all__ = ["TuningCache", "default_cache", "splitkv_problem", "choose_num_splits", "choose_splitkv", "tune_num_splits",
           "prefill_problem", "choose_prefill_variant", "tune_prefill_variant", "environment"]

FILE_NAME = "flashck_amd_tuning.json"
SCHEMA = 1


def _bucket_pow2(x: int) -> int:
    """Smallest power of two >= x (problems that round to the same bucket share a record)."""
    x = max(int(x), 1)
    return 1 << (x - 1).bit_length()


def splitkv_problem(batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k, head_dim, page_size=0, dtype="bf16") -> str:
    """Key of a split-KV problem class: exact head geometry, power-of-two buckets for batch, query rows and KV length."""
    return (f"dtype={dtype},hq={int(q_num_heads)},hk={int(kv_num_heads)},d={int(head_dim)},page={int(page_size)},"
            f"b<={_bucket_pow2(batch)},sq<={_bucket_pow2(seqlen_q)},sk<={_bucket_pow2(max_seqlen_k)}")


def environment() -> Dict[str, str]:
    """(rocm_version, device_name) of the current process; needs torch and, for the device name, a GPU."""
    import torch
    name = torch.cuda.get_device_name() if torch.cuda.is_available() else "cpu"
    return {"rocm_version": str(getattr(torch.version, "hip", None) or "none"), "device_name": name}


class TuningCache:
    def __init__(self, directory: Optional[str] = None, env: Optional[Dict[str, str]] = None):
        self._dir = directory
        self._env = env
        self._lock = threading.Lock()
        self._records: Optional[Dict[str, dict]] = None

    # -- storage -------------------------------------------------------------------------------------------------
    def _directory(self) -> str:
        return self._dir if self._dir is not None else flags.flag("FC_TUNING_DB_DIR")

    def path(self) -> Optional[str]:
        d = self._directory()
        return os.path.join(d, FILE_NAME) if d else None

    def _load(self) -> Dict[str, dict]:
        if self._records is None:
            self._records = {}
            p = self.path()
            if p and os.path.exists(p) and not flags.flag("FC_FLUSH_PROFILING_DB"):
                try:
                    with open(p) as f:
                        doc = json.load(f)
                    if isinstance(doc, dict) and doc.get("schema") == SCHEMA and isinstance(doc.get("records"), dict):
                        self._records = doc["records"]
                except (OSError, ValueError):
                    pass  # an unreadable cache is an empty cache
        return self._records

    def _save(self) -> None:
        p = self.path()
        if not p:
            return
        os.makedirs(os.path.dirname(p), exist_ok=True)
        fd, tmp = tempfile.mkstemp(prefix=FILE_NAME + ".", dir=os.path.dirname(p))
        try:
            with os.fdopen(fd, "w") as f:
                json.dump({"schema": SCHEMA, "records": self._records}, f, indent=1, sort_keys=True)
            os.replace(tmp, p)
        except BaseException:
            if os.path.exists(tmp):
                os.unlink(tmp)
            raise

    # -- records -------------------------------------------------------------------------------------------------
    def _key(self, kind: str, setting: str, problem: str) -> str:
        env = self._env if self._env is not None else environment()
        return "|".join((kind, env["rocm_version"], env["device_name"], setting, problem))

    def query(self, kind: str, problem: str, setting: str = "") -> Optional[dict]:
        with self._lock:
            if not self._load():
                return None  # nothing cached: do not even ask for the device name
            return self._load().get(self._key(kind, setting, problem))

    def insert(self, kind: str, problem: str, choice: dict, setting: str = "") -> None:
        with self._lock:
            self._load()[self._key(kind, setting, problem)] = dict(choice)
            self._save()

    def clear(self) -> None:
        with self._lock:
            self._records = {}
            self._save()

    def __len__(self) -> int:
        with self._lock:
            return len(self._load())


_default: Optional[TuningCache] = None


def default_cache() -> TuningCache:
    global _default
    if _default is None:
        _default = TuningCache()
    return _default


SPLITKV = "fmha_fwd_splitkv"


def choose_splitkv(heuristic: Callable[[], int], batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k, head_dim,
                   page_size=0, dtype="bf16", cache: Optional[TuningCache] = None):
    """(split count, kernel variant) for a split-KV launch: the cached winner for the problem class when tuning is on,
    else (`heuristic()`, 0 = the library picks the variant)."""
    if flags.flag("FC_TUNING_MODE") != 0:
        rec = (cache or default_cache()).query(
            SPLITKV, splitkv_problem(batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k, head_dim, page_size, dtype))
        if rec is not None and 1 <= int(rec.get("num_splits", 0)) <= 128:
            variant = int(rec.get("variant", 0))
            return int(rec["num_splits"]), (variant if variant in (0, 1, 2, 3, 4) else 0)
    return int(heuristic()), 0


def choose_num_splits(heuristic: Callable[[], int], batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k, head_dim,
                      page_size=0, dtype="bf16", cache: Optional[TuningCache] = None) -> int:
    """Split count alone (see choose_splitkv)."""
    return choose_splitkv(heuristic, batch, q_num_heads, kv_num_heads, seqlen_q, max_seqlen_k, head_dim, page_size, dtype, cache)[0]


def tune_num_splits(run: Callable[..., Optional[str]], timer: Callable[[Callable[[], None], int, int], float],
                    candidates: Iterable[int], problem: str, nbytes: int = 0, cache: Optional[TuningCache] = None,
                    variants: Iterable[int] = (0,)) -> dict:
    """Measure `run(num_splits)` - with more than the default variant: `run(num_splits, variant)` - for every candidate
    pair and record the fastest for `problem`, as ProfilingDB keeps (instance, split_k) per problem
    (core/profiling/profiling_db.cc:64-71).  `run` may return the name of the kernel it launched; a pair the problem
    cannot take (run raises ValueError / NotImplementedError) is skipped.

    `timer(fn, cold, repeats)` returns the mean seconds of one call of fn (on the GPU: events around `repeats` launches
    after `cold` untimed ones).  Returns the stored record.  An existing record is kept unless FC_FORCE_PROFILING is set.
    """
    cache = cache or default_cache()
    if not flags.flag("FC_FORCE_PROFILING"):
        rec = cache.query(SPLITKV, problem)
        if rec is not None:
            return rec
    cold, repeats = flags.flag("FC_TUNING_NUM_COLD_ITERATION"), flags.flag("FC_TUNING_NUM_REPEATS")
    best = None
    tried = {}
    variants = sorted(set(int(v) for v in variants)) or [0]
    for ns in sorted(set(int(c) for c in candidates)):
        if not 1 <= ns <= 128:
            continue
        for variant in variants:
            names = []

            def call(ns=ns, variant=variant):
                names.append(run(ns) if variants == [0] else run(ns, variant))

            try:
                t = float(timer(call, cold, repeats))
            except (ValueError, NotImplementedError):
                continue  # a variant this problem cannot take
            kernel = names[-1] if names else None
            tried[str(ns) if variants == [0] else f"{ns}/v{variant}"] = t * 1e6
            if flags.flag("FC_TUNING_LOG"):
                print(f"[flashck tuning] {problem}: num_splits={ns} variant={variant} {t * 1e6:.1f} us")
            if best is None or t < best[1]:
                best = (ns, t, variant, kernel)
    if best is None:
        raise ValueError("no valid num_splits candidate (1..128)")
    rec = {"num_splits": best[0], "variant": best[2], "latency_us": best[1] * 1e6, "tried_us": tried}
    if isinstance(best[3], str):
        rec["kernel"] = best[3]
    if nbytes:
        rec["bandwidth_gbs"] = nbytes / best[1] / 1e9
    cache.insert(SPLITKV, problem, rec)
    return rec


PREFILL = "fmha_fwd_prefill"


def prefill_problem(q_num_heads, kv_num_heads, head_dim, max_seqlen_q, total_q, page_size=0, dtype="bf16", mask_type=2) -> str:
    """Key of a prefill problem class: exact head geometry and mask type, power-of-two buckets for the longest query run
    and the packed query rows."""
    return (f"dtype={dtype},hq={int(q_num_heads)},hk={int(kv_num_heads)},d={int(head_dim)},page={int(page_size)},mask={int(mask_type)},"
            f"sq<={_bucket_pow2(max_seqlen_q)},tq<={_bucket_pow2(total_q)}")


def choose_prefill_variant(problem: str, cache: Optional[TuningCache] = None) -> int:
    """Tile variant recorded for the problem class when tuning is on, else 0 (the library's choice)."""
    if flags.flag("FC_TUNING_MODE") != 0:
        rec = (cache or default_cache()).query(PREFILL, problem)
        if rec is not None and 0 <= int(rec.get("variant", 0)) <= 4:
            return int(rec["variant"])
    return 0


def tune_prefill_variant(run: Callable[[int], Optional[str]], timer: Callable[[Callable[[], None], int, int], float],
                         variants: Iterable[int], problem: str, flops: int = 0, cache: Optional[TuningCache] = None) -> dict:
    """Measure `run(variant)` for every tile variant and record the fastest for `problem` - the (shape -> tile instance)
    half of what ProfilingDB keeps (core/profiling/profiling_db.cc:64-71).  A variant the problem cannot take (run raises
    ValueError / NotImplementedError) is skipped.  An existing record is kept unless FC_FORCE_PROFILING is set."""
    cache = cache or default_cache()
    if not flags.flag("FC_FORCE_PROFILING"):
        rec = cache.query(PREFILL, problem)
        if rec is not None:
            return rec
    cold, repeats = flags.flag("FC_TUNING_NUM_COLD_ITERATION"), flags.flag("FC_TUNING_NUM_REPEATS")
    best, tried = None, {}
    for variant in sorted(set(int(v) for v in variants)):
        names = []
        try:
            t = float(timer(lambda v=variant: names.append(run(v)), cold, repeats))
        except (ValueError, NotImplementedError):
            continue
        tried[f"v{variant}"] = t * 1e6
        if flags.flag("FC_TUNING_LOG"):
            print(f"[flashck tuning] {problem}: prefill_variant={variant} {t * 1e6:.1f} us")
        if best is None or t < best[1]:
            best = (variant, t, names[-1] if names else None)
    if best is None:
        raise ValueError("no prefill variant this problem can take")
    rec = {"variant": best[0], "latency_us": best[1] * 1e6, "tried_us": tried}
    if isinstance(best[2], str):
        rec["kernel"] = best[2]
    if flops:
        rec["tflops"] = flops / best[1] / 1e12
    cache.insert(PREFILL, problem, rec)
    return rec


def gpu_timer(fn: Callable[[], None], cold: int, repeats: int) -> float:
    """Mean seconds per call of fn, by events on the current stream."""
    import torch
    for _ in range(cold):
        fn()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(repeats):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) * 1e-3 / max(repeats, 1)
