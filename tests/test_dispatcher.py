"""DynamicDispatcher with fake backends, an injected timer and a temporary cache directory
(API of tritonix/dispatcher.py:38-175)."""
import hashlib
import json
import os

import pytest
import torch

from tritonix_amd.dispatcher import DynamicDispatcher, _disk_key, _tuning_key, dynamic_dispatch


def fast(a, b):
    """fast doc"""
    return "fast"


def slow(a, b):
    return "slow"


def broken(a, b):
    raise RuntimeError("no such kernel")


class Timer:
    def __init__(self, table):
        self.table, self.calls = table, []

    def __call__(self, fn, warmup=None, rep=None):
        out = fn()
        self.calls.append((out, warmup, rep))
        return self.table[out]


@pytest.fixture
def cache_dir(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITONIX_CACHE_DIR", str(tmp_path))
    return tmp_path


def test_tuning_key_matches_the_hand_trace(traces):
    a = torch.empty(1024, 512, dtype=torch.float16)
    b = torch.empty(512, 768, dtype=torch.float16)
    assert list(_tuning_key(["a", "b"], (a, b), {}, ["a", "b"])) == traces["dispatch_key_c1"]
    # keyed scalars contribute their value; un-keyed tensors are appended after the keyed ones
    assert _tuning_key(["k", "a"], (a,), {"k": 7, "b": b}, ["a", "b", "k"]) == (
        7, 1024, 512, "torch.float16", 512, 768, "torch.float16")
    assert _tuning_key(["zzz"], (a,), {}, ["a"]) == (1024, 512, "torch.float16")


def test_disk_key_closed_form():
    key = (8, 8, "torch.int8")
    want = hashlib.sha256("-".join(["op", str(["a", "b"]), str(key)]).encode()).hexdigest()
    assert _disk_key("op", ["b", "a"], key) == want


def test_picks_the_fastest_and_caches(cache_dir):
    t = Timer({"fast": 1.0, "slow": 2.0})
    d = dynamic_dispatch({"s": slow, "f": fast}, key=["a", "b"], bench_fn=t, warmup=3, rep=7)
    assert d.__name__ == "slow"            # named after its first backend
    a, b = torch.empty(4, 2), torch.empty(2, 3)
    assert d(a, b) == "fast"
    key = (4, 2, "torch.float32", 2, 3, "torch.float32")
    assert d.cache == {key: "f"} and d.timings == {key: {"s": 2.0, "f": 1.0}}
    assert d.best_config() == {key: "f"} and d.best_config() is not d.cache
    assert [c[1:] for c in t.calls] == [(3, 7), (3, 7)]
    n = len(t.calls)
    assert d(a, b) == "fast" and len(t.calls) == n     # second call: no benchmarking
    # the record on disk has the reference's schema
    files = list(cache_dir.rglob("backend_dispatch.json"))
    assert len(files) == 1
    rec = json.loads(files[0].read_text())
    assert rec == {"op": "slow", "key": list(key), "winner": "f", "timings": {"s": 2.0, "f": 1.0}}
    assert files[0].parent.name == _disk_key("slow", ["s", "f"], key)


def test_disk_record_short_circuits_benchmarking(cache_dir):
    a, b = torch.empty(4, 2), torch.empty(2, 3)
    d1 = dynamic_dispatch({"s": slow, "f": fast}, key=["a", "b"], bench_fn=Timer({"fast": 1.0, "slow": 2.0}))
    d1(a, b)
    t2 = Timer({"fast": 9.0, "slow": 0.1})
    d2 = dynamic_dispatch({"s": slow, "f": fast}, key=["a", "b"], bench_fn=t2)
    assert d2(a, b) == "fast" and t2.calls == []
    assert len(d2.cache) == 1
    d2.clear_cache()
    assert d2.cache == {} and d2.timings == {}
    assert d2(a, b) == "fast" and t2.calls == []       # clear_cache is memory-only
    d3 = dynamic_dispatch({"s": slow, "f": fast}, key=["a", "b"], bench_fn=t2, use_disk_cache=False)
    assert d3(a, b) == "slow"


def test_failing_backend_only_loses(cache_dir):
    d = dynamic_dispatch({"x": broken, "f": fast}, key=["a", "b"], bench_fn=Timer({"fast": 1.0}))
    assert d(torch.empty(1, 1), torch.empty(1, 1)) == "fast"
    assert list(d.timings.values()) == [{"f": 1.0}]
    d = dynamic_dispatch({"x": broken}, key=["a", "b"], bench_fn=Timer({}))
    with pytest.raises(RuntimeError, match="All backends failed"):
        d(torch.empty(1, 1), torch.empty(1, 1))


def test_no_backends_and_decorator_mode(cache_dir):
    @dynamic_dispatch(key=["a"])
    def op(a, b):
        """op doc"""

    assert isinstance(op, DynamicDispatcher) and op.__name__ == "op" and op.__doc__ == "op doc"
    with pytest.raises(RuntimeError, match="No backends registered"):
        op(1, 2)
    assert op.register("f", fast) is op


def test_force_backend(cache_dir):
    t = Timer({"fast": 1.0, "slow": 2.0})
    d = dynamic_dispatch({"s": slow, "f": fast}, key=["a", "b"], bench_fn=t)
    a, b = torch.empty(2, 2), torch.empty(2, 2)
    with d.force_backend("s"):
        assert d(a, b) == "slow"
    assert t.calls == [] and d.cache == {}            # forcing bypasses timing and caching
    with pytest.raises(KeyError):
        with d.force_backend("nope"):
            pass
    with pytest.raises(ZeroDivisionError):
        with d.force_backend("s"):
            1 / 0
    assert d(a, b) == "fast"                           # the forced slot was released
    d.alias("quick", "f")
    with d.force_backend("quick"):
        assert d(a, b) == "fast"


def test_package_matmul_dispatcher_shape():
    from tritonix_amd import matmul

    assert matmul.__name__ == "triton_matmul"
    # the reference's two backend names and no other (tritonix/ops/matmul.py:291-293)
    assert set(matmul._backends) == {"triton", "pytorch"}
    # the vendor library is reachable when forced, but is not a contender: only the HIP engine is timed
    assert set(matmul._contenders()) == {"triton"}
    assert matmul._arg_names == ["a", "b"] and matmul._key_names == ["a", "b"]
    with matmul.force_backend("pytorch"):
        out = matmul(torch.ones(2, 3), torch.ones(3, 4))
    assert torch.equal(out, torch.full((2, 4), 3.0))
    with matmul.force_backend("hip"):                  # alias of "triton"
        assert matmul._forced == "triton"


def test_unraced_backend_is_never_timed_and_never_wins(cache_dir):
    t = Timer({"fast": 5.0, "slow": 9.0, "oracle": 0.1})
    d = dynamic_dispatch({"s": slow, "f": fast}, key=["a", "b"], bench_fn=t)
    assert d.register("ref", lambda a, b: "oracle", raced=False) is d
    a, b = torch.empty(4, 2), torch.empty(2, 3)
    assert d(a, b) == "fast"
    assert [c[0] for c in t.calls] == ["slow", "fast"]              # "ref" was not timed
    key = (4, 2, "torch.float32", 2, 3, "torch.float32")
    assert d.cache == {key: "f"} and "ref" not in d.timings[key]
    with d.force_backend("ref"):
        assert d(a, b) == "oracle"
    # a record on disk that names an un-raced backend as the winner (written when it was still raced) is ignored
    d2 = dynamic_dispatch({"s": slow, "f": fast}, key=["a", "b"], bench_fn=Timer({"fast": 1.0, "slow": 2.0, "oracle": 0.1}))
    d2.register("ref", lambda a, b: "oracle")
    c, e = torch.empty(5, 2), torch.empty(2, 3)
    assert d2(c, e) == "oracle"
    d3 = dynamic_dispatch({"s": slow, "f": fast}, key=["a", "b"], bench_fn=Timer({"fast": 1.0, "slow": 2.0}))
    d3.register("ref", lambda a, b: "oracle", raced=False)
    assert d3(c, e) == "fast"
    # registering again as raced puts it back into the race
    d3.register("ref", lambda a, b: "oracle", raced=True)
    assert "ref" in d3._contenders()


def test_default_timer_is_the_package_do_bench(cache_dir, monkeypatch):
    """Without ``bench_fn`` the race is timed by ``tritonix_amd.testing.do_bench`` with the dispatcher's budgets."""
    import tritonix_amd.testing

    seen = []

    def stand_in(fn, warmup=25, rep=100):
        seen.append((warmup, rep))
        return {"fast": 1.0, "slow": 2.0}[fn()]

    monkeypatch.setattr(tritonix_amd.testing, "do_bench", stand_in)
    d = dynamic_dispatch({"s": slow, "f": fast}, key=["a", "b"], warmup=5, rep=11)
    assert d(torch.empty(3, 3), torch.empty(3, 3)) == "fast"
    assert seen == [(5, 11), (5, 11)]
