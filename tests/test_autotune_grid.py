"""Grid tuner driven by a fake launcher and a deterministic timer: visit order, OOM pruning, SKIP handling,
max_configs (hand-derived from tritonix/autotune.py:75-140; see tests/golden/hand_traces.json)."""
import pytest

from tritonix_amd.autotune import Choice, OutOfResources, PowerOfTwo, Range, TunableKernel, tunable


class FakeKernel:
    def __init__(self):
        self.specialize_keys = None
        self.hooked = []

    def __getitem__(self, grid):
        return ("launcher-for", grid)

    def add_pre_run_hook(self, h):
        self.hooked.append(h)


def make_kernel():
    return tunable(keys=["m"], space={"bm": PowerOfTwo(32, 128), "ns": Range(2, 3), "gm": Choice([4, 8])},
                   memory_params={"bm"})(FakeKernel())


class Harness:
    """launcher + timer pair: the timer calls the thunk once (so vetoes surface) and returns formula(cfg)."""

    def __init__(self, formula, oom=lambda c: c["bm"] == 128, veto=lambda c: False):
        self.formula, self.oom, self.veto = formula, oom, veto
        self.launched, self.oom_launches, self.current = [], 0, None

    def launcher(self, cfg):
        self.current = cfg
        if self.oom(cfg):
            self.oom_launches += 1
            raise OutOfResources(200000, 163840, "shared memory")
        if self.veto(cfg):
            raise ValueError("vetoed")
        self.launched.append([cfg["bm"], cfg["ns"], cfg["gm"]])

    def timer(self, fn, warmup=None, rep=None):
        fn()
        return self.formula(self.current)


def test_decorator_wires_the_kernel():
    k = make_kernel()
    assert isinstance(k, TunableKernel)
    assert k.kernel.specialize_keys == ["m"]
    assert k.memory_params == {"bm", "num_stages"}      # num_stages is always added
    assert k[(3, 4)] == ("launcher-for", (3, 4))        # __getitem__ passes through
    k.add_pre_run_hook(print)                           # __getattr__ passes through
    assert k.kernel.hooked == [print]
    assert TunableKernel(kernel=k, keys=[], space={}, memory_params=set()).kernel is k.kernel


def test_configs_is_the_cartesian_product_in_declaration_order():
    k = make_kernel()
    cfgs = k.configs()
    assert len(cfgs) == 12
    assert cfgs[0] == {"bm": 32, "ns": 2, "gm": 4} and cfgs[1] == {"bm": 32, "ns": 2, "gm": 8}
    assert cfgs[-1] == {"bm": 128, "ns": 3, "gm": 8}
    assert len(k.configs(filter_fn=lambda c: c["gm"] == 8)) == 6


def test_trie_dimensions_follow_the_space_declaration():
    k = tunable(keys=[], space={"block_m": PowerOfTwo(64, 256), "group_m": Choice([4, 8]), "num_stages": Range(2, 4),
                                "block_k": PowerOfTwo(32, 64)},
                memory_params={"block_k", "block_m"})(FakeKernel())
    trie, names, values = k._build_trie()
    assert names == ["block_m", "num_stages", "block_k"]
    assert values == [[64, 128, 256], [2, 3, 4], [32, 64]]
    assert trie.shape == (3, 3, 2)


def test_timer_A_small_tiles_win_and_oom_is_never_reached(traces):
    want = traces["tuner"]["timer_A"]
    h = Harness(lambda c: c["bm"] / 32 + c["ns"] + c["gm"] / 8)
    best = make_kernel().tune(h.launcher, bench_fn=h.timer)
    assert h.launched == want["evaluated"]
    assert h.oom_launches == want["oom_launches"] == 0
    assert best == want["best"]


def test_timer_B_big_tiles_win_until_the_oom_boundary(traces):
    want = traces["tuner"]["timer_B"]
    h = Harness(lambda c: 4 - c["bm"] / 64 + c["ns"] + c["gm"] / 8)
    best = make_kernel().tune(h.launcher, bench_fn=h.timer)
    assert h.launched == want["evaluated"]
    assert h.oom_launches == want["oom_launches"] == 1   # one failed launch, then the inner loop breaks
    assert best == want["best"]


def test_max_configs_caps_the_number_of_timed_configs(traces):
    for formula in (lambda c: c["bm"] / 32 + c["ns"] + c["gm"] / 8, lambda c: 4 - c["bm"] / 64 + c["ns"] + c["gm"] / 8):
        h = Harness(formula)
        assert make_kernel().tune(h.launcher, bench_fn=h.timer, max_configs=1) == traces["tuner"]["max_configs_1"]
        assert len(h.launched) == 1


def test_value_error_skips_one_config_and_is_not_counted():
    h = Harness(lambda c: 4 - c["bm"] / 64 + c["ns"] + c["gm"] / 8, veto=lambda c: c == {"bm": 64, "ns": 2, "gm": 4})
    best = make_kernel().tune(h.launcher, bench_fn=h.timer, max_configs=2)
    assert h.launched == [[64, 2, 8], [64, 3, 4]]
    assert best == {"bm": 64, "ns": 2, "gm": 8}


def test_filter_fn_and_nothing_runs():
    h = Harness(lambda c: 1.0)
    assert make_kernel().tune(h.launcher, bench_fn=h.timer, filter_fn=lambda c: False) is None
    assert h.launched == []
    h = Harness(lambda c: 1.0, oom=lambda c: True)
    assert make_kernel().tune(h.launcher, bench_fn=h.timer) is None


def test_oom_prunes_everything_above_in_all_memory_dimensions():
    k = tunable(keys=[], space={"bm": PowerOfTwo(32, 128), "bn": PowerOfTwo(32, 128), "num_stages": Range(2, 3)},
                memory_params={"bm", "bn"})(FakeKernel())
    seen = []

    def launcher(cfg):
        seen.append((cfg["bm"], cfg["bn"], cfg["num_stages"]))
        if cfg["bm"] * cfg["bn"] * cfg["num_stages"] > 64 * 64 * 3:
            raise OutOfResources(1, 0, "shared memory")

    def timer(fn, warmup=None, rep=None):
        fn()
        return 1.0  # flat: the unimodal pruner never fires

    k.tune(launcher, bench_fn=timer)
    failed = [s for s in seen if s[0] * s[1] * s[2] > 64 * 64 * 3]
    # nothing was launched that is >= an earlier failure in every memory coordinate
    for pos, s in enumerate(seen):
        for g in seen[:pos]:
            if g in failed:
                assert not all(x >= y for x, y in zip(s, g)), (s, g)
    ok = {s for s in seen if s not in failed}
    assert ok == {(bm, bn, ns) for bm in (32, 64, 128) for bn in (32, 64, 128) for ns in (2, 3)
                  if bm * bn * ns <= 64 * 64 * 3}


def test_other_exceptions_propagate():
    def launcher(cfg):
        raise KeyError("boom")

    def timer(fn, warmup=None, rep=None):
        fn()
        return 1.0

    with pytest.raises(KeyError):
        make_kernel().tune(launcher, bench_fn=timer)


def test_bayesian_needs_ax():
    try:
        import ax  # noqa: F401
    except ImportError:
        with pytest.raises(ImportError):
            make_kernel().tune(lambda cfg: None, method="bayesian", bench_fn=lambda fn, warmup=None, rep=None: 1.0)
