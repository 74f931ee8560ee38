"""MonotonicCascadeTrie: the known answers of the reference's tests/test_trie.py (12 cases) plus the
hand-derived centre-out enumeration orders."""
import pytest

from tritonix_amd.utils.pruners import MonotonicCascadeTrie
from tritonix_amd.utils.spaces import Choice, SpaceConfig


def make(*dims):
    return MonotonicCascadeTrie(SpaceConfig({str(i): Choice(range(d)) for i, d in enumerate(dims)}))


def test_shape_is_kept():
    assert make(4, 5, 3).shape == (4, 5, 3)
    assert make(4, 5, 3).dimensions == 3


def test_zero_sized_dimension_raises():
    with pytest.raises(ValueError):
        make(4, 0, 3)


def test_prune_dominates_upwards_only():
    t = make(4, 4, 4, 4)
    t.prune((2, 2, 0, 0))
    assert t.is_pruned((2, 2, 0, 0))
    assert t.is_pruned((3, 3, 3, 3))
    assert not t.is_pruned((2, 1, 3, 3))


def test_general_failure_replaces_specific_one():
    t = make(4, 4, 4, 4)
    t.prune((2, 2, 2, 2))
    t.prune((1, 1, 1, 1))
    assert t._minimal_failures == [(1, 1, 1, 1)]


def test_minimal_failures_reduce_even_outside_the_shape():
    t = make(4, 4, 4, 4)
    for f in [(1, 4, 4, 1), (3, 3, 3, 0), (0, 4, 0, 1), (1, 3, 0, 0)]:
        t.prune(f)
    assert set(t._minimal_failures) == {(1, 3, 0, 0), (0, 4, 0, 1)}


def test_prefix_doomed_uses_the_zero_completion():
    t = make(4, 4, 4, 4)
    t.prune((1, 2, 0, 1))
    assert not t._is_prefix_doomed((1, 2))
    assert not t._is_prefix_doomed((1, 2, 0))
    t.prune((1, 2, 0, 0))
    assert t._is_prefix_doomed((1, 2))
    assert t._is_prefix_doomed((1, 2, 0))
    assert not t._is_prefix_doomed((1, 1))
    assert not t._is_prefix_doomed(())


def test_nothing_pruned_initially():
    assert not make(4, 4, 3).is_pruned((2, 2, 1))


def test_non_dominated_configs_survive():
    t = make(4, 4, 3)
    t.prune((2, 1, 0))
    assert not t.is_pruned((1, 3, 2))
    assert not t.is_pruned((3, 0, 1))


def test_dominating_prune_shrinks_the_antichain():
    t = make(4, 4, 3)
    t.prune((2, 1, 0))
    t.prune((1, 2, 1))
    assert not t.is_pruned((1, 2, 0))
    assert t.is_pruned((1, 3, 1))
    t.prune((1, 2, 0))
    assert (1, 2, 0) in t._minimal_failures
    assert (1, 2, 1) not in t._minimal_failures
    assert t.is_pruned((1, 2, 1))


def test_generate_all_counts_the_survivors():
    t = make(3, 3, 3)
    t.prune((1, 1, 0))
    got = list(t.generate_all_unpruned())
    assert len(got) == 15  # 27 minus the 2*2*3 dominated ones
    assert (1, 1, 0) not in got and (2, 2, 2) not in got
    assert (1, 0, 2) in got and (0, 2, 1) in got
    assert got == sorted(got)  # lexicographic


def test_random_generator_only_returns_survivors():
    t = make(4, 4, 3)
    t.prune((2, 1, 0))
    t.prune((1, 2, 0))
    for _ in range(20):
        cfg = t.get_random_unpruned()
        assert cfg is not None and not t.is_pruned(cfg)


def test_fully_pruned_space():
    t = make(2, 2)
    t.prune((0, 0))
    assert t.get_random_unpruned() is None
    assert t.get_mid_point_unpruned() is None
    assert list(t.generate_all_unpruned()) == []
    assert list(t.generate_all_unpruned_midpoint()) == []


def test_wrong_length_config_raises():
    with pytest.raises(ValueError):
        make(3, 3).is_pruned((1,))


# ---- hand-derived enumeration orders -------------------------------------------------
def test_midpoint_orders(traces):
    tr = traces["midpoint_3x2"]
    t = make(3, 2)
    assert [list(c) for c in t.generate_all_unpruned_midpoint()] == tr["none"]
    t.prune((1, 1))
    assert [list(c) for c in t.generate_all_unpruned_midpoint()] == tr["after_prune_1_1"]
    t.prune((1, 0))
    assert [list(c) for c in t.generate_all_unpruned_midpoint()] == tr["after_prune_1_1_and_1_0"]
    assert [c[0] for c in make(4).generate_all_unpruned_midpoint()] == traces["midpoint_order_size4"]
    assert make(3, 2).get_mid_point_unpruned() == (1, 1)


def test_midpoint_generator_is_lazy():
    # a prune issued between two yields changes what comes next
    t = make(3, 2)
    it = t.generate_all_unpruned_midpoint()
    assert next(it) == (1, 1)
    t.prune((1, 0))  # kills (1,0), (2,0), (2,1) and everything above
    assert list(it) == [(0, 1), (0, 0)]


def test_midpoint_and_lexicographic_agree_as_sets():
    t = make(4, 3, 3)
    t.prune((2, 1, 1))
    t.prune((1, 2, 2))
    a = set(t.generate_all_unpruned())
    b = set(t.generate_all_unpruned_midpoint())
    brute = {(i, j, k) for i in range(4) for j in range(3) for k in range(3)
             if not ((i >= 2 and j >= 1 and k >= 1) or (i >= 1 and j >= 2 and k >= 2))}
    assert a == b == brute
