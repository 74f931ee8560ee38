"""Property tests of the two pruners against their brute-force definitions.

The trie (tritonix/utils/pruners.py:15-169 of the reference) must agree, on every index of a small space, with
"some recorded failure is <= the index in every coordinate", whatever the order failures arrive in; its
generators must enumerate exactly the complement.  The unimodal pruner (tritonix/utils/pruners.py:172-225) must
never cut the minimum of a function that really is unimodal along every coordinate.
"""
import itertools

from hypothesis import given, settings, strategies as st

from tritonix_amd.utils.pruners import CoordinateUnimodalFunction, MonotonicCascadeTrie
from tritonix_amd.utils.spaces import Choice, SpaceConfig


def space_of(shape):
    return SpaceConfig({f"p{i}": Choice(list(range(n))) for i, n in enumerate(shape)})


shapes = st.lists(st.integers(1, 4), min_size=1, max_size=4).map(tuple)


@st.composite
def shape_and_points(draw, max_points=8):
    shape = draw(shapes)
    point = st.tuples(*[st.integers(0, n - 1) for n in shape])
    return shape, draw(st.lists(point, min_size=0, max_size=max_points))


@settings(max_examples=200, deadline=None)
@given(shape_and_points())
def test_trie_matches_the_dominance_definition(case):
    shape, failures = case
    trie = MonotonicCascadeTrie(space_of(shape))
    for f in failures:
        trie.prune(f)
    every = list(itertools.product(*[range(n) for n in shape]))
    brute = {idx for idx in every if any(all(i >= f for i, f in zip(idx, fail)) for fail in failures)}
    assert {idx for idx in every if trie.is_pruned(idx)} == brute
    survivors = [idx for idx in every if idx not in brute]
    assert list(trie.generate_all_unpruned()) == survivors                       # lexicographic
    assert sorted(trie.generate_all_unpruned_midpoint()) == survivors            # same set, centre-out order
    first = trie.get_mid_point_unpruned()
    assert (first is None) == (not survivors)
    if survivors:
        assert first == next(iter(trie.generate_all_unpruned_midpoint()))
        assert trie.get_random_unpruned() in survivors
    # the stored failures are an antichain: none dominates another
    mins = trie._minimal_failures
    assert all(not all(a >= b for a, b in zip(x, y)) for x in mins for y in mins if x != y)


@settings(max_examples=100, deadline=None)
@given(shape_and_points(), st.randoms(use_true_random=False))
def test_trie_does_not_depend_on_arrival_order(case, rnd):
    shape, failures = case
    one, two = MonotonicCascadeTrie(space_of(shape)), MonotonicCascadeTrie(space_of(shape))
    for f in failures:
        one.prune(f)
    shuffled = list(failures)
    rnd.shuffle(shuffled)
    for f in shuffled:
        two.prune(f)
    assert sorted(one._minimal_failures) == sorted(two._minimal_failures)
    assert list(one.generate_all_unpruned()) == list(two.generate_all_unpruned())


@st.composite
def separable_unimodal(draw):
    """f(idx) = sum_d g_d(idx[d]) with every g_d strictly decreasing to its minimum, then strictly increasing."""
    shape = draw(st.lists(st.integers(2, 5), min_size=1, max_size=3).map(tuple))
    curves, argmin = [], []
    for n in shape:
        best = draw(st.integers(0, n - 1))
        steps = draw(st.lists(st.integers(1, 9), min_size=n, max_size=n))
        g = [0.0] * n
        for i in range(best - 1, -1, -1):
            g[i] = g[i + 1] + steps[i]
        for i in range(best + 1, n):
            g[i] = g[i - 1] + steps[i]
        curves.append(g)
        argmin.append(best)
    order = draw(st.permutations(list(itertools.product(*[range(n) for n in shape]))))
    return shape, curves, tuple(argmin), order


@settings(max_examples=150, deadline=None)
@given(separable_unimodal())
def test_unimodal_pruner_never_cuts_the_minimum(case):
    shape, curves, argmin, order = case
    pruner = CoordinateUnimodalFunction(space_of(shape))
    timed = 0
    for idx in order:
        if pruner.is_pruned(idx):
            continue
        pruner.record(idx, sum(g[i] for g, i in zip(curves, idx)))
        timed += 1
        assert not pruner.is_pruned(argmin)
    assert timed >= 1
    # on one coordinate line through the minimum, whatever is still unpruned after all records includes the minimum
    for d in range(len(shape)):
        line = [argmin[:d] + (i,) + argmin[d + 1:] for i in range(shape[d])]
        assert argmin in [p for p in line if not pruner.is_pruned(p)]
