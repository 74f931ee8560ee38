"""CoordinateUnimodalFunction: hand-derived record / is_pruned sequences (tritonix/utils/pruners.py:191-225)."""
from tritonix_amd.utils.pruners import CoordinateMonotonicFunction, CoordinateUnimodalFunction
from tritonix_amd.utils.spaces import Choice, SpaceConfig


def space(*dims):
    return SpaceConfig({str(i): Choice(range(d)) for i, d in enumerate(dims)})


def test_both_names_are_one_class():
    assert CoordinateMonotonicFunction is CoordinateUnimodalFunction


def test_one_dimensional_trace(traces):
    f = CoordinateUnimodalFunction(space(5))
    for step in traces["unimodal_1d"]:
        f.record(tuple(step["record"]), step["value"])
        for idx, want in step["pruned"].items():
            assert f.is_pruned((int(idx),)) is want, (step, idx)


def test_equal_values_never_prune():
    f = CoordinateUnimodalFunction(space(4))
    f.record((1,), 3.0)
    f.record((2,), 3.0)
    f.record((0,), 3.0)
    assert not any(f.is_pruned((i,)) for i in range(4))


def test_slices_are_independent():
    f = CoordinateUnimodalFunction(space(3, 2))
    f.record((0, 0), 1.0)
    f.record((1, 0), 2.0)
    assert f.is_pruned((2, 0)) is True    # slice (·, 0): window (0, 0)
    assert f.is_pruned((2, 1)) is False   # another slice
    assert f.is_pruned((0, 0)) is False


def test_window_is_recomputed_when_a_new_best_appears():
    f = CoordinateUnimodalFunction(space(6))
    f.record((2,), 5.0)
    f.record((4,), 9.0)      # window (0, 3)
    assert f.is_pruned((5,)) and not f.is_pruned((3,))
    f.record((3,), 1.0)      # best moves right: left neighbour 2 is worse -> lo = 3; 4 worse -> hi = 3
    assert f.is_pruned((2,)) and f.is_pruned((4,)) and not f.is_pruned((3,))
