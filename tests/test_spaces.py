"""Config-space domains: values pinned by the hand-derived table in tests/golden/hand_traces.json."""
import pytest

from tritonix_amd.utils.spaces import Choice, ConfigSpace, PowerOfTwo, Range, SpaceConfig


def test_domain_values(traces):
    env = {"PowerOfTwo": PowerOfTwo, "Range": Range, "Choice": Choice}
    for expr, want in traces["spaces"].items():
        dom = eval(expr, env)
        assert dom.values() == want, expr
        assert len(dom) == len(want)
        assert [dom[i] for i in range(len(want))] == want


def test_range_upper_bound_is_inclusive():
    assert Range(2, 5).values()[-1] == 5
    assert len(Range(2, 8)) == 7


def test_power_of_two_start_need_not_be_a_power():
    assert PowerOfTwo(24, 100).values() == [24, 48, 96]
    assert PowerOfTwo(3, 2).values() == []


def test_choice_copies_its_options():
    src = [4, 8]
    c = Choice(src)
    src.append(16)
    assert c.values() == [4, 8]
    assert Choice(range(3)).values() == [0, 1, 2]


def test_space_config_shape_len_lookup():
    sc = SpaceConfig({"a": Choice([1, 2, 3]), "b": Range(0, 1)})
    assert sc.shape == (3, 2)
    assert len(sc) == 6
    assert sc[(2, 1)] == [3, 1]
    assert ConfigSpace is SpaceConfig


def test_empty_param_is_rejected():
    with pytest.raises(ValueError):
        SpaceConfig({"a": Choice([1]), "b": Choice([])})
    with pytest.raises(ValueError):
        SpaceConfig({"a": Range(5, 2)})


def test_kernel_space_sizes():
    # the package's own spaces; the reference's declarations give 432 / 3024 / 1024 with an inclusive Range
    import math

    from tritonix_amd.ops.matmul import gemm_splitk_kernel, matmul_kernel
    from tritonix_amd.ops.swiglu import glu_kernel

    for kern in (matmul_kernel, gemm_splitk_kernel, glu_kernel):
        assert len(kern.configs()) == math.prod(len(p) for p in kern.space.values())
    ref = {"block_m": PowerOfTwo(32, 128), "block_n": PowerOfTwo(32, 128), "block_k": PowerOfTwo(16, 64),
           "group_m": Choice([4, 8]), "num_stages": Range(2, 5), "num_warps": Choice([4, 8])}
    assert len(SpaceConfig(ref)) == 432
    assert len(SpaceConfig({**ref, "split_k": Range(2, 8)})) == 3024
