"""Pins the CPU oracle before anything is compared against it: the example the reference holds, hand traces,
brute force on tiny inputs, closed forms and special cases chosen so a dropped term, a wrong index or a
transposed operand fails."""
import numpy as np
import pytest
import torch

import oracle
from tritonix_amd.ops.matmul import grouped_launch as host_grouped_launch
from tritonix_amd.ops.matmul import swizzle2d as host_swizzle2d


# ---- swizzle / tile order ------------------------------------------------------------
def test_swizzle_docstring_example(traces):
    out = [[None] * 4 for _ in range(4)]
    for i in range(4):
        for j in range(4):
            ni, nj = oracle.swizzle2d(i, j, 4, 4, 2)
            out[ni][nj] = i * 4 + j
    assert out == traces["swizzle_4x4_g2"]


def test_swizzle_ragged_last_group(traces):
    for i, j, ni, nj in traces["swizzle_3x2_g2"]:
        assert oracle.swizzle2d(i, j, 3, 2, 2) == (ni, nj)


def test_swizzle_is_a_bijection_and_matches_grouped_launch_and_the_host_copy():
    for si in range(1, 13):
        for sj in range(1, 13):
            for g in range(1, 10):
                seen = set()
                for i in range(si):
                    for j in range(sj):
                        o = oracle.swizzle2d(i, j, si, sj, g)
                        assert 0 <= o[0] < si and 0 <= o[1] < sj
                        seen.add(o)
                        assert host_swizzle2d(i, j, si, sj, g) == o
                        assert host_grouped_launch(i * sj + j, si * 32, sj * 32, 32, 32, g) == o
                        # the reference's own (unused) grouped_launch is the same map wherever the
                        # group is full; see test_reference_grouped_launch_differs_in_a_ragged_group
                        if si % g == 0:
                            assert oracle.grouped_launch(i * sj + j, si * 32, sj * 32, 32, 32, g) == o
                assert len(seen) == si * sj


def test_reference_grouped_launch_differs_in_a_ragged_group():
    # tritonix/ops/matmul.py:127 takes `pid % group_size` where tl.swizzle2d takes
    # `(pid % width) % group_size`: in a ragged last group the two disagree and the former is
    # no longer a bijection.  The HIP kernels and the host helper follow tl.swizzle2d (the
    # function the reference kernels actually call).
    si, sj, g = 5, 3, 2   # last group has one row
    ref_ids = {oracle.grouped_launch(p, si * 32, sj * 32, 32, 32, g) for p in range(si * sj)}
    swz_ids = {oracle.swizzle2d(p // sj, p % sj, si, sj, g) for p in range(si * sj)}
    assert len(swz_ids) == si * sj
    assert ref_ids == swz_ids          # one row in the last group: pid % 1 == 0 either way
    si, sj, g = 7, 3, 4   # last group has three rows, width 12, 12 % 3 == 0 -> still equal
    assert all(oracle.grouped_launch(p, si * 32, sj * 32, 32, 32, g) == oracle.swizzle2d(p // sj, p % sj, si, sj, g)
               for p in range(si * sj))
    si, sj, g = 7, 2, 4   # width 8, last group of three rows: 8 % 3 != 0 -> they part ways
    diff = [p for p in range(si * sj)
            if oracle.grouped_launch(p, si * 32, sj * 32, 32, 32, g) != oracle.swizzle2d(p // sj, p % sj, si, sj, g)]
    assert diff and min(diff) >= 8


def test_swizzle_walks_groups_column_major():
    # inside a group of g rows consecutive ids go down a column first
    order = sorted(((oracle.swizzle2d(i, j, 8, 5, 4), i * 5 + j) for i in range(8) for j in range(5)),
                   key=lambda t: t[1])
    assert [o for o, _ in order[:6]] == [(0, 0), (1, 0), (2, 0), (3, 0), (0, 1), (1, 1)]
    assert order[20][0] == (4, 0)


def test_xcd_remap_is_a_bijection_and_keeps_neighbours_on_one_xcd():
    for total in list(range(1, 70)) + [1024, 1792, 1000]:
        ids = [oracle.xcd_remap(p, total) for p in range(total)]
        assert sorted(ids) == list(range(total))
    # blocks pid, pid+8, pid+16 run on one XCD: their logical ids must be consecutive
    assert [oracle.xcd_remap(p, 1024) for p in (3, 11, 19)] == [384, 385, 386]


# ---- GEMM walk -----------------------------------------------------------------------
@pytest.mark.parametrize("m,n,k,bm,bn,bk,g", [(64, 64, 64, 32, 32, 16, 4), (70, 45, 53, 32, 32, 16, 2),
                                              (33, 17, 100, 16, 16, 32, 8), (5, 7, 3, 32, 32, 16, 4)])
def test_tiled_matmul_against_float64(m, n, k, bm, bn, bk, g):
    rng = np.random.default_rng(0)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    got = oracle.tiled_matmul(a, b, bm, bn, bk, g)
    want = a.astype(np.float64) @ b.astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-4)
    # not symmetric: a transposed-operand mistake cannot pass
    assert not np.allclose(got, (b.T.astype(np.float64) @ a.T.astype(np.float64)).T[::-1], atol=1e-2)


def test_tiled_matmul_closed_forms():
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    np.testing.assert_array_equal(oracle.tiled_matmul(a, np.eye(4, dtype=np.float32), 16, 16, 16, 4), a)
    ones = oracle.tiled_matmul(np.ones((40, 37), np.float32), np.ones((37, 50), np.float32), 32, 32, 16, 4)
    np.testing.assert_array_equal(ones, np.full((40, 50), 37.0, np.float32))
    # strided (transposed view) operands go through the stride arguments
    rng = np.random.default_rng(1)
    at = rng.standard_normal((20, 30)).astype(np.float32)
    b = rng.standard_normal((20, 10)).astype(np.float32)
    np.testing.assert_allclose(oracle.tiled_matmul(at.T, b, 16, 16, 16, 4), at.T @ b, rtol=1e-5, atol=1e-5)


def test_tiled_int8_is_exact():
    rng = np.random.default_rng(2)
    a = rng.integers(-127, 128, (50, 131), dtype=np.int8)
    b = rng.integers(-127, 128, (131, 41), dtype=np.int8)
    np.testing.assert_array_equal(oracle.tiled_matmul_i8(a, b, 32, 32, 32), a.astype(np.int64) @ b.astype(np.int64))
    full = np.full((4, 300), -127, np.int8)
    assert oracle.tiled_matmul_i8(full, full.T.copy(), 32, 32, 64)[0, 0] == 300 * 127 * 127
    ta, tb = torch.from_numpy(a), torch.from_numpy(b)
    assert torch.equal(oracle.reference_matmul(ta, tb), torch.from_numpy(oracle.tiled_matmul_i8(a, b)))


# ---- split-K partition ---------------------------------------------------------------
def test_splitk_cover_hand_trace(traces):
    cover = oracle.splitk_cover(100, 16, 3)
    assert cover.tolist() == [1] * 100
    want = traces["splitk_k100_bk16_s3"]
    # rebuild the ranges each pid_k loads and compare with the hand-derived ones
    for pid_k, ranges in want.items():
        got = []
        for k_loop in range(-(-100 // 48)):
            lo = k_loop * 48 + int(pid_k) * 16
            hi = min(lo + 16, 100)
            if lo < hi:
                got.append([lo, hi])
        assert got == ranges


@pytest.mark.parametrize("k,bk,s", [(1, 16, 2), (15, 16, 3), (16, 16, 4), (100, 16, 3), (257, 32, 7), (14336, 64, 16)])
def test_splitk_covers_every_k_exactly_once(k, bk, s):
    assert oracle.splitk_cover(k, bk, s).tolist() == [1] * k


def test_tiled_splitk_equals_plain_gemm():
    rng = np.random.default_rng(3)
    a = rng.standard_normal((20, 157)).astype(np.float32)
    b = rng.standard_normal((157, 33)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    for s in (2, 3, 8):
        np.testing.assert_allclose(oracle.tiled_splitk(a, b, s, 16, 16, 16, 4), want, rtol=1e-5, atol=1e-4)


# ---- GLU epilogue --------------------------------------------------------------------
def test_glu_closed_forms_and_interleave_convention():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((9, 21)).astype(np.float32)
    w1 = rng.standard_normal((21, 6)).astype(np.float32)
    w2 = rng.standard_normal((21, 6)).astype(np.float32)
    w12 = np.stack([w1, w2], axis=2).reshape(21, 12)        # gate in the even columns
    np.testing.assert_array_equal(w12[:, 0::2], w1)
    g, lin = (x.astype(np.float64) @ w1), (x.astype(np.float64) @ w2)
    sig = 1.0 / (1.0 + np.exp(-g))
    np.testing.assert_allclose(oracle.tiled_glu(x, w12, "silu", 16, 16, 16, 4), g * sig * lin, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(oracle.tiled_glu(x, w12, "sigmoid", 16, 16, 16, 4), sig * lin, rtol=1e-4, atol=1e-4)
    # any other activation: un-activated gate = elementwise product of two plain GEMMs
    np.testing.assert_allclose(oracle.tiled_glu(x, w12, "relu", 16, 16, 16, 4),
                               oracle.tiled_matmul(x, w1, 16, 16, 16, 4) * oracle.tiled_matmul(x, w2, 16, 16, 16, 4),
                               rtol=1e-5, atol=1e-5)
    # swapping the roles of gate and linear must change the silu result
    w21 = np.stack([w2, w1], axis=2).reshape(21, 12)
    assert not np.allclose(oracle.tiled_glu(x, w21, "silu"), oracle.tiled_glu(x, w12, "silu"), atol=1e-3)
    # the torch restatement agrees
    ref = oracle.reference_glu(torch.from_numpy(x), torch.from_numpy(w12), "silu").numpy()
    np.testing.assert_allclose(ref, g * sig * lin, rtol=1e-4, atol=1e-4)
    assert oracle.tiled_glu(np.zeros((3, 4), np.float32), np.ones((4, 6), np.float32), "sigmoid").tolist() == [[0.0] * 3] * 3


# ---- seeded inputs -------------------------------------------------------------------
def test_reference_matmul_float_branch_against_float64():
    """The fp32 CPU matmul the parity bar is anchored on, against a float64 numpy product of the same 16-bit
    inputs: fp32 accumulation over K=4096 terms of size ~1 stays within a few 1e-6 of the exact product relative
    to sqrt(K), far inside the 1e-2 bar; a transposed operand, a dropped K tail or a wrong upcast would not."""
    g = torch.Generator("cpu").manual_seed(21)
    for dt in (torch.float16, torch.bfloat16):
        a = torch.randn(96, 4096, generator=g).to(dt)
        b = torch.randn(4096, 80, generator=g).to(dt)
        want = a.double().numpy() @ b.double().numpy()
        got = oracle.reference_matmul(a, b)
        assert got.dtype == torch.float32 and got.shape == (96, 80)
        assert np.abs(got.double().numpy() - want).max() <= 2e-5 * np.sqrt(4096.0)
        # non-contiguous views must be honoured as views, not reinterpreted
        at = a.t().contiguous().t()
        assert torch.equal(oracle.reference_matmul(at, b), got)
    # within_tolerance itself: exact passes, an error of 3 % of the rms on one element fails
    ref = torch.randn(8, 8, generator=g)
    assert oracle.within_tolerance(ref.clone(), ref)[0]
    bad = ref.clone()
    bad[3, 4] += 0.03 * float(ref.pow(2).mean().sqrt()) + 0.02 * float(ref[3, 4].abs())
    assert not oracle.within_tolerance(bad, ref)[0]


def test_seeded_inputs_are_reproducible_and_shaped():
    a1, b1 = oracle.make_inputs("C1")
    a2, b2 = oracle.make_inputs("C1")
    assert torch.equal(a1, a2) and torch.equal(b1, b2)
    assert a1.shape == (1024, 512) and b1.shape == (512, 768) and a1.dtype == torch.float16
    a, b = oracle.make_inputs("C3", scale_down=8)
    assert a.shape == (16, 1792) and b.shape == (1792, 512) and a.dtype == torch.bfloat16
    x, w12 = oracle.make_inputs("C4", scale_down=16)
    assert x.shape == (256, 256) and w12.shape == (256, 1792)
    a, b = oracle.make_inputs("C5", scale_down=32)
    assert a.dtype == torch.int8 and int(a.min()) >= -127
    ok, maxerr, rel = oracle.within_tolerance(torch.ones(4), torch.ones(4) * 1.001)
    assert ok and maxerr < 2e-3
    assert not oracle.within_tolerance(torch.ones(4), torch.ones(4) * 1.5)[0]
