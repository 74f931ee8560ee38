"""Pins oracle/conv_oracle.c (the CPU restatement of tritonix/ops/conv2d/forward.py:19-165).

The reference has no test or stored vector for conv2d, so the restatement is checked against
``torch.nn.functional.conv2d`` in float64 (a library routine) on cases where a swapped height/width
argument, a wrong padding sign, a dropped dilation or a transposed weight index would fail, and against
closed forms that do not go through any convolution routine.
"""
import numpy as np
import pytest
import torch

import oracle

CASES = [
    # n, c_in, h, w, c_out, r, s, stride, padding, dilation, bias
    (2, 3, 9, 11, 5, 3, 3, (1, 1), (1, 1), (1, 1), True),
    (1, 4, 8, 8, 6, 1, 1, (1, 1), (0, 0), (1, 1), False),
    (2, 3, 13, 10, 4, 3, 2, (2, 1), (0, 2), (1, 2), True),      # everything asymmetric
    (1, 2, 12, 15, 3, 2, 4, (1, 3), (3, 1), (3, 1), True),
    (3, 5, 7, 7, 7, 5, 5, (1, 1), (2, 2), (1, 1), False),
    (1, 1, 5, 5, 1, 5, 5, (1, 1), (0, 0), (1, 1), True),        # one output pixel
    (2, 6, 10, 9, 33, 3, 3, (2, 2), (1, 1), (1, 1), True),      # c_out past one tile
    (1, 3, 6, 6, 2, 3, 3, (1, 1), (4, 4), (1, 1), False),       # padding wider than the filter
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("blocks", [(32, 32, 16), (16, 8, 4), (64, 64, 32)])
def test_tiled_conv2d_matches_torch_float64(case, blocks):
    n, c, h, w, k, r, s, stride, padding, dilation, has_bias = case
    g = torch.Generator().manual_seed(hash(case) % 1000)
    x = torch.randn(n, c, h, w, generator=g)
    wt = torch.randn(k, c, r, s, generator=g)
    b = torch.randn(k, generator=g) if has_bias else None
    want = torch.nn.functional.conv2d(x.double(), wt.double(), None if b is None else b.double(), stride, padding, dilation)
    got = oracle.tiled_conv2d(x.numpy(), wt.numpy(), None if b is None else b.numpy(), stride, padding, dilation, *blocks)
    assert got.shape == tuple(want.shape)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-4, atol=1e-4)


def test_output_size_formula():
    assert oracle.conv2d_output_size(224, 224, 7, 7, (2, 2), (3, 3), (1, 1)) == (112, 112)
    assert oracle.conv2d_output_size(56, 56, 3, 3, (1, 1), (1, 1), (1, 1)) == (56, 56)
    assert oracle.conv2d_output_size(10, 13, 3, 2, (2, 1), (0, 2), (1, 2)) == (4, 15)
    assert oracle.conv2d_output_size(7, 7, 3, 3, (1, 1), (0, 0), (2, 2)) == (3, 3)
    # filter larger than the padded image: not positive
    assert oracle.conv2d_output_size(2, 2, 5, 5, (1, 1), (0, 0), (1, 1))[0] <= 0


def test_one_by_one_filter_is_a_matrix_product():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((2, 6, 4, 5)).astype(np.float32)
    w = rng.standard_normal((3, 6, 1, 1)).astype(np.float32)
    got = oracle.tiled_conv2d(x, w)
    want = np.einsum("kc,nchw->nkhw", w[:, :, 0, 0].astype(np.float64), x.astype(np.float64))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("tap", [(0, 0), (0, 2), (2, 1), (1, 1)])
def test_one_hot_filter_is_a_shifted_copy(tap):
    """w[0, 0, th, tw] = 1: y[h, w] = x[h - pad + th*dil, w - pad + tw*dil], zero outside the image."""
    rng = np.random.default_rng(2)
    x = rng.standard_normal((1, 1, 6, 7)).astype(np.float32)
    w = np.zeros((1, 1, 3, 3), dtype=np.float32)
    w[0, 0, tap[0], tap[1]] = 1.0
    pad, dil = (2, 1), (2, 1)
    got = oracle.tiled_conv2d(x, w, None, (1, 1), pad, dil)
    ho, wo = got.shape[2:]
    want = np.zeros((ho, wo), dtype=np.float32)
    for i in range(ho):
        for j in range(wo):
            hi, wi = i - pad[0] + tap[0] * dil[0], j - pad[1] + tap[1] * dil[1]
            if 0 <= hi < 6 and 0 <= wi < 7:
                want[i, j] = x[0, 0, hi, wi]
    np.testing.assert_array_equal(got[0, 0], want)


def test_all_ones_filter_gives_box_sums_with_stride():
    rng = np.random.default_rng(3)
    x = rng.integers(-4, 5, size=(1, 2, 9, 8)).astype(np.float32)     # small integers: sums are exact
    w = np.ones((1, 2, 3, 2), dtype=np.float32)
    got = oracle.tiled_conv2d(x, w, np.array([0.5], dtype=np.float32), (2, 3), (0, 0), (1, 1))
    sat = np.zeros((10, 9))
    sat[1:, 1:] = x.sum(axis=1)[0].cumsum(0).cumsum(1)                # summed-area table over both channels
    ho, wo = got.shape[2:]
    assert (ho, wo) == (4, 3)
    for i in range(ho):
        for j in range(wo):
            h0, w0 = 2 * i, 3 * j
            box = sat[h0 + 3, w0 + 2] - sat[h0, w0 + 2] - sat[h0 + 3, w0] + sat[h0, w0]
            assert got[0, 0, i, j] == box + 0.5


def test_linearity_in_the_weight():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((1, 3, 7, 7)).astype(np.float32)
    w1 = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    w2 = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    a = oracle.tiled_conv2d(x, w1, None, (1, 1), (1, 1))
    b = oracle.tiled_conv2d(x, w2, None, (1, 1), (1, 1))
    c = oracle.tiled_conv2d(x, w1 + w2, None, (1, 1), (1, 1))
    np.testing.assert_allclose(a + b, c, rtol=1e-4, atol=1e-4)


def test_reference_conv2d_is_the_library_routine():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(1, 2, 5, 5, generator=g).bfloat16()
    w = torch.randn(3, 2, 3, 3, generator=g).bfloat16()
    got = oracle.reference_conv2d(x, w, None, (1, 1), (1, 1), (1, 1))
    assert got.dtype == torch.float32
    np.testing.assert_allclose(got.numpy(), oracle.tiled_conv2d(x.float().numpy(), w.float().numpy(), None, (1, 1), (1, 1)),
                               rtol=1e-5, atol=1e-5)
