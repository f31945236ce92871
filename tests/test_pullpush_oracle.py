"""Pins of the pull-push oracle (CPU): library routines, closed forms and finite differences.

None of these checks retypes the oracle's formulas: torch's pooling and interpolation
routines, properties every correct pull-push has, and numerical differentiation.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import pullpush_oracle as pp


def rand_case(rng, B, C, H, W, dtype=np.float64):
    mask = rng.uniform(0.05, 1.0, (B, H, W)).astype(dtype)
    data = rng.uniform(-1.0, 1.0, (B, C, H, W)).astype(dtype)
    return mask, data


SIZES = [(4, 4), (8, 6), (5, 7), (9, 4), (3, 3), (13, 10)]


@pytest.mark.parametrize("H,W", SIZES)
def test_window_indices_are_adaptive_pooling_windows(H, W):
    """start/end index against what adaptive_max_pool2d reports as argmax positions."""
    oH, oW = H // 2, W // 2
    # an image whose value is its flat index: the maximum of each window sits at its last pixel
    img = torch.arange(H * W, dtype=torch.float64).reshape(1, 1, H, W)
    _, idx = F.adaptive_max_pool2d(img, (oH, oW), return_indices=True)
    for i in range(oH):
        for j in range(oW):
            last = (pp.end_index(i, oH, H) - 1) * W + (pp.end_index(j, oW, W) - 1)
            assert int(idx[0, 0, i, j]) == last
    neg = -img
    _, idx = F.adaptive_max_pool2d(neg, (oH, oW), return_indices=True)
    for i in range(oH):
        for j in range(oW):
            first = pp.start_index(i, oH, H) * W + pp.start_index(j, oW, W)
            assert int(idx[0, 0, i, j]) == first


@pytest.mark.parametrize("H,W", SIZES)
@pytest.mark.parametrize("impl", [pp.down, pp.down_loops])
def test_down_with_uniform_mask_is_adaptive_average_pooling(H, W, impl):
    rng = np.random.default_rng(H * 100 + W)
    _, data = rand_case(rng, 2, 3, H, W)
    mask = np.full((2, H, W), 0.37)
    mask_low, data_low = impl(mask, data)
    want = F.adaptive_avg_pool2d(torch.from_numpy(data), (H // 2, W // 2)).numpy()
    np.testing.assert_allclose(data_low, want, rtol=1e-13, atol=1e-14)
    np.testing.assert_array_equal(mask_low, np.full((2, H // 2, W // 2), 0.37))


@pytest.mark.parametrize("H,W", SIZES)
@pytest.mark.parametrize("impl", [pp.down, pp.down_loops])
def test_down_mask_is_adaptive_max_pooling_and_data_the_weighted_mean(H, W, impl):
    rng = np.random.default_rng(H * 100 + W + 1)
    mask, data = rand_case(rng, 2, 3, H, W)
    mask_low, data_low = impl(mask, data)
    tm, td = torch.from_numpy(mask)[:, None], torch.from_numpy(data)
    out = (H // 2, W // 2)
    np.testing.assert_array_equal(mask_low, F.adaptive_max_pool2d(tm, out)[:, 0].numpy())
    # weighted mean = mean(m*d) / mean(m): the window sizes cancel
    want = (F.adaptive_avg_pool2d(tm * td, out) / F.adaptive_avg_pool2d(tm, out)).numpy()
    np.testing.assert_allclose(data_low, want, rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("impl", [pp.down, pp.down_loops])
def test_down_empty_window_gives_zero(impl):
    mask = np.zeros((1, 4, 4))
    mask[0, 0, 0] = 1.0
    data = np.full((1, 2, 4, 4), 3.0)
    mask_low, data_low = impl(mask, data)
    np.testing.assert_array_equal(mask_low[0], [[1, 0], [0, 0]])
    np.testing.assert_array_equal(data_low[0, 0], [[3, 0], [0, 0]])


@pytest.mark.parametrize("H,W", [(4, 4), (8, 6), (2, 10), (16, 12)])
@pytest.mark.parametrize("impl", [pp.up, pp.up_loops])
def test_up_with_full_low_mask_is_bilinear_interpolation(H, W, impl):
    """Even sizes: mask 0 at high resolution and 1 at low resolution leaves the bilinear
    up-sampling with half-pixel centres and clamped borders (9/16, 3/16, 3/16, 1/16)."""
    rng = np.random.default_rng(H + W)
    data_low = rng.uniform(-1, 1, (2, 3, H // 2, W // 2))
    mask_low = np.ones((2, H // 2, W // 2))
    mask = np.zeros((2, H, W))
    data = rng.uniform(-1, 1, (2, 3, H, W))
    mask_high, data_high = impl(mask, data, mask_low, data_low)
    want = F.interpolate(torch.from_numpy(data_low), scale_factor=2, mode="bilinear", align_corners=False).numpy()
    np.testing.assert_allclose(data_high, want, rtol=1e-13, atol=1e-14)
    np.testing.assert_allclose(mask_high, 1.0, rtol=1e-14)


@pytest.mark.parametrize("impl", [pp.up, pp.up_loops])
def test_up_blends_by_the_high_res_mask_and_renormalises_by_the_low_res_masks(impl):
    rng = np.random.default_rng(5)
    H, W = 6, 8
    mask, data = rand_case(rng, 1, 2, H, W)
    mask_low = np.zeros((1, 3, 4))
    data_low = rng.uniform(-1, 1, (1, 2, 3, 4))
    # only one low-res pixel is known: every high-res pixel that touches it is filled with its value
    mask_low[0, 1, 2] = 0.5
    _, data_high = impl(mask, data, mask_low, data_low)
    for i in range(H):
        for j in range(W):
            touches = any((ii, jj) == (1, 2) for ii, jj, _ in pp._neighbours(i, j))
            fill = data_low[0, :, 1, 2] if touches else 0.0
            want = mask[0, i, j] * data[0, :, i, j] + (1 - mask[0, i, j]) * fill
            np.testing.assert_allclose(data_high[0, :, i, j], want, rtol=1e-13, atol=1e-15)


@pytest.mark.parametrize("H,W", SIZES + [(1, 5), (6, 1), (2, 2)])
def test_vectorised_forms_equal_the_loops(H, W):
    rng = np.random.default_rng(H * 31 + W)
    mask, data = rand_case(rng, 2, 3, H, W)
    mask[0, : H // 2] = 0.0           # empty regions take the n == 0 branches
    adj = rng.uniform(-1, 1, data.shape)
    np.testing.assert_allclose(pp.pullpush(mask, data), pp.pullpush(mask, data, loops=True), rtol=1e-12, atol=1e-13)
    gm, gd = pp.pullpush_adjoint(mask, data, adj)
    gm2, gd2 = pp.pullpush_adjoint(mask, data, adj, loops=True)
    np.testing.assert_allclose(gm, gm2, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(gd, gd2, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("H,W", SIZES + [(1, 5), (32, 32)])
def test_full_mask_is_identity(H, W):
    rng = np.random.default_rng(1)
    _, data = rand_case(rng, 2, 4, H, W)
    mask = np.ones((2, H, W))
    np.testing.assert_allclose(pp.pullpush(mask, data), data, rtol=0, atol=1e-15)
    adj = rng.uniform(-1, 1, data.shape)
    _, gd = pp.pullpush_adjoint(mask, data, adj)
    np.testing.assert_allclose(gd, adj, rtol=0, atol=1e-15)


@pytest.mark.parametrize("H,W", [(8, 8), (16, 16), (16, 4), (12, 20), (7, 9)])
def test_constant_data_stays_constant(H, W):
    """Every step is a weighted mean, so a constant image is reproduced wherever
    information arrives; with one known pixel and a 1-pixel coarsest level that is everywhere."""
    rng = np.random.default_rng(2)
    mask = rng.uniform(0.0, 1.0, (1, H, W)) * (rng.uniform(0, 1, (1, H, W)) > 0.7)
    mask[0, H // 3, W // 2] = 0.8
    data = np.full((1, 2, H, W), -2.5)
    out = pp.pullpush(mask, data)
    if (H & (H - 1)) == 0 and (W & (W - 1)) == 0:
        np.testing.assert_allclose(out, -2.5, rtol=1e-13)
    else:
        assert np.all((np.abs(out + 2.5) < 1e-12) | (out == 0.0))


def test_single_known_pixel_floods_the_image():
    H = W = 16
    mask = np.zeros((1, H, W))
    mask[0, 5, 11] = 1.0
    rng = np.random.default_rng(3)
    data = rng.uniform(-1, 1, (1, 3, H, W))
    out = pp.pullpush(mask, data)
    want = np.broadcast_to(data[:, :, 5:6, 11:12], out.shape)
    np.testing.assert_allclose(out, want, rtol=1e-13)


def test_empty_mask_gives_zero():
    rng = np.random.default_rng(4)
    data = rng.uniform(-1, 1, (1, 3, 8, 8))
    np.testing.assert_array_equal(pp.pullpush(np.zeros((1, 8, 8)), data), np.zeros_like(data))


def test_output_is_linear_in_the_data():
    rng = np.random.default_rng(6)
    mask, d1 = rand_case(rng, 1, 2, 9, 12)
    _, d2 = rand_case(rng, 1, 2, 9, 12)
    lhs = pp.pullpush(mask, 2.0 * d1 - 3.0 * d2)
    np.testing.assert_allclose(lhs, 2.0 * pp.pullpush(mask, d1) - 3.0 * pp.pullpush(mask, d2), rtol=1e-11, atol=1e-12)


def _numeric_gradient(f, x, eps):
    g = np.zeros_like(x)
    flat, gflat = x.reshape(-1), g.reshape(-1)
    for k in range(flat.size):
        old = flat[k]
        flat[k] = old + eps
        hi = f()
        flat[k] = old - eps
        lo = f()
        flat[k] = old
        gflat[k] = (hi - lo) / (2 * eps)
    return g


@pytest.mark.parametrize("H,W", [(4, 4), (6, 8), (5, 7), (9, 4), (8, 8)])
@pytest.mark.parametrize("loops", [False, True])
def test_gradients_against_finite_differences(H, W, loops):
    """Random fractional masks have no ties, so the maximum is differentiable at the sample."""
    if loops and H * W > 48:
        pytest.skip("the loop form is checked on the small sizes")
    for seed in range(H * 17 + W, H * 17 + W + 50):
        rng = np.random.default_rng(seed)
        mask, data = rand_case(rng, 1, 2, H, W)
        mask[0, 0, :2] = 0.0          # an empty corner: exercises weights that vanish
        # Overlapping windows (odd sizes) can carry one pixel into two low-res maxima; a later
        # window then sees a tie and the reference's rule "every pixel that attains the maximum
        # gets the gradient" counts it twice. Differentiate only where no level has such a tie.
        saved = []
        pp._forward(mask, data, pp._NUMPY, saved)
        if all(np.unique(level[0]).size == level[0].size for level in saved):
            break
    else:
        pytest.fail("no tie-free sample found")
    adj = rng.uniform(-1, 1, data.shape)
    gm, gd = pp.pullpush_adjoint(mask, data, adj, loops=loops)
    loss = lambda: float(np.sum(pp.pullpush(mask, data) * adj))
    nd = _numeric_gradient(loss, data, 1e-6)
    np.testing.assert_allclose(gd, nd, rtol=1e-6, atol=1e-8)
    nm = _numeric_gradient(loss, mask, 1e-6)
    known = mask > 0                  # one-sided at exactly 0: the forward clamps the maximum at 0
    np.testing.assert_allclose(gm[known], nm[known], rtol=1e-5, atol=1e-7)


def test_adjoint_is_the_transpose_in_the_data():
    """<pullpush(mask, x), y> == <x, adjoint_data(mask, y)> for the linear map in the data."""
    rng = np.random.default_rng(8)
    mask, x = rand_case(rng, 2, 3, 11, 6)
    y = rng.uniform(-1, 1, x.shape)
    _, gd = pp.pullpush_adjoint(mask, x, y)
    np.testing.assert_allclose(np.sum(pp.pullpush(mask, x) * y), np.sum(x * gd), rtol=1e-12)
