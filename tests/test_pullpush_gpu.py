"""Pull-push inpainting on the GPU (through the C ABI) against the CPU oracle.

Tolerances: the double kernels against the float64 oracle rel 1e-10 (different summation
order, atomics); the float kernels rel 2e-3 / abs 2e-4 for gradients and rel 1e-4 / abs 1e-5
for the forward pass (fp32 sums over all pyramid levels against float64).
"""
import os

import numpy as np
import pytest
import torch

import pullpush_oracle as ppo
from qmlp import pullpush as qpp
from qmlp.pullpush import pullpush

pytestmark = pytest.mark.gpu

FWD_TOL = {torch.float64: dict(rtol=1e-10, atol=1e-12), torch.float32: dict(rtol=1e-4, atol=1e-5)}
ADJ_TOL = {torch.float64: dict(rtol=1e-9, atol=1e-11), torch.float32: dict(rtol=2e-3, atol=2e-4)}


@pytest.fixture(autouse=True, scope="module")
def _gpu_or_warm():
    if os.environ.get("QMLP_WARM_CACHE"):
        qpp.precompile(torch.float32)
        qpp.precompile(torch.float64)
        pytest.skip("kernel cache warmed")
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")


def make_case(seed, B, C, H, W, dtype, sparse=None):
    """Inputs that both sides see with identical values (drawn in the GPU's dtype)."""
    rng = np.random.default_rng(seed)
    np_dtype = np.float32 if dtype == torch.float32 else np.float64
    if sparse is None:
        mask = rng.uniform(0.05, 1.0, (B, H, W)).astype(np_dtype)
        if H > 2:
            mask[:, : H // 3, : W // 2] = 0     # an unknown region
    else:
        mask = (rng.uniform(0, 1, (B, H, W)) > 1 - sparse).astype(np_dtype)
    data = rng.uniform(-1, 1, (B, C, H, W)).astype(np_dtype)
    adj = rng.uniform(-1, 1, (B, C, H, W)).astype(np_dtype)
    return mask, data, adj


def gpu(x, dtype):
    return torch.from_numpy(x).to(device="cuda", dtype=dtype)


SHAPES = [(1, 1, 2, 2), (2, 3, 4, 4), (2, 3, 8, 6), (1, 4, 5, 7), (2, 2, 9, 4), (1, 15, 13, 10), (3, 1, 1, 5),
          (1, 2, 6, 1), (2, 3, 37, 53), (1, 3, 64, 64)]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("shape", SHAPES)
def test_forward_against_oracle(shape, dtype):
    mask, data, _ = make_case(sum(shape), *shape, dtype)
    print("pullpush forward", shape, dtype, flush=True)
    out = pullpush(gpu(mask, dtype), gpu(data, dtype))
    want = ppo.pullpush(mask.astype(np.float64), data.astype(np.float64))
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want, **FWD_TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("shape", SHAPES)
def test_adjoint_against_oracle(shape, dtype):
    mask, data, adj = make_case(sum(shape) + 1, *shape, dtype)
    print("pullpush adjoint", shape, dtype, flush=True)
    gm, gd = qpp.pullpush_backward(gpu(mask, dtype), gpu(data, dtype), gpu(adj, dtype))
    wm, wd = ppo.pullpush_adjoint(mask.astype(np.float64), data.astype(np.float64), adj.astype(np.float64))
    np.testing.assert_allclose(gd.cpu().numpy().astype(np.float64), wd, **ADJ_TOL[dtype])
    np.testing.assert_allclose(gm.cpu().numpy().astype(np.float64), wm, **ADJ_TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_sparse_binary_mask_like_the_reference_test(dtype):
    """5% known pixels with mask exactly 1 (tests_py/qmlp_tests/test_pushpull.py:39-44):
    many equal maxima, where every pixel that attains the maximum receives the gradient."""
    shape = (1, 3, 200, 264)
    mask, data, adj = make_case(11, *shape, dtype, sparse=0.05)
    print("pullpush sparse", shape, dtype, flush=True)
    tm, td = gpu(mask, dtype), gpu(data, dtype)
    out = pullpush(tm, td)
    m64, d64, a64 = (x.astype(np.float64) for x in (mask, data, adj))
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), ppo.pullpush(m64, d64), **FWD_TOL[dtype])
    # known pixels keep their values
    known = np.broadcast_to(mask[:, None] == 1, data.shape)
    np.testing.assert_array_equal(out.cpu().numpy()[known], data[known])
    gm, gd = qpp.pullpush_backward(tm, td, gpu(adj, dtype))
    wm, wd = ppo.pullpush_adjoint(m64, d64, a64)
    np.testing.assert_allclose(gd.cpu().numpy().astype(np.float64), wd, **ADJ_TOL[dtype])
    np.testing.assert_allclose(gm.cpu().numpy().astype(np.float64), wm, **ADJ_TOL[dtype])


def test_strided_tensors():
    """The kernels address through the strides: channels-last data and a transposed mask."""
    B, C, H, W = 2, 3, 10, 12
    mask, data, adj = make_case(21, B, C, H, W, torch.float64)
    tm = gpu(np.ascontiguousarray(mask.transpose(0, 2, 1)), torch.float64).transpose(1, 2)
    td = gpu(np.ascontiguousarray(data.transpose(0, 2, 3, 1)), torch.float64).permute(0, 3, 1, 2)
    assert not tm.is_contiguous() and not td.is_contiguous()
    print("pullpush strided", flush=True)
    out = pullpush(tm, td)
    assert out.stride() == td.stride()
    np.testing.assert_allclose(out.cpu().numpy(), ppo.pullpush(mask, data), **FWD_TOL[torch.float64])
    gm, gd = qpp.pullpush_backward(tm, td, gpu(adj, torch.float64))
    wm, wd = ppo.pullpush_adjoint(mask, data, adj)
    np.testing.assert_allclose(gd.cpu().numpy(), wd, **ADJ_TOL[torch.float64])
    np.testing.assert_allclose(gm.cpu().numpy(), wm, **ADJ_TOL[torch.float64])
    # a single row is copied through, also with strides
    print("pullpush strided row", flush=True)
    row_m, row_d = tm[:, 3:4, :], td[:, :, 3:4, :]
    assert torch.equal(pullpush(row_m, row_d), row_d)


def test_autograd_gradcheck_in_double():
    """The GPU adjoint against finite differences of the GPU forward pass (fractional random
    masks on even sizes: no ties in the maxima)."""
    rng = np.random.default_rng(5)
    mask = torch.from_numpy(rng.uniform(0.1, 1.0, (1, 8, 4))).cuda().requires_grad_(True)
    data = torch.from_numpy(rng.uniform(-1, 1, (1, 2, 8, 4))).cuda().requires_grad_(True)
    print("pullpush gradcheck", flush=True)
    assert torch.autograd.gradcheck(pullpush, (mask, data), eps=1e-6, atol=1e-6, rtol=1e-5, nondet_tol=1e-12)


def test_full_size_properties():
    """At a size the oracle does not reach in seconds: full mask = identity, a single known
    pixel floods a power-of-two image, linearity in the data."""
    B, C, H, W = 1, 4, 2048, 2048     # square power of two: the coarsest level is one pixel
    g = torch.Generator(device="cuda").manual_seed(3)
    data = torch.rand((B, C, H, W), device="cuda", generator=g) * 2 - 1
    print("pullpush large: identity", flush=True)
    ones = torch.ones((B, H, W), device="cuda")
    assert torch.equal(pullpush(ones, data), data)
    print("pullpush large: flood", flush=True)
    single = torch.zeros((B, H, W), device="cuda")
    single[:, 700, 300] = 1.0
    out = pullpush(single, data)
    want = data[:, :, 700:701, 300:301].expand_as(out)
    torch.testing.assert_close(out, want, rtol=1e-5, atol=1e-6)
    print("pullpush large: linearity", flush=True)
    mask = (torch.rand((B, H, W), device="cuda", generator=g) > 0.95).float()
    data2 = torch.rand((B, C, H, W), device="cuda", generator=g)
    lhs = pullpush(mask, 2 * data - 3 * data2)
    rhs = 2 * pullpush(mask, data) - 3 * pullpush(mask, data2)
    torch.testing.assert_close(lhs, rhs, rtol=1e-4, atol=1e-5)
    print("pullpush large: transpose", flush=True)
    y = torch.rand((B, C, H, W), device="cuda", generator=g, dtype=torch.float32)
    _, gd = qpp.pullpush_backward(mask, data, y)
    a = (pullpush(mask, data).double() * y.double()).sum()
    b = (data.double() * gd.double()).sum()
    assert abs(a.item() - b.item()) <= 1e-4 * abs(a.item())


def test_optimisation_through_the_inpainting_reduces_the_loss():
    """The use in tests_py/qmlp_tests/test_pushpull.py:56-70: optimise the data under a sparse mask."""
    g = torch.Generator(device="cuda").manual_seed(9)
    # a smooth image: 5% of its pixels are enough to inpaint the rest
    yy, xx = torch.meshgrid(torch.linspace(0, 1, 96, device="cuda"), torch.linspace(0, 1, 128, device="cuda"), indexing="ij")
    truth = torch.stack([0.5 + 0.5 * torch.sin(3 * xx + 2 * yy), yy * xx, 0.5 + 0.5 * torch.cos(4 * yy)])[None]
    mask = (torch.rand((1, 96, 128), device="cuda", generator=g) > 0.95).float()
    x = torch.rand_like(truth).requires_grad_(True)
    adam = torch.optim.Adam([x], lr=0.2)
    losses = []
    print("pullpush optimisation", flush=True)
    for _ in range(10):
        adam.zero_grad()
        loss = torch.nn.functional.mse_loss(pullpush(mask, x), truth)
        loss.backward()
        adam.step()
        losses.append(loss.item())
    assert losses[-1] < 0.5 * losses[0]


def test_errors():
    mask = torch.zeros((1, 4, 4), device="cuda")
    with pytest.raises(RuntimeError, match="16 channels"):
        pullpush(mask, torch.zeros((1, 16, 4, 4), device="cuda"))
    with pytest.raises(RuntimeError, match="entries at dimension"):
        pullpush(mask, torch.zeros((1, 2, 4, 5), device="cuda"))
    with pytest.raises(RuntimeError, match="type"):
        pullpush(mask, torch.zeros((1, 2, 4, 4), device="cuda", dtype=torch.float64))
    with pytest.raises(RuntimeError, match="float or double"):
        pullpush(mask.half(), torch.zeros((1, 2, 4, 4), device="cuda", dtype=torch.float16))
    with pytest.raises(RuntimeError, match="dimensions"):
        pullpush(mask[0], torch.zeros((1, 2, 4, 4), device="cuda"))
    with pytest.raises(ValueError, match="GPU"):
        pullpush(mask.cpu(), torch.zeros((1, 2, 4, 4)))
    # empty batch: nothing to do
    out = pullpush(torch.zeros((0, 4, 4), device="cuda"), torch.zeros((0, 2, 4, 4), device="cuda"))
    assert out.shape == (0, 2, 4, 4)
