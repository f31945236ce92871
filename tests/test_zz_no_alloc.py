"""The entry point of the C ABI that allocates nothing, qmlp_network_inference_noalloc, against
qmlp_network_inference on the same inputs: bit for bit (every point is evaluated on its own,
whatever the order of the batch), on two calls in a row, the second on a smaller batch, with a
network whose batches are ordered by grid slab in the library's static device buffer; then networks
that never use the buffer, and the hand-over of the buffer between streams."""
import gc
import json
import os

import numpy as np
import pytest
import torch

import qmlp
import baseline_configs as bc

pytestmark = pytest.mark.gpu


def sorted_grid_cfg():
    cfg = json.loads(json.dumps(bc.CONFIGS[5]["cfg"]))
    cfg["options"] = {"sort_points": 1}          # every batch is ordered, whatever its size
    return cfg


def test_inference_that_allocates_nothing_matches_inference():
    cfg = sorted_grid_cfg()
    net = qmlp.Network(json.dumps(cfg))
    if os.environ.get("QMLP_WARM_CACHE"):
        net.precompile(0)
        pytest.skip("kernel cache warmed")
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    rng = np.random.default_rng(11)
    params = torch.from_numpy(bc.make_parameters(5, rng)).cuda()
    table = torch.from_numpy(bc.make_table(5, net.encoding(0).num_parameters(), rng, 1.0)).half().cuda()
    enc = [table, None]
    sizes = (200_000, 70_001)
    xs = [torch.from_numpy(rng.uniform(0, 1, (n, 4)).astype(np.float32)).cuda() for n in sizes]
    # the ordinary entry point first: it compiles and loads the kernels these batch sizes use
    want = [net.inference(x, params, enc) for x in xs]
    torch.cuda.synchronize()
    assert float(want[0].abs().max()) > 0.01
    outs = [torch.full((n, 2), float("nan"), device="cuda") for n in sizes]
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]       # device-wide: also sees a hipMalloc of the library
    for x, out in zip(xs, outs):                 # two calls in a row, the second one smaller
        net.inference_noalloc(x, out, params, enc)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    for n, out, w in zip(sizes, outs, want):
        assert torch.equal(out, w), "batch of %d points" % n
    # and once more in the other order: the buffer keeps the previous call's contents
    for i in (1, 0):
        outs[i].fill_(float("nan"))
        net.inference_noalloc(xs[i], outs[i], params, enc)
        assert torch.equal(outs[i], want[i])

    # a batch whose order does not fit the static buffer is refused with a clear message
    big = torch.zeros((2_600_000, 4), device="cuda")
    with pytest.raises(qmlp.QmlpError, match="static buffer of 50331648 bytes"):
        net.inference_noalloc(big, torch.empty((big.shape[0], 2), device="cuda"), params, enc)
    # a network whose kernels are not loaded yet is refused as well: loading allocates
    fresh = qmlp.Network(json.dumps(cfg))
    with pytest.raises(qmlp.QmlpError, match="not loaded yet"):
        fresh.inference_noalloc(xs[1], outs[1], params, enc)


def test_networks_that_do_not_order_their_batch_allocate_nothing_either():
    """Networks whose batches stay as given never touch the static buffer; what matters for them is that
    every kernel a batch size takes is loaded: a hash-grid network on a batch that is cut into two launches of
    different kernel shapes, an identity-encoded network, and a batch size that needs a shape not yet seen."""
    if os.environ.get("QMLP_WARM_CACHE"):
        qmlp.Network(json.dumps(bc.CONFIGS[2]["cfg"])).precompile(0)
        qmlp.Network(json.dumps(bc.CONFIGS[1]["cfg"])).precompile(0)
        pytest.skip("kernel cache warmed")
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    rng = np.random.default_rng(5)
    grid = qmlp.Network(json.dumps(bc.CONFIGS[2]["cfg"]))
    params = torch.from_numpy(bc.make_parameters(2, rng)).cuda()
    table = torch.from_numpy(bc.make_table(2, grid.encoding(0).num_parameters(), rng, 1.0)).half().cuda()
    # 2^20 + 2^18 points: one launch of the shape with the encoded rows in registers, one of a smaller shape
    n = (1 << 20) + (1 << 18)
    x = torch.from_numpy(rng.uniform(0, 1, (n, 3)).astype(np.float32)).cuda()
    small = x[:3000].contiguous()
    with pytest.raises(qmlp.QmlpError, match="not loaded yet"):
        grid.inference_noalloc(x, torch.empty((n, 1), device="cuda"), params, [table])
    want = grid.inference(x, params, [table])
    out = torch.full((n, 1), float("nan"), device="cuda")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    grid.inference_noalloc(x, out, params, [table])
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.equal(out, want)
    # 3000 points take the shape of one tile per wavefront, which no call has loaded so far
    with pytest.raises(qmlp.QmlpError, match="not loaded yet"):
        grid.inference_noalloc(small, torch.empty((3000, 1), device="cuda"), params, [table])
    want_small = grid.inference(small, params, [table])
    out_small = torch.empty((3000, 1), device="cuda")
    grid.inference_noalloc(small, out_small, params, [table])
    assert torch.equal(out_small, want_small)

    mlp = qmlp.Network(json.dumps(bc.CONFIGS[1]["cfg"]))
    p1 = torch.from_numpy(bc.make_parameters(1, rng)).cuda()
    x1 = torch.from_numpy(rng.uniform(0, 1, (70_001, 3)).astype(np.float32)).cuda()
    want1 = mlp.inference(x1, p1, [])
    out1 = torch.full((70_001, 1), float("nan"), device="cuda")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    mlp.inference_noalloc(x1, out1, p1, [])
    mlp.inference_noalloc(x1[:1000], out1[:1000], p1, [])       # the same kernel serves every size
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.equal(out1, want1)


def test_static_buffer_is_handed_from_stream_to_stream_only_when_the_first_has_finished():
    """All calls on a device share the static buffer. A call on another stream than the last one is
    accepted once that stream's work is done, and refused while it is still running."""
    cfg = sorted_grid_cfg()
    net = qmlp.Network(json.dumps(cfg))
    if os.environ.get("QMLP_WARM_CACHE"):
        net.precompile(0)
        pytest.skip("kernel cache warmed")
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    rng = np.random.default_rng(13)
    params = torch.from_numpy(bc.make_parameters(5, rng)).cuda()
    table = torch.from_numpy(bc.make_table(5, net.encoding(0).num_parameters(), rng, 1.0)).half().cuda()
    enc = [table, None]
    x = torch.from_numpy(rng.uniform(0, 1, (300_000, 4)).astype(np.float32)).cuda()
    want = net.inference(x, params, enc)
    out = torch.empty_like(want)
    net.inference_noalloc(x, out, params, enc)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        out2 = torch.empty_like(want)
        net.inference_noalloc(x, out2, params, enc)          # the first stream is idle: accepted
    side.synchronize()
    assert torch.equal(out2, want)
    # work that keeps the side stream busy for a while, then a call on the first stream
    with torch.cuda.stream(side):
        big = torch.empty(1 << 28, device="cuda")
        for _ in range(20):
            big.normal_()
        net.inference_noalloc(x, out2, params, enc)
    with pytest.raises(qmlp.QmlpError, match="last used on another stream"):
        net.inference_noalloc(x, out, params, enc)
    torch.cuda.synchronize()
    net.inference_noalloc(x, out, params, enc)               # now it has finished
    torch.cuda.synchronize()
    assert torch.equal(out, want) and torch.equal(out2, want)


def test_prepare_leaves_nothing_to_load_or_allocate_for_a_train_step():
    """qmlp_network_prepare(numel, flags) loads every kernel a train step on such a batch takes, creates the
    streams of the weight-update kernels and allocates nothing later: forward and adjoint then neither compile,
    nor read the kernel cache, nor allocate device memory (what a caller under graph capture needs)."""
    cfg = json.loads(json.dumps(bc.CONFIGS[3]["cfg"]))
    cfg["options"] = {"parallel_weight_update": True, "fused_weight_update": 0}
    if os.environ.get("QMLP_WARM_CACHE"):
        qmlp.Network(json.dumps(cfg)).precompile(7)
        pytest.skip("kernel cache warmed")
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    n, flags = 1 << 16, 7
    rng = np.random.default_rng(21)
    params = torch.from_numpy(bc.make_parameters(3, rng)).cuda()
    x = torch.from_numpy(bc.make_inputs(3, n, rng)).cuda()
    adj = torch.from_numpy(rng.uniform(-1, 1, (n, 1)).astype(np.float32)).cuda()

    def train(net, table):
        out, tmp = net.forward_raw(x, params, [table], flags)
        adj_x, g_net, g_enc = net.adjoint_raw(x, adj, flags, tmp, params, [table])
        torch.cuda.synchronize()
        return out, adj_x, g_net, g_enc[0]

    plain = qmlp.Network(json.dumps(cfg))
    table = torch.from_numpy(bc.make_table(3, plain.encoding(0).num_parameters(), rng, 1.0)).half().cuda()
    spare = train(plain, table)
    want = train(plain, table)
    del plain, spare                     # torch's allocator keeps the blocks of one more step for the results below
    net = qmlp.Network(json.dumps(cfg))
    net.prepare(n, flags)
    gc.collect()                         # networks of earlier tests that wait for the collector would unload their kernels below
    torch.cuda.synchronize()
    stats = qmlp._lib.kernel_cache_stats()
    free_before = torch.cuda.mem_get_info()[0]
    got = train(net, table)
    assert qmlp._lib.kernel_cache_stats() == stats, "a kernel was compiled or read from the cache after prepare()"
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]) and torch.equal(got[2], want[2])
    scale = float(want[3].abs().max())
    assert torch.allclose(got[3] / scale, want[3] / scale, rtol=1e-4, atol=2e-6)
