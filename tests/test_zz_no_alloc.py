"""The entry point of the C ABI that allocates nothing, qmlp_network_inference_noalloc, against
qmlp_network_inference on the same inputs: bit for bit (every point is evaluated on its own,
whatever the order of the batch), on two calls in a row, the second on a smaller batch, with a
network whose batches are ordered by grid slab in the library's static device buffer."""
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
