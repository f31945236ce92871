"""The PyTorch front end (FusedNetwork, FusedEncoding, FusedActivation) on the GPU, in the
shape of the reference's Python suite (tests_py/qmlp_tests/test_network_base.py:87-256,
test_activations.py:8-66, test_encoding.py:10-188, test_network_image.py:13-78).

The comparison partner is plain torch on the same device: ``SimulatedNetwork``
(torch.nn.Linear + activation modules in half precision) and torch's activation functions.
Tolerances are the reference suite's: outputs and input gradients rtol 1e-2 / atol 1e-3,
weight gradients rtol 1e-1 / atol 1e-3, at most 5% of the entries outside (the torch network
rounds every layer to half, the fused kernels accumulate in fp32).
"""
import copy
import io
import json
import os
import pickle

import numpy as np
import pytest
import torch

import qmlp
from qmlp import FusedActivation, FusedEncoding, FusedNetwork, SimulatedNetwork, copy_torch_to_fused

pytestmark = pytest.mark.gpu

WARM = bool(os.environ.get("QMLP_WARM_CACHE"))


def warm_or_gpu(network_cfg=None, activation=None, encoding_cfg=None):
    """In a CPU cache-warming pass compile what the test needs into the kernel cache and stop."""
    if WARM:
        if network_cfg is not None:
            qmlp.Network(network_cfg).precompile(7)
        if activation is not None:
            qmlp.Activation(activation).precompile()
        if encoding_cfg is not None:
            enc = qmlp.Encoding(encoding_cfg)
            for mode in (0, 1, 2, 3):
                enc.precompile(mode)
        pytest.skip("kernel cache warmed")
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")


def network_cfg(c_in, widths, activations, bias=False):
    return json.dumps({
        "num_inputs": c_in, "num_outputs": widths[-1],
        "activation_specification": ["qmlp/builtin-activations.json"],
        "encodings": [{"id": "Identity", "start_in": 0, "n_in": c_in}],
        "network": [{"n_out": w, "bias": bias, "activation": a} for w, a in zip(widths, activations)]})


def compare_tensors(actual, expected, name, rtol, atol, fail_threshold=0.05):
    """_compare_tensors of the reference suite (test_network_base.py:56-70)."""
    actual = actual.detach().cpu().to(torch.float32).numpy()
    expected = expected.detach().cpu().to(torch.float32).numpy()
    assert actual.shape == expected.shape, name
    different = ~np.isclose(actual, expected, rtol=rtol, atol=atol)
    assert different.mean() <= fail_threshold, "%s: %.2f%% of the entries differ" % (name, 100 * different.mean())


def compare_networks(fused, plain, rtol, atol):
    for layer in range(plain.num_layers()):
        for bias in ((False, True) if plain.has_bias(layer) else (False,)):
            want = plain.get_weight(layer, bias, True)
            got = fused.get_weight(layer, bias, True)
            got = got[tuple(slice(0, s) for s in want.shape)]      # the fused network pads widths to 16
            compare_tensors(got, want, "layer %d %s gradient" % (layer, "bias" if bias else "weight"), rtol, atol)


def run_network_suite(cfg, batch_sizes=(16, 32, 128, 513, 48621)):
    """_test_network of the reference suite (test_network_base.py:87-147)."""
    fused = FusedNetwork(cfg)
    plain = SimulatedNetwork(cfg).to("cuda")
    copy_torch_to_fused(fused, plain)
    n_in, n_out = fused.channels_in(), fused.channels_out()
    rtol, atol, rtol_wgrad = 1e-2, 1e-3, 1e-1
    g = torch.Generator(device="cuda").manual_seed(n_in * 100 + n_out)
    for N in batch_sizes:
        print("python suite N =", N, flush=True)
        x = torch.randn((N, n_in), device="cuda", generator=g)
        grad_output = torch.randn((N, n_out), device="cuda", generator=g)
        with torch.no_grad():
            compare_tensors(fused(x), plain(x), "inference, N=%d" % N, rtol, atol)
        for p in list(plain.parameters()) + list(fused.parameters()):
            p.grad = None
        x_plain = x.clone().requires_grad_(True)
        x_fused = x.clone().requires_grad_(True)
        y_plain, y_fused = plain(x_plain), fused(x_fused)
        compare_tensors(y_fused, y_plain, "forward, N=%d" % N, rtol, atol)
        torch.autograd.backward(y_plain, grad_output)
        torch.autograd.backward(y_fused, grad_output)
        compare_tensors(x_fused.grad, x_plain.grad, "input gradients, N=%d" % N, rtol, atol)
        compare_networks(fused, plain, rtol_wgrad, atol)


SINGLE = [(c_in, c_out, act) for c_in in (16, 32, 48) for c_out in (16, 32, 48) for act in ("celu", "identity")]


@pytest.mark.parametrize("c_in,c_out,act", SINGLE)
def test_network_single_layer(c_in, c_out, act):
    cfg = network_cfg(c_in, [c_out], [act])
    warm_or_gpu(network_cfg=cfg)
    run_network_suite(cfg)


# a spread over the product the reference loops over (3 x 3 x 3 widths, 2 x 2 activations)
TWO = [(16, 16, 16, "celu", "celu"), (16, 48, 32, "identity", "celu"), (32, 16, 48, "celu", "identity"),
       (32, 32, 32, "identity", "identity"), (48, 16, 16, "celu", "identity"), (48, 48, 48, "celu", "celu"),
       (16, 32, 48, "identity", "identity"), (48, 32, 16, "identity", "celu")]


@pytest.mark.parametrize("c_in,c_hidden,c_out,act_hidden,act_last", TWO)
def test_network_two_layers(c_in, c_hidden, c_out, act_hidden, act_last):
    cfg = network_cfg(c_in, [c_hidden, c_out], [act_hidden, act_last])
    warm_or_gpu(network_cfg=cfg)
    run_network_suite(cfg)


THREE = [(16, 16, 16, "celu", "celu"), (32, 48, 16, "celu", "identity"), (48, 32, 48, "identity", "celu"),
         (16, 48, 32, "identity", "identity"), (48, 16, 32, "celu", "celu")]


@pytest.mark.parametrize("c_in,c_hidden,c_out,act_hidden,act_last", THREE)
def test_network_three_layers(c_in, c_hidden, c_out, act_hidden, act_last):
    cfg = network_cfg(c_in, [c_hidden, c_hidden, c_out], [act_hidden, act_hidden, act_last])
    warm_or_gpu(network_cfg=cfg)
    run_network_suite(cfg, batch_sizes=(32, 513, 48621))


def test_network_with_bias_and_unpadded_widths():
    """Widths that are no multiples of 16 and biased layers (the reference has no bias gradients)."""
    cfg = network_cfg(5, [20, 24, 3], ["relu", "sine", "identity"], bias=True)
    warm_or_gpu(network_cfg=cfg)
    run_network_suite(cfg, batch_sizes=(35, 4267))


@pytest.mark.parametrize("name", ["relu", "sine", "celu", "identity"])
def test_activation_against_torch(name):
    """_validate_activation of the reference suite (test_activations.py:8-36) on (5, 3) and a larger shape."""
    warm_or_gpu(activation=name)
    activ = FusedActivation(name)
    baseline = FusedActivation.get_activation(name).to(dtype=torch.half, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(1)
    for shape in ((5, 3), (1000, 37)):
        print("activation", name, shape, flush=True)
        x = torch.randn(shape, dtype=torch.half, device="cuda", generator=g).requires_grad_(True)
        y = activ(x)
        y_want = baseline(x)
        assert torch.allclose(y, y_want, rtol=2e-3, atol=1e-3)
        target = torch.randn(shape, dtype=torch.half, device="cuda", generator=g)
        torch.nn.functional.mse_loss(y, target).backward()
        got = x.grad.detach().clone()
        x.grad = None
        torch.nn.functional.mse_loss(baseline(x), target).backward()
        assert torch.allclose(got, x.grad, rtol=2e-3, atol=1e-4)
    # strided input and output shapes; empty input
    xt = torch.randn((37, 64), dtype=torch.half, device="cuda", generator=g).t()
    assert torch.allclose(activ(xt), baseline(xt), rtol=2e-3, atol=1e-3)
    assert activ(torch.zeros((0, 4), dtype=torch.half, device="cuda")).shape == (0, 4)


def test_inline_activation_and_errors():
    spec = json.dumps({"id": "square", "forward": "z = __hmul(x, x)",
                       "adjoint": "adjx = __hmul(__hmul(__float2half(2.0f), x), adjz)"})
    warm_or_gpu(activation=spec)
    activ = FusedActivation(spec)
    x = torch.linspace(-2, 2, 64, dtype=torch.half, device="cuda").reshape(8, 8).requires_grad_(True)
    y = activ(x)
    assert torch.allclose(y, x * x, rtol=1e-3, atol=1e-3)
    y.sum().backward()
    assert torch.allclose(x.grad, 2 * x.detach(), rtol=1e-3, atol=1e-3)
    with pytest.raises(RuntimeError, match="HALF"):
        activ(torch.zeros((4, 4), device="cuda"))


GRID_2D = {"id": "HashGrid", "start_in": 0, "n_in": 2, "n_levels": 2, "n_features_per_level": 4,
           "log2_hashmap_size": -1, "min_resolution": 8, "max_resolution": 16, "combination_mode": "concat",
           "bounding_box_min": [-1, -1], "bounding_box_size": [2, 2]}


def test_encoding_module_autograd_and_gradcheck():
    """_validate_encoding of the reference suite (test_encoding.py:10-78): shapes, parameter
    creation, both gradients, and torch.autograd.gradcheck with its loose settings."""
    cfg = json.dumps(GRID_2D)
    warm_or_gpu(encoding_cfg=cfg)
    enc = FusedEncoding(cfg)
    assert enc.has_parameters() and enc.num_output_channels() == 8 and enc.max_input_channel() == 1
    params = enc.create_parameter_tensor().requires_grad_(True)
    g = torch.Generator(device="cuda").manual_seed(2)
    # the grid is piecewise linear: keep the points away from the cell borders of both levels
    # (resolutions 8 and 16) so that finite differences stay inside one cell
    cand = torch.rand((4000, 2), device="cuda", generator=g) * 1.8 - 0.9
    pos = (cand + 1) / 2
    inside = torch.ones(len(cand), dtype=torch.bool, device="cuda")
    for res in (8, 16):
        frac = (pos * (res - 1)) % 1
        inside &= ((frac > 0.2) & (frac < 0.8)).all(dim=1)
    x = cand[inside][:8].clone().requires_grad_(True)
    assert x.shape == (8, 2)
    y = enc(x, params)
    assert y.shape == (8, 8)
    target = torch.randn(y.shape, device="cuda", generator=g)
    torch.nn.functional.mse_loss(y, target).backward()
    assert x.grad.shape == x.shape and params.grad.shape == params.shape
    assert float(params.grad.abs().sum()) > 0 and float(x.grad.abs().sum()) > 0

    def wrap_input(xd):
        return enc(xd.to(torch.float32), params.detach()).to(torch.double)

    def wrap_params(pd):
        return enc(x.detach(), pd.to(params.dtype)).to(torch.double)

    xd = x.detach().to(torch.double).requires_grad_(True)
    assert torch.autograd.gradcheck(wrap_input, xd, eps=1e-2, atol=1e-1, rtol=1e-1, nondet_tol=1e-3)
    pd = params.detach().to(torch.double).requires_grad_(True)
    assert torch.autograd.gradcheck(wrap_params, pd, eps=1e-1, atol=1e-1, nondet_tol=1e-3)


def test_identity_encoding_module():
    cfg = json.dumps({"id": "Identity", "start_in": 1, "n_in": 3})
    warm_or_gpu(encoding_cfg=cfg)
    enc = FusedEncoding(cfg)
    assert not enc.has_parameters() and enc.num_output_channels() == 3 and enc.max_input_channel() == 3
    x = torch.randn((100, 5), device="cuda").requires_grad_(True)
    y = enc(x)
    assert torch.equal(y, x[:, 1:4])        # the stand-alone kernels write fp32, nothing is rounded
    y.sum().backward()
    want = torch.zeros_like(x)
    want[:, 1:4] = 1
    assert torch.equal(x.grad, want)


def fit_cfg(activation, grid):
    encodings = [{"id": "Identity", "start_in": 0, "n_in": 2}]
    if grid:
        encodings.insert(0, dict(GRID_2D, bounding_box_min=[0, 0], bounding_box_size=[1, 1], n_levels=4,
                                 min_resolution=4, max_resolution=32, n_features_per_level=2))
    return json.dumps({
        "num_inputs": 2, "num_outputs": 3,
        "activation_specification": ["qmlp/builtin-activations.json"],
        "encodings": encodings,
        "network": [{"n_out": 32, "bias": True, "activation": activation},
                    {"n_out": 32, "bias": True, "activation": activation},
                    {"n_out": 3, "bias": True, "activation": "identity"}]})


@pytest.mark.parametrize("activation,grid", [("relu", False), ("sine", False), ("relu", True)])
def test_fit_an_image_with_adam(activation, grid):
    """The training loop of test_network_image.py:13-58 (fp32 master weights, Adam) on a
    synthetic 64 x 64 image: the loss has to fall to about a third of that of the mean image or less."""
    cfg = fit_cfg(activation, grid)
    warm_or_gpu(network_cfg=cfg)
    torch.manual_seed(0)
    net = FusedNetwork(cfg, weight_dtype=torch.float32)
    if grid:
        with torch.no_grad():
            net.encoding_parameters[0].uniform_(-0.1, 0.1)
    yy, xx = torch.meshgrid(torch.linspace(0, 1, 64, device="cuda"), torch.linspace(0, 1, 64, device="cuda"), indexing="ij")
    positions = torch.stack((xx, yy), dim=-1).reshape(-1, 2)
    target = torch.stack((0.5 + 0.5 * torch.sin(6 * xx), yy * xx, (xx - 0.5) ** 2 + (yy - 0.5) ** 2), dim=-1).reshape(-1, 3)
    optim = torch.optim.Adam(net.parameters(), lr=1e-2)
    first = None
    print("image fit", activation, grid, flush=True)
    for _ in range(300):
        optim.zero_grad()
        loss = torch.nn.functional.mse_loss(net(positions), target)
        loss.backward()
        optim.step()
        first = loss.item() if first is None else first
    baseline = torch.nn.functional.mse_loss(target.mean(0, keepdim=True).expand_as(target), target).item()
    assert loss.item() < 0.35 * baseline, (first, loss.item(), baseline)


def test_state_dict_pickle_and_deepcopy():
    """Module state travels like any torch module's; the native object is rebuilt from the
    specification (the reference pickles its custom classes by cfg, bind_network.cpp:404-410)."""
    cfg = fit_cfg("relu", True)
    warm_or_gpu(network_cfg=cfg)
    net = FusedNetwork(cfg, weight_dtype=torch.float32)
    with torch.no_grad():
        net.encoding_parameters[0].normal_(0, 0.1)
    x = torch.rand((200, 2), device="cuda")
    with torch.no_grad():
        want = net(x)
    other = FusedNetwork(cfg, weight_dtype=torch.float32)
    other.load_state_dict(net.state_dict())
    clones = [other, copy.deepcopy(net), pickle.loads(pickle.dumps(net))]
    buffer = io.BytesIO()
    torch.save(net, buffer)
    buffer.seek(0)
    clones.append(torch.load(buffer, weights_only=False))
    for clone in clones:
        with torch.no_grad():
            assert torch.equal(clone(x), want)
    assert repr(net).startswith("FusedNetwork(")


def test_inference_and_train_step_replay_from_a_hip_graph():
    """Nothing on the call path allocates, synchronises or clears memory with a memset, so a
    caller can capture it: inference and a whole train step (forward, backward, weight update,
    reduce) are recorded once and replayed several times with fresh inputs, with eager work and
    synchronisations in between; every replay has to give the eager result bit for bit (the
    grid gradients, summed with atomics, up to fp32 rounding)."""
    cfg = fit_cfg("relu", True)
    warm_or_gpu(network_cfg=cfg)
    net = qmlp.Network(cfg)
    g = torch.Generator(device="cuda").manual_seed(4)
    params = ((torch.rand(net.num_network_parameters(), device="cuda", generator=g) - 0.5) * 0.5).half()
    enc = net.encoding(0)
    table = (torch.rand(enc.num_parameters(), device="cuda", generator=g) - 0.5).to(enc.parameter_dtype())
    tables = [table, None]
    N, flags = 5000, 7
    x = torch.rand((N, 2), device="cuda", generator=g)
    adj = torch.rand((N, 3), device="cuda", generator=g)
    grad_net = torch.zeros(net.num_network_parameters(), device="cuda")
    grad_table = torch.zeros(enc.num_parameters(), device="cuda")
    adj_x = torch.zeros_like(x)

    def step():
        out, tmp = net.forward_raw(x, params, tables, flags)
        net.adjoint_raw(x, adj, flags, tmp, params, tables, grad_network=grad_net,
                        grad_encodings=[grad_table, None], adj_input=adj_x)
        return out, net.inference(x, params, tables)

    def eager():
        for t in (grad_net, grad_table, adj_x):
            t.zero_()
        out, inf = step()
        torch.cuda.synchronize()
        return [t.clone() for t in (out, inf, grad_net, grad_table, adj_x)]

    eager()                                   # kernels loaded, occupancy queried
    graph = torch.cuda.CUDAGraph()
    for t in (grad_net, grad_table, adj_x):
        t.zero_()
    print("hip graph: capture", flush=True)
    with torch.cuda.graph(graph):
        out_g, inf_g = step()
    for replay in range(4):
        x.copy_(torch.rand((N, 2), device="cuda", generator=g))
        adj.copy_(torch.rand((N, 3), device="cuda", generator=g))
        want = eager()                        # eager work and a synchronisation between the replays
        for t in (grad_net, grad_table, adj_x):
            t.zero_()                         # a fill kernel, outside of the graph
        print("hip graph: replay", replay, flush=True)
        graph.replay()
        torch.cuda.synchronize()
        got = [out_g, inf_g, grad_net, grad_table, adj_x]
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), "outputs of replay %d" % replay
        assert torch.equal(got[2], want[2]), "weight gradients of replay %d" % replay
        assert torch.allclose(got[3], want[3], rtol=1e-4, atol=1e-6), "grid gradients of replay %d" % replay
        assert torch.allclose(got[4], want[4], rtol=1e-5, atol=1e-7), "input gradients of replay %d" % replay


def test_a_prepared_network_is_captured_without_an_eager_call_first():
    """``prepare(n, flags)`` loads the kernels of a batch of that size and allocates the workspace that
    orders it by grid slab. A capture right after it, without any eager call before, records inference
    and a train step of a network whose batches are sorted (dense grid beyond the L2, ``sort_points``
    1): loading a kernel or allocating inside the capture would fail it."""
    import baseline_configs as bc
    cfg = json.loads(json.dumps(bc.CONFIGS[5]["cfg"]))
    cfg.setdefault("options", {})["sort_points"] = 1
    cfg = json.dumps(cfg)
    warm_or_gpu(network_cfg=cfg)
    g = torch.Generator(device="cuda").manual_seed(9)
    N, flags = 20000, 7

    def make():
        net = qmlp.Network(cfg)
        return net, net.encoding(0)

    net, enc = make()
    params = ((torch.rand(net.num_network_parameters(), device="cuda", generator=g) - 0.5) * 0.5).half()
    table = (torch.rand(enc.num_parameters(), device="cuda", generator=g) - 0.5).to(enc.parameter_dtype())
    tables = [table, None]
    x = torch.rand((N, 4), device="cuda", generator=g)
    adj = torch.rand((N, 2), device="cuda", generator=g)
    grad_net = torch.zeros(net.num_network_parameters(), device="cuda")
    grad_table = torch.zeros(enc.num_parameters(), device="cuda")
    adj_x = torch.zeros_like(x)

    def step(n):
        out, tmp = n.forward_raw(x, params, tables, flags)
        n.adjoint_raw(x, adj, flags, tmp, params, tables, grad_network=grad_net,
                      grad_encodings=[grad_table, None], adj_input=adj_x)
        return out, n.inference(x, params, tables)

    net.prepare(N, flags)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    print("prepared network: capture", flush=True)
    with torch.cuda.graph(graph):
        out_g, inf_g = step(net)
    print("prepared network: replay", flush=True)
    graph.replay()
    torch.cuda.synchronize()
    got = [t.clone() for t in (out_g, inf_g, grad_net, grad_table, adj_x)]
    # a second network object, eager
    other, _ = make()
    for t in (grad_net, grad_table, adj_x):
        t.zero_()
    out, inf = step(other)
    torch.cuda.synchronize()
    assert torch.equal(got[0], out) and torch.equal(got[1], inf)
    assert torch.equal(got[2], grad_net)
    assert torch.allclose(got[3], grad_table, rtol=1e-4, atol=1e-6)
    assert torch.equal(got[4], adj_x)
    with pytest.raises(qmlp.QmlpError):
        net.prepare(-1, 0)


def two_grid_cfg():
    grid = {"id": "HashGrid", "start_in": 0, "n_in": 2, "n_levels": 2, "n_features_per_level": 4,
            "log2_hashmap_size": 10, "min_resolution": 8, "max_resolution": 64, "combination_mode": "concat",
            "bounding_box_min": [-1.0, -1.0], "bounding_box_size": [2.0, 2.0]}
    return json.dumps({"num_inputs": 2, "num_outputs": 3,
                       "activation_specification": ["qmlp/builtin-activations.json"],
                       "encodings": [grid, dict(grid, n_levels=2, min_resolution=5, max_resolution=9)],
                       "network": [{"n_out": 32, "bias": True, "activation": "celu"},
                                   {"n_out": 3, "bias": False, "activation": "identity"}]})


@pytest.mark.parametrize("scriptable", [False, True])
@pytest.mark.parametrize("frozen", [0, 1])
def test_two_grids_one_of_them_frozen(scriptable, frozen):
    """Encoding gradients with one trainable and one frozen grid: the kernel adds the gradients
    of every grid, so the frozen one gets a throw-away tensor (bind_network.cpp:277-290). The
    trainable grid's gradient equals the one of the run where both are trainable, the frozen
    one has none."""
    cfg = two_grid_cfg()
    warm_or_gpu(network_cfg=cfg)
    torch.manual_seed(5)
    net = FusedNetwork(cfg, weight_dtype=torch.float32, scriptable=scriptable)
    for p in net.encoding_parameters:
        p.data.uniform_(-1, 1)
    x = torch.rand((3000, 2), device="cuda") * 2 - 1
    target = torch.randn((3000, 3), device="cuda")

    def grads(frozen_index):
        for i, p in enumerate(net.encoding_parameters):
            p.requires_grad_(i != frozen_index)
            p.grad = None
        net.weights.grad = None
        torch.nn.functional.mse_loss(net(x), target).backward()
        return [None if p.grad is None else p.grad.clone() for p in net.encoding_parameters], net.weights.grad.clone()

    both, w_both = grads(-1)
    got, w_got = grads(frozen)
    assert got[frozen] is None
    live = 1 - frozen
    assert float(both[live].abs().sum()) > 0
    # float atomics: the order of the additions differs between runs
    assert torch.allclose(got[live], both[live], rtol=1e-4, atol=1e-6)
    assert torch.equal(w_got, w_both)


def test_network_call_after_a_standalone_call_of_its_encoding():
    """net.inference -> net.encoding(0) called on its own with the same table -> net.inference:
    the standalone call leaves the native encoding unbound, the network call has to bind the
    table again."""
    cfg = two_grid_cfg()
    if WARM:
        e = json.loads(cfg)["encodings"][0]
        warm_or_gpu(network_cfg=cfg, encoding_cfg=json.dumps(e))
    warm_or_gpu()
    net = qmlp.Network(cfg)
    torch.manual_seed(6)
    params = torch.randn(net.num_network_parameters(), device="cuda").half() / 4
    tables = [torch.rand(net.encoding(i).num_parameters(), device="cuda") for i in range(2)]
    x = torch.rand((777, 2), device="cuda") * 2 - 1
    first = net.inference(x, params, tables)
    alone = net.encoding(0).inference_with_parameter(x, tables[0])
    assert alone.shape == (777, 8)
    again = net.inference(x, params, tables)
    assert torch.equal(first, again)
    gi, gp = net.encoding(0).adjoint_with_parameter(x, tables[0], torch.ones_like(alone))
    assert gp.shape == tables[0].shape
    assert torch.equal(first, net.inference(x, params, tables))


def test_memset_of_the_loader_is_a_fill_kernel_that_handles_any_alignment():
    """qmlp_hip_memset_async (what Tensor::zero_ and zeroGradients() use) launches a kernel instead
    of hipMemsetAsync, so that a captured train step records no memset node; ranges that start
    and end off a 16-byte boundary, inside a larger buffer whose other bytes must stay."""
    import ctypes
    warm_or_gpu()
    lib = qmlp._lib.lib
    buf = torch.full((70_000,), 0x5a, dtype=torch.uint8, device="cuda")
    want = buf.clone()
    stream = qmlp._lib.current_stream(buf.device)
    for offset, count, value in ((0, 16, 1), (3, 1, 2), (5, 11, 3), (29, 4099, 0), (4500, 65_000, 0xee), (69_999, 1, 7), (100, 0, 9)):
        assert lib.qmlp_hip_memset_async(ctypes.c_void_p(buf.data_ptr() + offset), value, ctypes.c_size_t(count), stream) == 0
        want[offset:offset + count] = value
    torch.cuda.synchronize()
    assert torch.equal(buf, want)
    # recorded into a HIP graph it stays a kernel: replays give the same bytes
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            s = qmlp._lib.current_stream(buf.device)
            assert lib.qmlp_hip_memset_async(ctypes.c_void_p(buf.data_ptr() + 7), 0, ctypes.c_size_t(33_333), s) == 0
    want[7:7 + 33_333] = 0
    for _ in range(3):
        buf[7:7 + 33_333] = 0x11
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(buf, want)
