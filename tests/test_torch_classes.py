"""torch.classes.qmlp_cu.* (quick-mlp_amd/csrc/torch/qmlp_torch.cpp, on the C ABI): registration, pickling and
TorchScript on the CPU; on the GPU the same numbers as the ctypes mirror of the classes, autograd, and
script / trace -> save -> load round trips like the reference's Python tests
(tests_py/qmlp_tests/test_activations.py:38-55, test_encoding.py:80-105)."""
import io
import json
import os

import pytest
import torch

import qmlp

try:
    Q = qmlp.load_library()
except ImportError:      # not built yet (a GPU box only loads what is built; here it takes a minute)
    import subprocess
    subprocess.run(["make", "-C", os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                                               "quick-mlp_amd", "csrc", "torch")], check=True, capture_output=True)
    Q = qmlp.load_library()

NETWORK_CFG = json.dumps({
    "num_inputs": 16, "num_outputs": 16, "activation_specification": ["qmlp/builtin-activations.json"],
    "encodings": [{"id": "Identity", "start_in": 0, "n_in": 16}],
    "network": [{"n_out": 16, "bias": False, "activation": "celu"}]})
GRID_CFG = json.dumps({"id": "HashGrid", "start_in": 0, "n_in": 2, "n_levels": 2, "n_features_per_level": 4,
                       "log2_hashmap_size": -1, "min_resolution": 8, "max_resolution": 16, "combination_mode": "concat",
                       "bounding_box_min": [-1, -1], "bounding_box_size": [2, 2]})


class ActivationModule(torch.nn.Module):
    def __init__(self, name: str):
        super().__init__()
        self.activation = Q.Activation(name)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.activation.forward(x)


class NetworkModule(torch.nn.Module):
    def __init__(self, cfg: str):
        super().__init__()
        self.network = Q.Network(cfg, ".")
        weights = torch.zeros(self.network.num_network_parameters(), dtype=torch.float16)
        self.weights = torch.nn.Parameter(weights)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.network.forward(x, self.weights, [])


def test_classes_are_registered_and_pickle_by_their_specification():
    assert Q.Network.MatrixSize() == 16 and Q.Network.WarpSize() == 64 and Q.Network.MaxSharedMemoryBytes() == 160 * 1024
    assert isinstance(Q.QuickMLP.is_cuda_available(), bool)
    net = Q.Network(NETWORK_CFG, ".")
    assert (net.num_layers(), net.channels_in(), net.channels_out(), net.num_encodings()) == (1, 16, 16, 1)
    assert net.num_network_parameters() == 256 and net.cfg() == NETWORK_CFG and net.parent() == "."
    enc = net.encoding(0)
    assert json.loads(enc.to_json())["id"] == "Identity" and not enc.has_parameters() and enc.num_output_channels() == 16
    grid = Q.Encoding(GRID_CFG)
    assert grid.has_parameters() and grid.num_output_channels() == 8 and grid.max_input_channel() == 1
    for obj, check in ((net, lambda o: o.num_network_parameters() == 256), (grid, lambda o: o.num_output_channels() == 8),
                       (Q.Activation("sine"), lambda o: o.cfg() == "sine")):
        buffer = io.BytesIO()
        torch.save(obj, buffer)
        buffer.seek(0)
        assert check(torch.load(buffer, weights_only=False))
    with pytest.raises(RuntimeError, match="No activation with id"):
        Q.Activation("swish")


def test_modules_with_the_classes_script_save_and_load(tmp_path):
    scripted = torch.jit.script(NetworkModule(NETWORK_CFG))
    assert "forward" in scripted.code
    path = str(tmp_path / "network.pt")
    torch.jit.save(scripted, path)
    loaded = torch.jit.load(path)
    assert loaded.network.num_network_parameters() == 256 and loaded.weights.shape == (256,)
    scripted = torch.jit.script(ActivationModule("celu"))
    torch.jit.save(scripted, str(tmp_path / "activation.pt"))
    assert torch.jit.load(str(tmp_path / "activation.pt")).activation.cfg() == "celu"


def _gpu_or_skip():
    if os.environ.get("QMLP_WARM_CACHE"):
        qmlp.Network(NETWORK_CFG).precompile(7)
        qmlp.Activation("sine").precompile()
        enc = qmlp.Encoding(GRID_CFG)
        for mode in (0, 1, 2, 3):
            enc.precompile(mode)
        qmlp.pullpush.precompile(torch.float32)
        pytest.skip("kernel cache warmed")
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")


@pytest.mark.gpu
def test_network_class_gives_the_numbers_of_the_ctypes_mirror(tmp_path):
    _gpu_or_skip()
    g = torch.Generator(device="cuda").manual_seed(0)
    net_t, net_c = Q.Network(NETWORK_CFG, "."), qmlp.Network(NETWORK_CFG)
    params = net_t.create_inference_parameters()
    net_t.initialize_inference_parameters(params)
    assert params.dtype == torch.float16 and float(params.float().abs().max()) <= 0.25 and float(params.float().abs().sum()) > 0
    view = net_t.parameter_view(0, False, params)
    assert view.shape == (16, 16) and view.data_ptr() == params.data_ptr() and net_t.parameter_view(0, True, params) is None
    x = torch.randn((1000, 16), device="cuda", generator=g)
    assert torch.equal(net_t.inference(x, params, []), net_c.inference(x, params, []))
    # autograd, fp32 master weights
    adj = torch.randn((1000, 16), device="cuda", generator=g)
    grads = []
    for net in (net_t, net_c):
        xi = x.clone().requires_grad_(True)
        w = params.float().requires_grad_(True)
        out = net.forward(xi, w, [])
        out.backward(adj)
        grads.append((out.detach(), xi.grad, w.grad))
    for a, b in zip(*grads):
        assert torch.equal(a, b)
    assert grads[0][2].dtype == torch.float32 and float(grads[0][2].abs().sum()) > 0
    # a scripted module that owns the network: save, load, same output
    module = NetworkModule(NETWORK_CFG).cuda()
    with torch.no_grad():
        module.weights.copy_(params)
    scripted = torch.jit.script(module)
    torch.jit.save(scripted, str(tmp_path / "network.pt"))
    loaded = torch.jit.load(str(tmp_path / "network.pt"))
    with torch.no_grad():
        assert torch.equal(loaded(x), net_c.inference(x, params, []))
    y = loaded(x.clone().requires_grad_(True))
    y.sum().backward()
    assert loaded.weights.grad is not None and loaded.weights.grad.dtype == torch.float16


@pytest.mark.gpu
def test_activation_and_encoding_classes(tmp_path):
    _gpu_or_skip()
    g = torch.Generator(device="cuda").manual_seed(1)
    act_t, act_c = Q.Activation("sine"), qmlp.Activation("sine")
    x = torch.randn((5, 3), device="cuda", generator=g, dtype=torch.float16).requires_grad_(True)
    y = act_t.forward(x)
    assert torch.equal(y, act_c.inference(x.detach())) and torch.allclose(y, torch.sin(x), rtol=2e-3, atol=1e-3)
    y.sum().backward()
    assert torch.allclose(x.grad, torch.cos(x.detach()), rtol=2e-3, atol=1e-3)
    # trace -> freeze -> save -> load, as in the reference's activation test
    module = ActivationModule("sine").eval()
    traced = torch.jit.freeze(torch.jit.trace(module, (x.detach(),)))
    torch.jit.save(traced, str(tmp_path / "activation.pt"))
    assert torch.equal(torch.jit.load(str(tmp_path / "activation.pt"))(x.detach()), y.detach())

    enc_t, enc_c = Q.Encoding(GRID_CFG), qmlp.Encoding(GRID_CFG)
    table = enc_t.create_inference_parameters()
    assert table.shape == (enc_c.num_parameters(),) and table.dtype == enc_c.parameter_dtype()
    table = torch.randn(table.shape, device="cuda", generator=g).to(table.dtype)
    pos = torch.rand((300, 2), device="cuda", generator=g) * 1.8 - 0.9
    assert torch.equal(enc_t.inference_with_parameter(pos, table), enc_c.inference_with_parameter(pos, table))
    results = []
    for enc in (enc_t, enc_c):
        p = pos.clone().requires_grad_(True)
        t = table.clone().requires_grad_(True)
        out = enc.forward_with_parameter(p, t)
        out.square().sum().backward()
        results.append((out.detach(), p.grad, t.grad))
    assert torch.equal(results[0][0], results[1][0]) and torch.equal(results[0][1], results[1][1])
    assert torch.allclose(results[0][2], results[1][2], rtol=1e-4, atol=1e-5)      # atomics: order of the sums
    identity = Q.Encoding(json.dumps({"id": "Identity", "start_in": 1, "n_in": 1}))
    assert torch.equal(identity.forward(pos), pos[:, 1:2])
    with pytest.raises(RuntimeError, match="has parameters"):
        enc_t.inference(pos)


@pytest.mark.gpu
def test_pullpush_class():
    _gpu_or_skip()
    g = torch.Generator(device="cuda").manual_seed(2)
    mask = (torch.rand((1, 12, 16), device="cuda", generator=g) > 0.7).float()
    data = torch.rand((1, 3, 12, 16), device="cuda", generator=g).requires_grad_(True)
    out = Q.utils.pullpush(mask, data)
    assert torch.equal(out, qmlp.pullpush.pullpush(mask, data.detach()))
    out.sum().backward()
    gm, gd = Q.utils.pullpush_backward(mask, data.detach(), torch.ones_like(out))
    assert torch.equal(data.grad, gd) and gm.shape == mask.shape
    assert torch.equal(Q.utils.pullpush_forward(mask, data.detach()), out.detach())


@pytest.mark.gpu
def test_scriptable_modules_trace_save_and_load(tmp_path):
    """FusedActivation / FusedEncoding / FusedNetwork with scriptable=True hold the torch custom
    classes: torch.jit.trace -> freeze -> save -> load as in the reference's module tests, and the
    same numbers as the default modules."""
    _gpu_or_skip()
    g = torch.Generator(device="cuda").manual_seed(3)

    act = qmlp.FusedActivation("sine", scriptable=True).eval()
    x = torch.randn((5, 3), device="cuda", generator=g, dtype=torch.float16)
    traced = torch.jit.freeze(torch.jit.trace(act, (x,)))
    torch.jit.save(traced, str(tmp_path / "act.pt"))
    assert torch.equal(torch.jit.load(str(tmp_path / "act.pt"))(x), qmlp.FusedActivation("sine")(x))

    enc = qmlp.FusedEncoding(GRID_CFG, scriptable=True).eval()
    table = enc.create_parameter_tensor()
    pos = torch.rand((64, 2), device="cuda", generator=g) * 1.8 - 0.9
    traced = torch.jit.freeze(torch.jit.trace(enc, (pos, table)))
    torch.jit.save(traced, str(tmp_path / "enc.pt"))
    assert torch.equal(torch.jit.load(str(tmp_path / "enc.pt"))(pos, table), qmlp.FusedEncoding(GRID_CFG)(pos, table))

    torch.manual_seed(0)
    net = qmlp.FusedNetwork(NETWORK_CFG, weight_dtype=torch.float32, scriptable=True)
    plain = qmlp.FusedNetwork(NETWORK_CFG, weight_dtype=torch.float32)
    plain.load_state_dict(net.state_dict())
    xin = torch.randn((500, 16), device="cuda", generator=g)
    adj = torch.randn((500, 16), device="cuda", generator=g)
    outs = []
    for module in (net, plain):
        xi = xin.clone().requires_grad_(True)
        y = module(xi)
        y.backward(adj)
        outs.append((y.detach(), xi.grad, module.weights.grad.clone()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    net.eval()
    with torch.no_grad():
        traced = torch.jit.trace(net, (xin,))
    torch.jit.save(traced, str(tmp_path / "net.pt"))
    loaded = torch.jit.load(str(tmp_path / "net.pt"))
    with torch.no_grad():
        assert torch.equal(loaded(xin), outs[1][0])
    # pickling and deepcopy of the module that holds the custom class
    import copy
    import pickle
    for clone in (copy.deepcopy(net), pickle.loads(pickle.dumps(net))):
        with torch.no_grad():
            assert torch.equal(clone(xin), outs[1][0])
        assert clone.encoding(0).num_output_channels() == 16
