"""The launch options of a network specification ("options": overwrite_blocksize_inference /
_forward / _backward / _weight_update, parallel_weight_update, skew_shared_memory; reference:
src_cpp/src/fused_network.cpp:45-69) change the workgroups of every generated kernel. Each value
runs against the CPU oracle on the GPU; the reference exercises them as the three sections
serial / parallel / parallel + skew of tests_cpp/test_against_eigen1.cpp:70-86."""
import json
import re

import numpy as np
import pytest

import qmlp
from helpers import (Case, FLAG_ENC, FLAG_INPUT, FLAG_WEIGHTS, assert_close, check_gradients, identity_cfg,
                     random_parameters, warm_cache)

pytestmark = pytest.mark.gpu


def _identity_network():
    cfg = identity_cfg(19, [48, 32, 5], ["celu", "sine", "identity"], [True, False, True])
    return cfg, None, 19, 5


def _grid_network():
    """The fused grid + identity network of test_fused_grid_network_against_oracle."""
    grid = {"id": "HashGrid", "start_in": 1, "n_in": 3, "n_levels": 6, "n_features_per_level": 2,
            "log2_hashmap_size": 10, "min_resolution": 4, "max_resolution": 128, "combination_mode": "concat",
            "bounding_box_min": [-0.5, 0.0, 0.25], "bounding_box_size": [1.0, 2.0, 0.5], "parameter_precision": "half"}
    cfg = {"num_inputs": 4, "num_outputs": 3, "activation_specification": ["qmlp/builtin-activations.json"],
           "encodings": [grid, {"id": "Identity", "start_in": 0, "n_in": 2}],
           "network": [{"n_out": 32, "bias": True, "activation": "celu"},
                       {"n_out": 3, "bias": False, "activation": "identity"}]}
    return cfg, grid, 4, 3


def _streamed_network():
    """200 K fp16 weights: three of the layers are staged into LDS right before they run."""
    widths = [128] * 6 + [16]
    return identity_cfg(19, widths, ["celu"] * len(widths), [True] * len(widths)), None, 19, 16


NETWORKS = {"identity": _identity_network, "grid": _grid_network, "streamed": _streamed_network}


def _run(cfg, grid, n_in, n_out, N, seed=5):
    case = Case(cfg)
    rng = np.random.default_rng(seed)
    case.set_parameters(random_parameters(case.oracle, rng))
    lo, sz = np.zeros(n_in, np.float32), np.ones(n_in, np.float32)
    if grid is not None:
        case.set_table(0, rng.uniform(-1, 1, case.oracle.encodings[0][1].n_params))
        s = grid["start_in"]
        lo[s:s + 3] = grid["bounding_box_min"]
        sz[s:s + 3] = grid["bounding_box_size"]
    else:
        lo[:] = -1
        sz[:] = 2
    X = (lo + sz * rng.uniform(0, 1, (N, n_in))).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, n_out)) / 16).astype(np.float32)
    flags = FLAG_INPUT | FLAG_WEIGHTS | (FLAG_ENC if grid is not None else 0)
    inference = case.gpu_inference(X)
    got = case.gpu_train(X, adj, flags)
    expected = case.oracle.forward(X)
    assert_close(inference, expected, "inference")
    assert_close(got["out"], expected, "forward")
    check_gradients(case, X, adj, flags, got)
    return case, inference, got


def _launch_bounds(source, kernel):
    m = re.search(r"__launch_bounds__\((\d+)\)[^;{]*?\b%s\b" % kernel, source, re.S)
    assert m, kernel
    return int(m.group(1))


@pytest.mark.parametrize("block", [64, 128, 512, 1024])
@pytest.mark.parametrize("which", sorted(NETWORKS))
def test_overwritten_block_sizes_of_the_fused_kernels(which, block):
    cfg, grid, n_in, n_out = NETWORKS[which]()
    N = 3000 if which != "streamed" else 1500
    plain = json.loads(json.dumps(cfg))
    cfg["options"] = {"overwrite_blocksize_inference": block, "overwrite_blocksize_forward": block,
                      "overwrite_blocksize_backward": block}
    warm_cache(plain, cfg)
    _, base_inference, base = _run(plain, grid, n_in, n_out, N)
    case, inference, got = _run(cfg, grid, n_in, n_out, N)
    net = case.net
    # the kernels are generated for workgroups of this size (less only where the staging rows
    # of so many wavefronts exceed the LDS, as the reference shrinks its blocks)
    sizes = {"inference": _launch_bounds(net.generated_source("inference"), "NetworkKernelInferenceAndForward"),
             "forward": _launch_bounds(net.generated_source("forward"), "NetworkKernelInferenceAndForward"),
             "backward": _launch_bounds(net.generated_source("backward", 7 if grid else 3), "NetworkKernelBackward")}
    for kind, size in sizes.items():
        assert size == block or (size < block and size % 64 == 0 and which == "streamed"), (kind, size)
    # every point is evaluated on its own: the shape of the workgroups does not show in the outputs
    assert np.array_equal(inference, base_inference)
    assert np.array_equal(got["out"], base["out"])
    assert np.array_equal(got["adj_x"], base["adj_x"])


@pytest.mark.parametrize("block", [64, 256])
@pytest.mark.parametrize("which", sorted(NETWORKS))
def test_overwritten_block_size_of_the_weight_update(which, block):
    cfg, grid, n_in, n_out = NETWORKS[which]()
    # every layer gets a weight-update kernel of its own
    cfg["options"] = {"overwrite_blocksize_weight_update": block, "fused_weight_update": 0}
    case, _, _ = _run(cfg, grid, n_in, n_out, 3000 if which != "streamed" else 1500)
    assert _launch_bounds(case.net.generated_source("weight_update"), "WeightUpdateKernel") == block


@pytest.mark.parametrize("section,options", [
    ("serial-noSkew", {"parallel_weight_update": False, "skew_shared_memory": False}),
    ("parallel-noSkew", {"parallel_weight_update": True, "skew_shared_memory": False}),
    ("parallel-skew", {"parallel_weight_update": True, "skew_shared_memory": True}),
])
@pytest.mark.parametrize("which", ["identity", "grid"])
def test_option_sections_of_the_reference_tests(which, section, options):
    """The same numbers whatever the section: the weight-update kernels of the layers run one
    after the other or side by side on their own streams, and the LDS layout is free of bank
    conflicts by construction, so the skew option changes nothing."""
    cfg, grid, n_in, n_out = NETWORKS[which]()
    plain = json.loads(json.dumps(cfg))
    # layers with a kernel of their own are what the option distributes over streams
    cfg["options"] = dict(options, fused_weight_update=0)
    cfg_default = json.loads(json.dumps(cfg))
    cfg_default["options"] = {"fused_weight_update": 0}
    warm_cache(plain, cfg, cfg_default)
    _, base_inference, base = _run(plain, grid, n_in, n_out, 4267)
    _, inference, got = _run(cfg, grid, n_in, n_out, 4267)
    assert np.array_equal(inference, base_inference)
    assert np.array_equal(got["out"], base["out"])
    _, _, serial = _run(cfg_default, grid, n_in, n_out, 4267)
    assert np.array_equal(got["grads"], serial["grads"])      # fixed order of the sums on every stream
