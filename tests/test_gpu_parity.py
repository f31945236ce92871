"""GPU parity tests: the HIP path, called through the C ABI of libqmlp.so, against the CPU
oracle on the same seeded inputs. Shapes follow the reference's own tests
(tests_cpp/test_against_eigen1.cpp:26-61, test_against_eigen2.cpp:17-28,
tests_py/qmlp_tests/test_network_base.py:87-256). Tolerance of every floating point
comparison: rel 1e-2 / abs 1e-3 against the fp32 oracle, no entry may exceed it."""
import json
import os

import numpy as np
import pytest
import torch

import qmlp
import qmlp_oracle as qo
from helpers import (ABS, REL, Case, FLAG_ENC, FLAG_INPUT, FLAG_WEIGHTS, assert_close, baseline_case,
                     check_gradients, identity_cfg, random_parameters, require_gpu, warm_cache)
import baseline_configs as bc

pytestmark = pytest.mark.gpu

ONE_LAYER = [(c0, c1, act) for (c0, c1) in [(16, 16), (16, 32), (48, 16), (48, 32), (16, 48), (32, 16), (32, 48)]
             for act in ("sine", "celu", "identity", "relu")]


@pytest.mark.parametrize("c0,c1,act", ONE_LAYER)
@pytest.mark.parametrize("bias", [False, True])
def test_one_layer_against_oracle(c0, c1, act, bias):
    case = Case(identity_cfg(c0, [c1], [act], [bias]))
    rng = np.random.default_rng(42)
    N = 35
    for trial in range(3):
        case.set_parameters(random_parameters(case.oracle, rng))
        X = rng.uniform(0, 1, (N, c0)).astype(np.float32)
        adj = rng.uniform(-1, 1, (N, c1)).astype(np.float32)
        assert_close(case.gpu_inference(X), case.oracle.forward(X), "inference")
        got = case.gpu_train(X, adj, FLAG_INPUT)
        assert_close(got["out"], case.oracle.forward(X), "forward")
        check_gradients(case, X, adj, FLAG_INPUT, got, kinks=act == "relu", kink_fraction=0.09)
        got = case.gpu_train(X, adj, FLAG_WEIGHTS)
        check_gradients(case, X, adj, FLAG_WEIGHTS, got, kinks=act == "relu", kink_fraction=0.09)


TWO_LAYER = [(16, 16, 16), (19, 16, 16), (16, 16, 23), (20, 16, 24), (32, 48, 16), (32, 48, 32)]


@pytest.mark.parametrize("c0,c1,c2", TWO_LAYER)
@pytest.mark.parametrize("acts", [("identity", "identity"), ("sine", "identity"), ("celu", "celu"), ("relu", "sine")])
def test_two_layers_against_oracle(c0, c1, c2, acts):
    case = Case(identity_cfg(c0, [c1, c2], list(acts), [False, False]))
    rng = np.random.default_rng(42)
    N = 32
    case.set_parameters(random_parameters(case.oracle, rng))
    X = rng.uniform(-1, 1, (N, c0)).astype(np.float32)
    adj = rng.uniform(-1, 1, (N, c2)).astype(np.float32)
    assert_close(case.gpu_inference(X), case.oracle.forward(X), "inference")
    kinks = "relu" in acts
    for flags in (FLAG_INPUT, FLAG_WEIGHTS, FLAG_INPUT | FLAG_WEIGHTS):
        check_gradients(case, X, adj, flags, case.gpu_train(X, adj, flags), kinks, "flags %d: " % flags)
    # the adjoint at one entry of a padded last layer (the case the reference marks as failing)
    one = np.zeros_like(adj)
    one[2, min(14, c2 - 1)] = 2.0
    check_gradients(case, X, one, FLAG_INPUT, case.gpu_train(X, one, FLAG_INPUT), kinks, "single entry: ")


def test_one_activation_per_channel():
    """Lists of activations, one per output channel (the reference parses them and then throws,
    src_cpp/src/fused_network.cpp:112-125,447)."""
    acts0 = ["relu", "sine", "celu", "identity"] * 5
    acts1 = ["sine", "identity", "celu", "celu", "sine"]
    case = Case(identity_cfg(16, [20, 5], [acts0, acts1], [True, False]))
    rng = np.random.default_rng(31)
    case.set_parameters(random_parameters(case.oracle, rng))
    N = 700
    X = rng.uniform(-1, 1, (N, 16)).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, 5)) / 8).astype(np.float32)
    assert_close(case.gpu_inference(X), case.oracle.forward(X), "inference")
    flags = FLAG_INPUT | FLAG_WEIGHTS
    got = case.gpu_train(X, adj, flags)
    assert_close(got["out"], case.oracle.forward(X), "forward")
    check_gradients(case, X, adj, flags, got, kinks=True)
    # a uniform list equals the single name
    same = Case(identity_cfg(16, [20, 5], [["celu"] * 20, "identity"], [True, False]))
    single = Case(identity_cfg(16, [20, 5], ["celu", "identity"], [True, False]))
    p = random_parameters(single.oracle, rng)
    same.set_parameters(p)
    single.set_parameters(p)
    assert np.array_equal(same.gpu_inference(X), single.gpu_inference(X))


@pytest.mark.parametrize("widths,act", [([128] * 6 + [16], "celu"), ([256, 256, 256, 3], "sine"), ([512, 208, 16], "identity")])
def test_networks_whose_weights_exceed_the_lds(widths, act):
    """More than 160 KB of fp16 weights: some layers stay in LDS, the others are staged into a
    shared LDS buffer right before they run (the first two networks) or, if a single layer
    exceeds the LDS, gathered from global memory (the third: W in the forward pass, a transposed
    copy in the adjoint memory in the adjoint pass)."""
    n_in = 19
    case = Case(identity_cfg(n_in, widths, [act] * len(widths), [True] * len(widths)))
    fwd, bwd = case.net.generated_source("forward"), case.net.generated_source("backward", 7)
    if widths[0] == 512:
        assert "forward<STORE, true, " in fwd and "transposedWeights +" in bwd
    else:
        assert "the stream buffer is free" in fwd and "the stream buffer is free" in bwd
    rng = np.random.default_rng(77)
    case.set_parameters(random_parameters(case.oracle, rng))
    N = 1500
    X = rng.uniform(-1, 1, (N, n_in)).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, widths[-1])) / N).astype(np.float32)
    assert_close(case.gpu_inference(X), case.oracle.forward(X), "inference")
    for flags in (FLAG_INPUT | FLAG_WEIGHTS, FLAG_INPUT):
        got = case.gpu_train(X, adj, flags)
        assert_close(got["out"], case.oracle.forward(X), "forward")
        check_gradients(case, X, adj, flags, got, what="flags %d: " % flags)


@pytest.mark.parametrize("widths", [[16], [32, 16], [48, 32, 16], [16, 48, 48]])
@pytest.mark.parametrize("act", ["celu", "identity"])
@pytest.mark.parametrize("N", [16, 32, 128, 513, 48621])
def test_python_suite_shapes(widths, act, N):
    n_in = 16
    case = Case(identity_cfg(n_in, widths, [act] * len(widths), [True] * len(widths)))
    rng = np.random.default_rng(N)
    case.set_parameters(random_parameters(case.oracle, rng))
    X = rng.uniform(-1, 1, (N, n_in)).astype(np.float32)
    adj = rng.uniform(-1, 1, (N, widths[-1])).astype(np.float32)
    assert_close(case.gpu_inference(X), case.oracle.forward(X), "inference")
    got = case.gpu_train(X, adj, FLAG_INPUT | FLAG_WEIGHTS)
    assert_close(got["out"], case.oracle.forward(X), "forward")
    check_gradients(case, X, adj, FLAG_INPUT | FLAG_WEIGHTS, got)


@pytest.mark.parametrize("widths,acts,N", [([32, 32, 16], ["relu", "celu", "identity"], 5000),
                                          ([64, 64, 16], ["celu", "relu", "identity"], 20001),
                                          ([64] * 8 + [16], ["relu", "celu"] * 4 + ["identity"], 131073)])
def test_weight_gradients_summed_in_the_backward_kernel_match_the_weight_update_kernels(widths, acts, N):
    """options.fused_weight_update: 0 = one weight-update kernel per layer reads the adjoint pre-activations that the
    backward kernel stored; -1 (default) = the backward kernel sums the gradient tiles of the layers with the fewest
    tiles itself (Layer::weightGradient), up to 16 tiles; 1 = up to 32 tiles. Same products, another order of the
    fp32 sums: all three against each other and, the smallest batch, against the oracles. The backward kernel of the
    last network takes 113 KB of LDS: one workgroup per compute unit, fewer than the 512 batch slices of 131 073
    points, so it also zeroes the slices beyond its grid."""
    n_in = 16
    rng = np.random.default_rng(len(widths))
    X = rng.uniform(-1, 1, (N, n_in)).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, widths[-1])) / np.sqrt(N)).astype(np.float32)
    params = None
    got = {}
    for mode in (0, -1, 1):
        cfg = identity_cfg(n_in, widths, acts, [True] * (len(widths) - 1) + [False])
        cfg["options"] = {"fused_weight_update": mode}
        case = Case(cfg)
        if params is None:
            params = random_parameters(case.oracle, rng)
        case.set_parameters(params)
        src = case.net.generated_source("backward", FLAG_INPUT | FLAG_WEIGHTS)
        assert ("::template weightGradient<" in src) == (mode != 0)
        flags = FLAG_INPUT | FLAG_WEIGHTS
        got[mode] = case.gpu_train(X, adj, flags)
        if mode == -1 and widths == [64, 64, 16]:
            # 27 gradient tiles, the 16 of the 64 x 64 layer among them: all in the accumulation registers of a
            # kernel that runs one wavefront per SIMD, none of them spilled
            assert src.count("::template weightGradient<") == 3 and "amdgpu_waves_per_eu(1, 1)" in src
            res = json.loads(case.net.generated_source("backward_resources", flags))
            assert res["scratch_bytes"] == 0 and 256 < res["registers"] <= 512 and res["block"] == 256, res
        # (the larger batches only mode against mode, which is the tighter comparison: with gradient entries of order
        # one, sums over tens of thousands of points with ReLU units that an fp16 rounding switches leave the
        # tolerances of the oracle comparison, for the weight-update kernels as for the fused sums)
        if N <= 5000:
            check_gradients(case, X, adj, flags, got[mode], kinks=True, what="fused_weight_update %d: " % mode)
    # the layers that keep a weight-update kernel may run on streams of their own beside the caller's: same sums
    cfg = identity_cfg(n_in, widths, acts, [True] * (len(widths) - 1) + [False])
    cfg["options"] = {"fused_weight_update": -1, "parallel_weight_update": True}
    case = Case(cfg)
    case.set_parameters(params)
    side_by_side = case.gpu_train(X, adj, FLAG_INPUT | FLAG_WEIGHTS)
    assert np.array_equal(side_by_side["grads"], got[-1]["grads"])
    scale = float(np.abs(got[0]["grads"]).max())
    for mode in (-1, 1):
        assert np.allclose(got[mode]["grads"] / scale, got[0]["grads"] / scale, rtol=1e-3, atol=1e-5), mode
        assert np.array_equal(got[mode]["adj_x"], got[0]["adj_x"]) and np.array_equal(got[mode]["out"], got[0]["out"])


def test_round_mode_oracle_is_tighter():
    """Against the oracle that rounds where the device rounds, the error shrinks by an order."""
    case = Case(identity_cfg(16, [64, 64, 4], ["relu", "celu", "identity"], [True, True, True]))
    rng = np.random.default_rng(1)
    case.set_parameters(random_parameters(case.oracle, rng))
    X = rng.uniform(-1, 1, (1000, 16)).astype(np.float32)
    got = case.gpu_inference(X)
    assert_close(got, case.oracle.forward(X, round_mode=0), "fp32 oracle")
    assert_close(got, case.oracle.forward(X, round_mode=1), "fp16-rounding oracle", rel=2e-3, abs_=2e-4)


# ---------------------------------------------------------------------------- edge cases
@pytest.mark.parametrize("N", [0, 1, 63, 64, 65, 127, 129, 4267])
def test_ragged_batch_sizes(N):
    case = Case(identity_cfg(5, [32, 3], ["relu", "identity"], [True, False]))
    rng = np.random.default_rng(N + 1)
    case.set_parameters(random_parameters(case.oracle, rng))
    X = rng.uniform(-1, 1, (N, 5)).astype(np.float32)
    adj = rng.uniform(-1, 1, (N, 3)).astype(np.float32)
    out = case.gpu_inference(X)
    assert out.shape == (N, 3)
    if N == 0:
        got = case.gpu_train(X, adj, FLAG_INPUT | FLAG_WEIGHTS)
        assert got["adj_x"].shape == (0, 5) and not got["grads"].any()
        return
    assert_close(out, case.oracle.forward(X), "inference")
    got = case.gpu_train(X, adj, FLAG_INPUT | FLAG_WEIGHTS)
    check_gradients(case, X, adj, FLAG_INPUT | FLAG_WEIGHTS, got, kinks=True)


def test_strided_tensors_and_gradient_accumulation():
    case = Case(identity_cfg(4, [16, 2], ["celu", "identity"], [False, True]))
    rng = np.random.default_rng(5)
    case.set_parameters(random_parameters(case.oracle, rng))
    N = 200
    X = rng.uniform(-1, 1, (N, 4)).astype(np.float32)
    adj = rng.uniform(-1, 1, (N, 2)).astype(np.float32)
    big_in = torch.zeros((N, 9), device="cuda")
    x = big_in[:, 1:9:2]                      # stride (9, 2)
    x.copy_(torch.from_numpy(X))
    xt = torch.from_numpy(X.T.copy()).cuda().t()   # column-major input
    ref_out = case.oracle.forward(X)
    for inp in (x, xt):
        out = case.net.inference(inp, case.params, [])
        assert_close(out.cpu().numpy(), ref_out, "strided inference")
    # strided adjoint output and accumulation into existing gradients
    a = torch.zeros((N, 6), device="cuda")[:, ::3]
    a.copy_(torch.from_numpy(adj))
    out, tmp = case.net.forward_raw(x, case.params, [], 3)
    adj_in = torch.ones((N, 8), device="cuda")[:, ::2]
    gnet = torch.full((case.net.num_network_parameters(),), 0.5, device="cuda")
    case.net.adjoint_raw(x, a, 3, tmp, case.params, [], grad_network=gnet, adj_input=adj_in)
    torch.cuda.synchronize()
    got = dict(adj_x=adj_in.cpu().numpy() - 1.0, grads=gnet.cpu().numpy() - 0.5)
    check_gradients(case, X, adj, 3, got, what="accumulated ")


def test_shape_and_type_errors_are_reported():
    import qmlp
    case = Case(identity_cfg(4, [16, 2], ["relu", "identity"], [False, False]))
    case.set_parameters(np.zeros(case.oracle.num_parameters, np.float32))
    with pytest.raises(qmlp.QmlpError, match="must have 4 entries"):
        case.net.inference(torch.zeros((8, 5), device="cuda"), case.params, [])
    with pytest.raises(qmlp.QmlpError, match="must be of type FLOAT"):
        case.net.inference(torch.zeros((8, 4), device="cuda", dtype=torch.float16), case.params, [])
    with pytest.raises(qmlp.QmlpError, match="Illegal tensor shape"):
        case.net.inference(torch.zeros((8, 4), device="cuda"), case.params[:-1], [])


# ---------------------------------------------------------------------------- hash grid
GRID_SPECS = [
    dict(n_in=3, n_levels=6, n_features_per_level=2, log2_hashmap_size=10, min_resolution=4, max_resolution=128),
    dict(n_in=2, n_levels=5, n_features_per_level=4, log2_hashmap_size=-1, min_resolution=16, max_resolution=2048),
    dict(n_in=4, n_levels=1, n_features_per_level=8, log2_hashmap_size=-1, min_resolution=6, max_resolution=6),
    dict(n_in=1, n_levels=3, n_features_per_level=1, log2_hashmap_size=4, min_resolution=2, max_resolution=64),
    dict(n_in=3, n_levels=4, n_features_per_level=3, log2_hashmap_size=9, min_resolution=5, max_resolution=70,
         combination_mode="add"),
    dict(n_in=5, n_levels=2, n_features_per_level=2, log2_hashmap_size=8, min_resolution=2, max_resolution=7),
    dict(n_in=6, n_levels=2, n_features_per_level=1, log2_hashmap_size=12, min_resolution=2, max_resolution=5),
    # many features per entry: 32 and 64 lanes share one point in the gradient scatter
    dict(n_in=2, n_levels=2, n_features_per_level=16, log2_hashmap_size=6, min_resolution=3, max_resolution=12),
    dict(n_in=2, n_levels=1, n_features_per_level=32, log2_hashmap_size=-1, min_resolution=5, max_resolution=5),
]


SLICE_GRIDS = [
    # 3-D, 6 levels, dense and hashed (several slices per level only in the large variants below)
    (dict(n_in=3, n_levels=6, n_features_per_level=2, log2_hashmap_size=10, min_resolution=4, max_resolution=128), "half"),
    # hashed levels of 2^16 entries x 2 features = 4 slices each, dense levels of 1, 1 and 3 slices
    (dict(n_in=3, n_levels=7, n_features_per_level=2, log2_hashmap_size=16, min_resolution=8, max_resolution=300), "float"),
    # one dense 4-D level of 20^4 x 8 features: 40 slices, pairs along the last coordinate straddle slice borders
    (dict(n_in=4, n_levels=1, n_features_per_level=8, log2_hashmap_size=-1, min_resolution=20, max_resolution=20), "half"),
    # dense 2-D levels up to 400^2 cells, 3 features (slices of 10 922 entries), levels summed ("add")
    (dict(n_in=2, n_levels=4, n_features_per_level=3, log2_hashmap_size=-1, min_resolution=5, max_resolution=400,
          combination_mode="add"), "float"),
    (dict(n_in=1, n_levels=3, n_features_per_level=1, log2_hashmap_size=4, min_resolution=2, max_resolution=64), "float"),
    (dict(n_in=6, n_levels=2, n_features_per_level=1, log2_hashmap_size=12, min_resolution=2, max_resolution=5), "half"),
    # entries of 6 bytes: a pair of them is loaded at once from an address that is a multiple of 2 only
    (dict(n_in=2, n_levels=3, n_features_per_level=3, log2_hashmap_size=9, min_resolution=4, max_resolution=90), "half"),
]


def _grid_cfg(spec, precision="float", start=0):
    d = spec["n_in"]
    cfg = {"id": "HashGrid", "start_in": start, "combination_mode": "concat",
           "bounding_box_min": [-1.0 + 0.25 * i for i in range(d)],
           "bounding_box_size": [2.0 + 0.5 * i for i in range(d)], "parameter_precision": precision}
    cfg.update(spec)
    return cfg


def _per_point_sets(idx, w):
    """Per point and level the table entries sorted by index, with the weights of equal entries
    (corners that coincide at a clamped border, or that collide in a hashed level) added up."""
    idx = np.asarray(idx).astype(np.int64)
    order = np.argsort(idx, axis=-1, kind="stable")
    idx = np.take_along_axis(idx, order, -1)
    w = np.take_along_axis(np.asarray(w, np.float64), order, -1)
    # running sum of the weights over runs of equal indices, kept at the last entry of each run
    same = np.concatenate([np.zeros(idx.shape[:-1] + (1,), bool), idx[..., 1:] == idx[..., :-1]], -1)
    acc = w.copy()
    for k in range(1, idx.shape[-1]):
        acc[..., k] += np.where(same[..., k], acc[..., k - 1], 0.0)
    last = np.concatenate([idx[..., 1:] != idx[..., :-1], np.ones(idx.shape[:-1] + (1,), bool)], -1)
    return idx, np.where(last, acc, 0.0)


# single dense levels of 4 MB and more: their batches can be sorted by slab, and their gradients summed by columns
COLUMN_GRIDS = [
    ({"n_in": 3, "n_levels": 1, "n_features_per_level": 2, "log2_hashmap_size": -1, "min_resolution": 128, "max_resolution": 128}, "half"),
    ({"n_in": 2, "n_levels": 1, "n_features_per_level": 4, "log2_hashmap_size": -1, "min_resolution": 1000, "max_resolution": 1000}, "float"),
    ({"n_in": 4, "n_levels": 1, "n_features_per_level": 8, "log2_hashmap_size": -1, "min_resolution": 32, "max_resolution": 32}, "half"),
]
COLUMN_GRID_CFGS = [_grid_cfg(s, p) for s, p in COLUMN_GRIDS] + [bc.densegrid4d("half")]


@pytest.mark.parametrize("spec", GRID_SPECS + [bc.hashgrid3d("float"), bc.hashgrid3d("half"), bc.densegrid4d("half")]
                         + [dict(s, parameter_precision=p) for s, p in SLICE_GRIDS[1:4] + SLICE_GRIDS[6:] + COLUMN_GRIDS[:2]])
def test_grid_indices_are_bit_exact(spec):
    """The table entries the device code touches, against the oracle's restatement of the
    reference's index arithmetic (encoding_hashgrid.cuh:17-60,279-287): the index function on its
    own (mode 0, corner by corner in the reference's order), and the entries that the code of the
    fused kernels really uses -- the paired gathers of the forward pass (mode 1: dense pairs
    along the last coordinate, hashed pairs idx / idx^1) and the lane-group gradient scatter of
    the backward pass (mode 2) -- as sets per point and level, bit for bit, with their weights.
    Mode 3, for grids of up to four dimensions: what the gradient records of large batches stand
    for (kernels/grid_gradient.h: the slice of the record's bucket plus the two 16-bit offsets
    as the slice kernel decodes them, and the entries of other slices that the records kernel adds
    itself). Mode 4, for single dense levels whose batches are sorted by slab: the elements behind the sums
    of the column kernel (kernels/grid_gradient_columns.h: the place in the LDS of the owner of the corner's
    node, and back to the table as the kernel writes its sums)."""
    import json
    import qmlp
    cfg = _grid_cfg(spec, spec.get("parameter_precision", "float")) if "id" not in spec else spec
    enc = qmlp.Encoding(json.dumps(cfg))
    f = cfg["n_features_per_level"]
    modes = [0, 1] + ([2] if f & (f - 1) == 0 and f <= 32 else [])
    try:
        enc.hashgrid_corners(None, 3)       # compiles the kernel of mode 3, or says that the grid has no slices
        modes.append(3)
    except qmlp.QmlpError as e:
        # more than four dimensions, or a level of more than 512 slices
        assert "no gradient slices" in str(e) and (cfg["n_in"] > 4 or cfg["max_resolution"] == 2048)
    try:
        enc.hashgrid_corners(None, 4)       # compiles the kernel of mode 4, or says that the grid has no columns
        modes.append(4)
    except qmlp.QmlpError as e:
        # several levels, hashed levels, or a dense level below the 4 MB from which batches are sorted by slab
        assert "no gradient columns" in str(e) and (cfg["n_levels"] > 1 or cfg not in [dict(c) for c in COLUMN_GRID_CFGS])
    if os.environ.get("QMLP_WARM_CACHE"):
        for m in modes:
            enc.hashgrid_corners(None, m)
    require_gpu()
    g = qo.HashGrid(cfg)
    assert [(r, h, o) for (r, h, o, _) in enc.hashgrid_levels()] == [(r, h, o) for (r, h, o, _) in g.level_table()]
    rng = np.random.default_rng(17)
    d = g.dim
    lo = np.array(cfg["bounding_box_min"], np.float32)
    sz = np.array(cfg["bounding_box_size"], np.float32)
    N = 20000
    X = (lo + sz * rng.uniform(-0.05, 1.05, (N, d))).astype(np.float32)   # includes points outside the box
    X[:64] = lo + sz * rng.integers(0, 2, (64, d))                        # and exact box corners
    table = torch.zeros(enc.num_parameters(), device="cuda", dtype=enc.parameter_dtype())
    enc.set_parameter(table)
    x = torch.from_numpy(X).cuda()
    idx, w = enc.hashgrid_corners(x)
    torch.cuda.synchronize()
    ref_idx, ref_w = g.corners(X)
    assert np.array_equal(idx.cpu().numpy().view(np.uint32), ref_idx)
    assert np.allclose(w.cpu().numpy(), ref_w, rtol=1e-5, atol=1e-6)
    want_idx, want_w = _per_point_sets(ref_idx, ref_w)
    assert int(want_idx.max()) + f <= enc.num_parameters()
    for mode in modes[1:]:
        idx, w = enc.hashgrid_corners(x, mode)
        torch.cuda.synchronize()
        got_idx = idx.cpu().numpy().view(np.uint32)
        assert np.isfinite(w.cpu().numpy()).all(), "mode %d left slots unwritten" % mode
        got_idx, got_w = _per_point_sets(got_idx, w.cpu().numpy())
        assert np.array_equal(got_idx, want_idx), "mode %d" % mode
        assert np.allclose(got_w, want_w, rtol=1e-5, atol=1e-6), "mode %d" % mode


@pytest.mark.parametrize("spec", GRID_SPECS)
@pytest.mark.parametrize("precision", ["float", "half"])
def test_standalone_grid_encoding(spec, precision):
    import json
    import qmlp
    cfg = _grid_cfg(spec, precision, start=1)
    require_gpu(cfg)
    enc = qmlp.Encoding(json.dumps(cfg))
    g = qo.HashGrid(cfg)
    rng = np.random.default_rng(3)
    d = g.dim
    N = 3000
    lo = np.array([0.0] + cfg["bounding_box_min"], np.float32)
    sz = np.array([1.0] + cfg["bounding_box_size"], np.float32)
    X = (lo + sz * rng.uniform(0, 1, (N, d + 1))).astype(np.float32)
    table32 = rng.standard_normal(g.n_params).astype(np.float32)
    table_dev = torch.from_numpy(table32).to(enc.parameter_dtype()).cuda()
    table_ref = table_dev.float().cpu().numpy()
    x = torch.from_numpy(X).cuda()
    out = enc.inference_with_parameter(x, table_dev)
    assert_close(out.cpu().numpy(), g.forward(table_ref, X), "grid forward", rel=1e-4, abs_=1e-5)
    adj = rng.standard_normal((N, g.num_outputs)).astype(np.float32)
    ax, gp = enc.adjoint_with_parameter(x, table_dev, torch.from_numpy(adj).cuda())
    ref_ax, ref_gp = g.adjoint(table_ref, X, adj, res_factor=1)
    assert_close(ax.cpu().numpy(), ref_ax, "grid input gradients", rel=1e-3, abs_=1e-3)
    tol = 2e-2 if precision == "half" else 1e-4     # the returned gradient takes the dtype of the parameters
    assert_close(gp.float().cpu().numpy(), ref_gp, "grid parameter gradients", rel=tol, abs_=tol)


@pytest.mark.parametrize("dim", [1, 2])
def test_dense_grid_against_grid_sample(dim):
    """The reference's encoding tests (tests_py/qmlp_tests/test_encoding.py:123-188): a dense
    grid of resolution 2 with 4 features on [-1,1]^D equals torch grid_sample."""
    import json
    import qmlp
    R, C = 2, 4
    cfg = {"id": "HashGrid", "start_in": 0, "n_in": dim, "n_levels": 1, "n_features_per_level": C,
           "log2_hashmap_size": -1, "min_resolution": R, "max_resolution": 16, "combination_mode": "add",
           "bounding_box_min": [-1] * dim, "bounding_box_size": [2] * dim}
    require_gpu(cfg)
    enc = qmlp.FusedEncoding(json.dumps(cfg))
    torch.manual_seed(0)
    params = enc.create_parameter_tensor().requires_grad_(True)
    x = (torch.rand((50, dim), device="cuda") * 2 - 1).requires_grad_(True)
    out = enc(x, params)
    v = torch.randn_like(out)
    (out * v).sum().backward()
    p2 = params.detach().clone().requires_grad_(True)
    x2 = x.detach().clone().requires_grad_(True)
    if dim == 1:
        inp = p2.reshape(1, R, 1, C).permute(0, 3, 2, 1)
        grid = torch.cat([x2.reshape(1, -1, 1, 1), torch.zeros_like(x2).reshape(1, -1, 1, 1)], dim=3)
    else:
        inp = p2.reshape(1, R, R, C).permute(0, 3, 2, 1)
        grid = x2.reshape(1, -1, 1, 2)
    want = torch.nn.functional.grid_sample(inp, grid, mode="bilinear", align_corners=True,
                                           padding_mode="border")[0, :, :, 0].t()
    (want * v).sum().backward()
    assert torch.allclose(out, want, atol=1e-5)
    assert torch.allclose(params.grad, p2.grad, atol=1e-4)
    assert torch.allclose(x.grad, x2.grad, atol=1e-4)


@pytest.mark.parametrize("precision", ["float", "half"])
def test_fused_grid_network_against_oracle(precision):
    """HashGrid + identity -> MLP in one kernel, O(1) table values so that the tolerance bites."""
    spec = dict(n_in=3, n_levels=6, n_features_per_level=2, log2_hashmap_size=10, min_resolution=4,
                max_resolution=128)
    grid = _grid_cfg(spec, precision, start=1)
    cfg = {"num_inputs": 4, "num_outputs": 3, "activation_specification": ["qmlp/builtin-activations.json"],
           "encodings": [grid, {"id": "Identity", "start_in": 0, "n_in": 2}],
           "network": [{"n_out": 32, "bias": True, "activation": "celu"},
                       {"n_out": 3, "bias": False, "activation": "identity"}]}
    case = Case(cfg)
    rng = np.random.default_rng(9)
    case.set_parameters(random_parameters(case.oracle, rng))
    g = case.oracle.encodings[0][1]
    case.set_table(0, rng.uniform(-1, 1, g.n_params))
    N = 5000
    lo = np.array([0.0] + grid["bounding_box_min"], np.float32)
    sz = np.array([1.0] + grid["bounding_box_size"], np.float32)
    X = (lo + sz * rng.uniform(0, 1, (N, 4))).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, 3)) * 0.05).astype(np.float32)
    assert_close(case.gpu_inference(X), case.oracle.forward(X), "inference")
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    got = case.gpu_train(X, adj, flags)
    assert_close(got["out"], case.oracle.forward(X), "forward")
    check_gradients(case, X, adj, flags, got)
    # each flag alone gives the same numbers
    got_e = case.gpu_train(X, adj, FLAG_ENC)
    check_gradients(case, X, adj, FLAG_ENC, got_e, what="alone: ")
    assert got_e["adj_x"] is None and got_e["grads"] is None


def test_network_with_two_grids_against_oracle():
    """Two grid encodings in one network (a 2-D hashed one with 4 features and a small dense 3-D one
    whose gradients are all summed in LDS first) next to an identity encoding."""
    grid_a = _grid_cfg(dict(n_in=2, n_levels=5, n_features_per_level=4, log2_hashmap_size=9, min_resolution=4,
                            max_resolution=96), "half", start=0)
    grid_b = _grid_cfg(dict(n_in=3, n_levels=2, n_features_per_level=2, log2_hashmap_size=-1, min_resolution=5,
                            max_resolution=9), "float", start=2)
    cfg = {"num_inputs": 5, "num_outputs": 2, "activation_specification": ["qmlp/builtin-activations.json"],
           "encodings": [grid_a, grid_b, {"id": "Identity", "start_in": 1, "n_in": 3}],
           "network": [{"n_out": 48, "bias": True, "activation": "sine"},
                       {"n_out": 32, "bias": False, "activation": "celu"},
                       {"n_out": 2, "bias": True, "activation": "identity"}]}
    case = Case(cfg)
    rng = np.random.default_rng(31)
    case.set_parameters(random_parameters(case.oracle, rng))
    for i in (0, 1):
        case.set_table(i, rng.uniform(-1, 1, case.oracle.encodings[i][1].n_params))
    N = 7001
    lo = np.array(grid_a["bounding_box_min"] + grid_b["bounding_box_min"], np.float32)
    sz = np.array(grid_a["bounding_box_size"] + grid_b["bounding_box_size"], np.float32)
    X = (lo + sz * rng.uniform(-0.05, 1.05, (N, 5))).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, 2)) * 0.05).astype(np.float32)
    assert_close(case.gpu_inference(X), case.oracle.forward(X), "inference")
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    got = case.gpu_train(X, adj, flags)
    assert_close(got["out"], case.oracle.forward(X), "forward")
    check_gradients(case, X, adj, flags, got)


@pytest.mark.parametrize("spec,precision", SLICE_GRIDS)
def test_grid_gradients_summed_by_slices_match_the_atomic_scatter_and_the_oracle(spec, precision):
    """options.slice_gradients = 1: the backward kernel stores the adjoint of the encoded rows and one
    workgroup per slice of the gradient table sums the contributions of the whole batch in LDS
    (kernels/grid_gradient.h); 0: the backward kernel scatters with float atomics. Same entries,
    same weights, another order of the fp32 additions; both against the fp32 oracle. The grid
    sits behind an identity encoding (channel offset 2) and reads its coordinates from input
    channel 1 on; the second call adds onto the gradients of the first."""
    d = spec["n_in"]
    grid = _grid_cfg(spec, precision, start=1)
    n_in = d + 1
    base = {"num_inputs": n_in, "num_outputs": 2, "activation_specification": ["qmlp/builtin-activations.json"],
            "encodings": [{"id": "Identity", "start_in": 0, "n_in": 2}, grid],
            "network": [{"n_out": 32, "bias": True, "activation": "celu"},
                        {"n_out": 2, "bias": False, "activation": "identity"}]}
    cases = {}
    # 0: atomics; 1: slices; 2: slices, and the input gradients from a second gather of the table as in mode 0
    # instead of from the position derivatives that the forward pass of mode 1 keeps
    options = {0: {"slice_gradients": 0}, 1: {"slice_gradients": 1}, 2: {"slice_gradients": 1, "input_derivatives": 0}}
    warm_cache(*[dict(base, options=o) for o in options.values()])
    for mode, o in options.items():
        cfg = json.loads(json.dumps(base))
        cfg["options"] = o
        cases[mode] = Case(cfg)
    rng = np.random.default_rng(12)
    params = random_parameters(cases[0].oracle, rng)
    table = rng.uniform(-1, 1, cases[0].oracle.encodings[1][1].n_params)
    for c in cases.values():
        c.set_parameters(params)
        c.set_table(1, table)
    lo = np.array([0.0] + grid["bounding_box_min"], np.float32)
    sz = np.array([1.0] + grid["bounding_box_size"], np.float32)
    # one round of every slice workgroup; many rounds and a ragged last tile; all points in one small
    # region (the records of a level then fall into one or two buckets, which overflow: the rest is added
    # to the gradient tensor by the records kernel itself). The records kernel runs with fewer points per
    # workgroup for batches that would not give every compute unit a workgroup of the largest size: of the sizes
    # 1024 / 512 / 256 / 128 these batches take the last, the third and (140001 points) the second.
    sizes = [(3000, False), (70001, False), (70001, True)] + ([(140001, False)] if d == 3 else [])
    for N, clustered in sizes:
        u = rng.uniform(-0.05, 1.05, (N, n_in)) if not clustered else 0.37 + 2e-3 * rng.uniform(0, 1, (N, n_in))
        X = (lo + sz * u).astype(np.float32)
        adj = (rng.uniform(-1, 1, (N, 2)) * 0.05).astype(np.float32)
        for flags in (FLAG_ENC, FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC):
            got = {mode: c.gpu_train(X, adj, flags) for mode, c in cases.items() if mode < 2 or flags & FLAG_INPUT}
            a, b = got[0]["table_grads"][1], got[1]["table_grads"][1]
            scale = max(1.0, float(np.abs(a).max()))
            assert np.allclose(a / scale, b / scale, rtol=1e-4, atol=2e-6), "N=%d flags=%d: %g" % (N, flags, np.abs(a - b).max())
            if flags & FLAG_WEIGHTS:
                assert np.array_equal(got[0]["grads"], got[1]["grads"]) and np.array_equal(got[0]["grads"], got[2]["grads"])
                # gathered a second time, in the same order of operations: the bits of the atomic path
                assert np.array_equal(got[0]["adj_x"], got[2]["adj_x"])
                # (fixed-point sums, but entries next to a slice boundary and coarse levels also receive float atomics)
                assert np.allclose(got[1]["table_grads"][1] / scale, got[2]["table_grads"][1] / scale, rtol=1e-4, atol=2e-6)
                # from the stored derivatives (kept in the precision of the table: relative 2^-11 each for half)
                sx = float(np.abs(got[0]["adj_x"]).max())
                assert np.allclose(got[1]["adj_x"] / sx, got[0]["adj_x"] / sx, rtol=2e-3, atol=1e-3 if precision == "half" else 1e-5)
                assert np.array_equal(got[1]["out"], got[2]["out"])
            # (weight gradients are those of the other mode bit for bit: checked against the oracle elsewhere)
            check_gradients(cases[1], X, adj, FLAG_ENC, got[1], what="slices, N=%d flags=%d: " % (N, flags))
            if N == 3000 and flags & FLAG_INPUT:
                # the input gradients from the stored derivatives against the fp32 evaluation, at the tolerance of the target
                ref = cases[1].oracle.backward(X, adj, FLAG_INPUT, round_mode=0)
                sx = max(1.0, float(np.abs(ref["adj_x"]).max()))
                assert_close(got[1]["adj_x"] / sx, ref["adj_x"] / sx, "input gradients from stored derivatives vs fp32 oracle")
    # Points several box widths outside are extrapolated with weights far above one (the reference does not clamp the
    # fractional position either; 3 widths outside a level of resolution 128: |w| up to 5e7 in 3-D), while the
    # fixed-point sums of the slice kernel count on weights of at most one: the records kernel adds such records to
    # the gradient tensor itself. The corners of such a point coincide at the border of the grid, so an entry
    # receives huge terms of both signs that cancel to the adjoint itself, and float additions leave rounding noise
    # of the size of |w| x 2^-24 x |adjoint| there in either mode: the entries that these points touch stay at that
    # level, all other entries agree as usual. A NaN coordinate gives NaN weights: the gradients of the entries it
    # touches are NaN in both modes.
    N = 70001
    X = (lo + sz * rng.uniform(0, 1, (N, n_in))).astype(np.float32)
    far = np.arange(7, N, 1000)
    X[far] = (lo + sz * rng.uniform(-3.0, 4.0, (len(far), n_in))).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, 2)) * 0.05).astype(np.float32)
    probe = qmlp.Encoding(json.dumps(grid))
    probe.set_parameter(torch.zeros(probe.num_parameters(), device="cuda", dtype=probe.parameter_dtype()))
    far_idx, far_w = probe.hashgrid_corners(torch.from_numpy(X[far]).cuda())
    touched = np.zeros(probe.num_parameters(), bool)
    for f in range(spec["n_features_per_level"]):
        touched[far_idx.cpu().numpy().astype(np.int64).ravel() + f] = True
    largest = float(far_w.abs().max())
    assert largest > 100
    got = {mode: c.gpu_train(X, adj, FLAG_ENC) for mode, c in cases.items() if mode < 2}
    a, b = got[0]["table_grads"][1], got[1]["table_grads"][1]
    assert np.isfinite(a).all() and np.isfinite(b).all()
    scale = float(np.abs(a[~touched]).max())
    assert scale > 0 and np.allclose(a[~touched] / scale, b[~touched] / scale, rtol=1e-4, atol=2e-5)
    noise = 1.0 + len(far) * largest * 2.0 ** -20          # adjoints of the encoded features are below one
    assert np.abs(a[touched]).max() < noise and np.abs(b[touched]).max() < noise, (np.abs(a[touched]).max(), np.abs(b[touched]).max())
    X = (lo + sz * rng.uniform(0, 1, (N, n_in))).astype(np.float32)
    X[5, 1] = np.nan
    got = {mode: c.gpu_train(X, adj, FLAG_ENC) for mode, c in cases.items() if mode < 2}
    a, b = got[0]["table_grads"][1], got[1]["table_grads"][1]
    assert np.isnan(a).any() and np.array_equal(np.isnan(a), np.isnan(b))
    ok = ~np.isnan(a)
    scale = float(np.abs(a[ok]).max())
    # (with a NaN adjoint in the batch the slice kernel adds floats in LDS: two float sums in different orders)
    assert np.allclose(a[ok] / scale, b[ok] / scale, rtol=1e-4, atol=2e-5)
    X[5, 1] = lo[1]
    # gradients are accumulated: a second call onto the same tensor doubles them
    x, a = torch.from_numpy(X).cuda(), torch.from_numpy(adj).cuda()
    c = cases[1]
    out, tmp = c.net.forward_raw(x, c.params, c.encoding_parameters(), FLAG_ENC)
    _, _, genc = c.net.adjoint_raw(x, a, FLAG_ENC, tmp, c.params, c.encoding_parameters())
    once = genc[1].clone()
    c.net.adjoint_raw(x, a, FLAG_ENC, tmp, c.params, c.encoding_parameters(), grad_encodings=genc)
    torch.cuda.synchronize()
    assert torch.allclose(genc[1], 2 * once, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("features,levels", [(16, 2), (32, 1), (1, 6)])
def test_fused_network_with_wide_and_narrow_grid_entries(features, levels):
    """1, 16 and 32 features per entry in the fused kernels: 2, 32 and 64 lanes share a point
    when the grid gradients are scattered."""
    grid = _grid_cfg(dict(n_in=2, n_levels=levels, n_features_per_level=features, log2_hashmap_size=7,
                          min_resolution=3, max_resolution=3 if levels == 1 else 40), "half", start=0)
    cfg = {"num_inputs": 2, "num_outputs": 2, "activation_specification": ["qmlp/builtin-activations.json"],
           "encodings": [grid],
           "network": [{"n_out": 32, "bias": True, "activation": "celu"},
                       {"n_out": 2, "bias": False, "activation": "identity"}]}
    case = Case(cfg)
    rng = np.random.default_rng(features)
    case.set_parameters(random_parameters(case.oracle, rng))
    case.set_table(0, rng.uniform(-1, 1, case.oracle.encodings[0][1].n_params))
    N = 3001
    lo = np.array(grid["bounding_box_min"], np.float32)
    sz = np.array(grid["bounding_box_size"], np.float32)
    X = (lo + sz * rng.uniform(0, 1, (N, 2))).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, 2)) * 0.05).astype(np.float32)
    assert_close(case.gpu_inference(X), case.oracle.forward(X), "inference")
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    got = case.gpu_train(X, adj, flags)
    check_gradients(case, X, adj, flags, got)


# ---------------------------------------------------------------------------- line integration
def _line_cfg(blending, precision="float", start=0):
    child = {"id": "HashGrid", "start_in": 0, "n_in": 3, "n_levels": 4, "n_features_per_level": 2,
             "log2_hashmap_size": 10, "min_resolution": 4, "max_resolution": 40, "combination_mode": "concat",
             "bounding_box_min": [-1.0, -1.0, -0.5], "bounding_box_size": [2.0, 2.0, 1.0],
             "parameter_precision": precision}
    return {"id": "LineIntegration", "start_in": start, "n_in": 3, "volume": child, "stepsize": 0.13,
            "blending": blending}


def _rays(rng, N, lead=0):
    start = rng.uniform(-2.5, 2.5, (N, 3))
    target = rng.uniform(-0.9, 0.9, (N, 3)) * np.array([1.0, 1.0, 0.5])
    d = target - start
    d /= np.linalg.norm(d, axis=1, keepdims=True)
    X = np.concatenate([rng.uniform(-1, 1, (N, lead)), start, d], 1).astype(np.float32)
    X[0, lead:] = [0.2, -3.0, 0.1, 0.0, 1.0, 0.0]          # zero direction components
    X[1, lead:] = [5.0, 5.0, 5.0, 1.0, 0.0, 0.0]           # misses the box
    X[2, lead:] = [0.1, 0.2, 0.0, 0.6, 0.0, 0.8]           # starts inside
    X[3, lead:] = [0.1, 0.2, 0.0, 0.0, 0.0, 0.0]           # no direction: unbounded interval, no sample
    return X


@pytest.mark.parametrize("blending", ["additive", "average"])
def test_standalone_line_integration(blending):
    """Ray marching through a child grid (tests_cpp/test_hashgrid.cpp:68-150 of the reference only
    prints its results; here the device is compared with the oracle's march)."""
    import json
    import qmlp
    cfg = _line_cfg(blending, start=1)
    require_gpu(cfg)
    enc = qmlp.Encoding(json.dumps(cfg))
    li = qo.LineIntegration(cfg)
    assert enc.num_output_channels() == li.num_outputs == 8 and enc.max_input_channel() == 6
    assert enc.num_parameters() == li.n_params
    rng = np.random.default_rng(21)
    N = 2000
    X = _rays(rng, N, lead=1)
    table = rng.standard_normal(li.n_params).astype(np.float32)
    x, t = torch.from_numpy(X).cuda(), torch.from_numpy(table).cuda()
    out = enc.inference_with_parameter(x, t).cpu().numpy()
    want = li.forward(table, X)
    assert np.all(out[1] == 0) and np.abs(want).max() > 1
    assert_close(out, want, "line integration forward", rel=1e-4, abs_=1e-4)
    adj = rng.standard_normal((N, li.num_outputs)).astype(np.float32)
    ax, gp = enc.adjoint_with_parameter(x, t, torch.from_numpy(adj).cuda())
    ref_ax, ref_gp = li.adjoint(table, X, adj, res_factor=1)
    s = float(np.abs(ref_ax).max())
    assert_close(ax.cpu().numpy() / s, ref_ax / s, "line integration input gradients", rel=1e-3, abs_=1e-4)
    s = float(np.abs(ref_gp).max())
    assert_close(gp.cpu().numpy() / s, ref_gp / s, "line integration table gradients", rel=1e-3, abs_=1e-4)


def test_fused_network_with_line_integration():
    line = _line_cfg("average", "half", start=0)
    cfg = {"num_inputs": 6, "num_outputs": 2, "activation_specification": ["qmlp/builtin-activations.json"],
           "encodings": [line],
           "network": [{"n_out": 32, "bias": True, "activation": "celu"},
                       {"n_out": 2, "bias": False, "activation": "identity"}]}
    case = Case(cfg)
    rng = np.random.default_rng(23)
    case.set_parameters(random_parameters(case.oracle, rng))
    case.set_table(0, rng.uniform(-1, 1, case.oracle.encodings[0][1].n_params))
    N = 3000
    X = _rays(rng, N)
    adj = (rng.uniform(-1, 1, (N, 2)) * 0.05).astype(np.float32)
    assert_close(case.gpu_inference(X), case.oracle.forward(X), "inference")
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    got = case.gpu_train(X, adj, flags)
    assert_close(got["out"], case.oracle.forward(X), "forward")
    check_gradients(case, X, adj, flags, got)


# ---------------------------------------------------------------------------- BASELINE configurations
def _mse_adjoint(out, target):
    return (2.0 * (out - target) / out.size).astype(np.float32)


@pytest.mark.parametrize("cfg_id,N", [(1, 1 << 16), (2, 1 << 14), (4, 1 << 14), (5, 1 << 14)])
def test_baseline_inference(cfg_id, N):
    # O(1) table values: with the published U(+-1e-4) tables every output is below abs 1e-3
    case, rng = baseline_case(cfg_id, table_scale=1.0 if cfg_id in (2, 5) else None)
    X = bc.make_inputs(cfg_id, N, rng)
    ref = case.oracle.forward(X)
    assert (ref != 0).mean() > 0.5, "the comparison would be between zeros"
    assert_close(case.gpu_inference(X), ref, "inference cfg%d" % cfg_id)


@pytest.mark.parametrize("cfg_id", [2, 5])
def test_baseline_inference_published_table_scale(cfg_id):
    """The published table scales (U(+-1e-4), N(0, 0.01)): compare relative to the output scale."""
    case, rng = baseline_case(cfg_id)
    X = bc.make_inputs(cfg_id, 1 << 14, rng)
    ref = case.oracle.forward(X)
    s = max(float(np.abs(ref).max()), 1e-6)
    # ReLU kinks: a few points sit next to a switching unit (see helpers.check_gradients)
    assert_close(case.gpu_inference(X) / s, ref / s, "scaled inference cfg%d" % cfg_id, rel=REL, abs_=2e-3,
                 allowed_fraction=0.02)
    ref1 = case.oracle.forward(X, round_mode=1)
    assert_close(case.gpu_inference(X) / s, ref1 / s, "scaled inference cfg%d vs rounding oracle" % cfg_id,
                 rel=5e-3, abs_=1e-3, allowed_fraction=1e-3)


@pytest.mark.parametrize("cfg_id,N,slices", [(3, 1 << 14, -1), (4, 1 << 13, -1), (5, 1 << 14, -1), (3, 1 << 14, 1), (5, 1 << 14, 1)])
def test_baseline_train_step(cfg_id, N, slices):
    """slices = 1: the grid gradients summed per slice of the table (the path the benchmark's batch sizes take, which
    a batch of this size would not take by itself), so that the table gradients of the 16-level grid meet the oracle
    through the records and slice kernels."""
    case, rng = baseline_case(cfg_id, table_scale=1.0 if cfg_id in (3, 5) else None, options={"slice_gradients": slices})
    X = bc.make_inputs(cfg_id, N, rng)
    target = bc.make_targets(cfg_id, X)
    out_ref = case.oracle.forward(X)
    adj = _mse_adjoint(out_ref, target) * N      # keep the adjoint O(1) per point
    flags = FLAG_INPUT | FLAG_WEIGHTS | (FLAG_ENC if cfg_id in (3, 5) else 0)
    got = case.gpu_train(X, adj, flags)
    assert (out_ref != 0).mean() > 0.5 and np.abs(got["grads"]).max() > 0, "the comparison would be between zeros"
    assert_close(got["out"], out_ref, "forward")
    check_gradients(case, X, adj, flags, got, kinks=cfg_id in (3, 5))
    # weight and input gradients are summed in a fixed order: a second run gives the same bits
    # (the grid gradients are summed with atomics and may differ in the last bits)
    again = case.gpu_train(X, adj, flags)
    assert np.array_equal(again["grads"], got["grads"]) and np.array_equal(again["adj_x"], got["adj_x"])


def test_full_size_properties_cfg2():
    """At the benchmark's full size (2^20 points) the oracle is too slow; check what the
    domain fixes instead: points are independent, so any split or permutation of the batch
    gives bit-identical outputs, and a strided sample agrees with the oracle."""
    case, rng = baseline_case(2)
    N = 1 << 20
    X = bc.make_inputs(2, N, rng)
    x = torch.from_numpy(X).cuda()
    enc = case.encoding_parameters()
    full = case.net.inference(x, case.params, enc)
    halves = torch.cat([case.net.inference(x[:N // 2 + 13], case.params, enc),
                        case.net.inference(x[N // 2 + 13:], case.params, enc)])
    assert torch.equal(full, halves)
    perm = torch.randperm(N, device="cuda")
    assert torch.equal(case.net.inference(x[perm].contiguous(), case.params, enc), full[perm])
    # small batches run kernels of another shape (fewer tiles per wave): same bits per point
    for n in (1000, 1 << 16, 1 << 18):
        assert torch.equal(case.net.inference(x[:n], case.params, enc), full[:n])
    sample = np.arange(0, N, 97)
    ref = case.oracle.forward(X[sample], round_mode=1)
    s = np.abs(ref).max()
    assert_close(full.cpu().numpy()[sample] / s, ref / s, "sampled oracle check", rel=5e-3, abs_=1e-3,
                 allowed_fraction=1e-3)
    # and against the fp32 evaluation itself, at the tolerance of the fp16 path. With the benchmark's tables
    # of U(+-1e-4) the encoded features are subnormal in fp16 (spacing 6e-8, several per cent of a value),
    # so this comparison runs on the same network with tables of U(+-1): same kernels, same indices.
    big, rng1 = baseline_case(2, table_scale=1.0)
    out1 = big.net.inference(x, big.params, big.encoding_parameters()).cpu().numpy()[sample]
    ref0 = big.oracle.forward(X[sample], round_mode=0)
    s1 = np.abs(ref0).max()
    assert_close(out1 / s1, ref0 / s1, "sampled fp32 oracle check", rel=REL, abs_=ABS, allowed_fraction=2e-3)


def test_full_size_properties_cfg3_train():
    """Train step at 2^18 points: gradients are linear in dL/dy, and a sample of points
    matches the oracle's input gradients."""
    case, rng = baseline_case(3, table_scale=1.0)
    N = 1 << 18
    X = bc.make_inputs(3, N, rng)
    adj = rng.uniform(-1, 1, (N, 1)).astype(np.float32)
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    a = case.gpu_train(X, adj, flags)
    b = case.gpu_train(X, 2 * adj, flags)
    for key in ("adj_x", "grads"):
        s = np.abs(a[key]).max()
        assert_close(b[key] / s, 2 * a[key] / s, "linearity of " + key, rel=1e-2, abs_=1e-3)
    ta, tb = a["table_grads"][0], b["table_grads"][0]
    assert_close(tb, 2 * ta, "linearity of grid gradients", rel=1e-2, abs_=1e-3 * np.abs(ta).max())
    sample = np.arange(0, N, 517)
    ref = case.oracle.backward(X[sample], adj[sample], FLAG_INPUT, round_mode=1)
    s = np.abs(ref["adj_x"]).max()
    assert_close(a["adj_x"][sample] / s, ref["adj_x"] / s, "sampled input gradients", rel=5e-3, abs_=1e-3,
                 allowed_fraction=2e-3)
    # the fp32 evaluation: ReLU units that an fp16 rounding switches show up as a few entries in a hundred
    ref0 = case.oracle.backward(X[sample], adj[sample], FLAG_INPUT, round_mode=0)
    assert_close(a["adj_x"][sample] / s, ref0["adj_x"] / s, "sampled input gradients vs fp32", rel=REL, abs_=ABS,
                 allowed_fraction=2e-2)
    # At this size the grid gradients are summed by slices and the input gradients come from the records
    # kernel; the same network with the scatter inside the backward kernel (one atomic per contribution):
    # outputs bit for bit, weight and grid gradients up to the order of the fp32 additions.
    cfg = json.loads(json.dumps(bc.CONFIGS[3]["cfg"]))
    cfg.setdefault("options", {})["slice_gradients"] = 0
    scatter = Case(cfg, bc.ORACLE_ACTIVATIONS)
    scatter.set_parameters(case.params_np)
    scatter.set_table(0, case.tables_np[0])
    c = scatter.gpu_train(X, adj, flags)
    assert np.array_equal(c["out"], a["out"])
    # (the input gradients of the slice path come from the position derivatives that its forward pass kept as halves,
    # those of the scatter path from a second gather: 2^-11 relative per derivative)
    sx = float(np.abs(c["adj_x"]).max())
    assert np.allclose(a["adj_x"] / sx, c["adj_x"] / sx, rtol=2e-3, atol=1e-3)
    # (the backward kernel in front of the slice kernels sums the weight gradients of all layers itself, the one that
    # scatters leaves them to the weight-update kernels: the same products in another order of the fp32 sums)
    scale = float(np.abs(c["grads"]).max())
    assert np.allclose(a["grads"] / scale, c["grads"] / scale, rtol=1e-3, atol=1e-5)
    tc = c["table_grads"][0]
    assert_close(ta, tc, "grid gradients by slices against the atomic scatter", rel=1e-3, abs_=1e-5 * float(np.abs(tc).max()))
    assert float(np.abs(tc).max()) > 0


@pytest.mark.parametrize("cfg_id,N", [(4, 1 << 20), (5, 1 << 21)])
def test_full_size_properties_cfg4_cfg5(cfg_id, N):
    """Configurations 4 and 5 at their benchmark sizes: inference is bit-identical under
    splits and permutations of the batch and matches the oracle on a sample; the gradients
    of a train step are additive over a split of the batch (weight and grid gradients are
    sums over the points) and linear in dL/dy."""
    case, rng = baseline_case(cfg_id, table_scale=1.0 if cfg_id == 5 else None)
    X = bc.make_inputs(cfg_id, N, rng)
    x = torch.from_numpy(X).cuda()
    enc = case.encoding_parameters()
    print("full size cfg%d: inference" % cfg_id, flush=True)
    full = case.net.inference(x, case.params, enc)
    cut = N // 3 + 5
    parts = torch.cat([case.net.inference(x[:cut], case.params, enc), case.net.inference(x[cut:], case.params, enc)])
    assert torch.equal(full, parts)
    perm = torch.randperm(N, device="cuda")
    assert torch.equal(case.net.inference(x[perm].contiguous(), case.params, enc), full[perm])
    sample = np.arange(0, N, 257)
    ref = case.oracle.forward(X[sample], round_mode=1)
    assert (ref != 0).mean() > 0.5, "the comparison would be between zeros"
    s = float(np.abs(ref).max())
    assert_close(full.cpu().numpy()[sample] / s, ref / s, "sampled oracle check", rel=5e-3, abs_=1e-3,
                 allowed_fraction=1e-3 if cfg_id == 5 else 0.0)
    ref0 = case.oracle.forward(X[sample], round_mode=0)
    assert_close(full.cpu().numpy()[sample] / s, ref0 / s, "sampled fp32 oracle check", rel=REL, abs_=ABS,
                 allowed_fraction=2e-3 if cfg_id == 5 else 0.0)

    print("full size cfg%d: train step" % cfg_id, flush=True)
    adj = rng.uniform(-1, 1, (N, case.oracle.n_out)).astype(np.float32)
    flags = FLAG_INPUT | FLAG_WEIGHTS | (FLAG_ENC if cfg_id == 5 else 0)
    whole = case.gpu_train(X, adj, flags)
    first = case.gpu_train(X[:cut], adj[:cut], flags)
    second = case.gpu_train(X[cut:], adj[cut:], flags)
    assert np.array_equal(whole["out"], np.concatenate([first["out"], second["out"]]))
    assert np.array_equal(whole["adj_x"], np.concatenate([first["adj_x"], second["adj_x"]]))
    s = max(float(np.abs(whole["grads"]).max()), 1e-6)
    assert_close((first["grads"] + second["grads"]) / s, whole["grads"] / s, "additivity of the weight gradients",
                 rel=1e-3, abs_=1e-4)
    if cfg_id == 5:
        t = whole["table_grads"][0]
        assert_close(first["table_grads"][0] + second["table_grads"][0], t, "additivity of the grid gradients",
                     rel=1e-3, abs_=1e-4 * np.abs(t).max())
    doubled = case.gpu_train(X, 2 * adj, flags)
    assert_close(doubled["grads"] / s, 2 * whole["grads"] / s, "linearity of the weight gradients", rel=1e-2, abs_=1e-3)
    sample = np.arange(0, N, 1031)
    ref = case.oracle.backward(X[sample], adj[sample], FLAG_INPUT, round_mode=1)
    s = max(float(np.abs(ref["adj_x"]).max()), 1e-6)
    # a few entries in a thousand differ by more: last-bit differences of the half-precision sin / exp
    # intrinsics (cfg4) and ReLU units switching next to zero (cfg5)
    assert_close(whole["adj_x"][sample] / s, ref["adj_x"] / s, "sampled input gradients", rel=5e-3, abs_=1e-3,
                 allowed_fraction=2e-3)
    ref0 = case.oracle.backward(X[sample], adj[sample], FLAG_INPUT, round_mode=0)
    assert_close(whole["adj_x"][sample] / s, ref0["adj_x"] / s, "sampled input gradients vs fp32", rel=REL, abs_=ABS,
                 allowed_fraction=2e-2 if cfg_id == 5 else 2e-3)


def test_batch_with_more_than_2_to_the_31_input_elements():
    """2^28 points of 16 channels: element offsets beyond 32 bits. The points at both ends and
    around the 2^31-element mark give the same bits as in a small batch of their own."""
    case = Case(identity_cfg(16, [16, 1], ["relu", "identity"], [False, False]))
    rng = np.random.default_rng(5)
    case.set_parameters(random_parameters(case.oracle, rng))
    N = 1 << 28
    print("large batch: %d points" % N, flush=True)
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.rand((N, 16), device="cuda", generator=g) * 2 - 1
    out = case.net.inference(x, case.params, [None])
    assert out.shape == (N, 1)
    mark = (1 << 31) // 16
    for start in (0, mark - 500, N - 1000):
        part = x[start:start + 1000].contiguous()
        assert torch.equal(case.net.inference(part, case.params, [None]), out[start:start + 1000])
    sample = x[mark - 64:mark + 64].cpu().numpy()
    assert_close(out[mark - 64:mark + 64].cpu().numpy(), case.oracle.forward(sample), "around the 2^31 mark")
    del x, out
    torch.cuda.empty_cache()


def test_grid_network_batches_that_take_several_launches():
    """Networks that gather are run in launches of at most two steps of the resident workgroups
    (2^20 points for configuration 2). A longer batch has to give the same bits as its parts
    cut anywhere else, and the intermediates of a forward pass in several launches have to
    serve the backward pass: gradients are additive over a split of the batch."""
    case, rng = baseline_case(3, table_scale=1.0)
    N = (1 << 20) + (1 << 19) + 1000
    X = bc.make_inputs(3, N, rng)
    x = torch.from_numpy(X).cuda()
    enc = case.encoding_parameters()
    print("several launches: inference of %d points" % N, flush=True)
    whole = case.net.inference(x, case.params, enc)
    cut = 700001
    parts = torch.cat([case.net.inference(x[:cut], case.params, enc), case.net.inference(x[cut:], case.params, enc)])
    assert torch.equal(whole, parts)
    sample = np.arange(0, N, 4099)
    ref = case.oracle.forward(X[sample], round_mode=1)
    s = float(np.abs(ref).max())
    assert_close(whole.cpu().numpy()[sample] / s, ref / s, "sampled oracle check", rel=5e-3, abs_=1e-3, allowed_fraction=1e-3)

    print("several launches: train step", flush=True)
    adj = rng.uniform(-1, 1, (N, 1)).astype(np.float32)
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    a = case.gpu_train(X, adj, flags)
    b = case.gpu_train(X[:cut], adj[:cut], flags)
    c = case.gpu_train(X[cut:], adj[cut:], flags)
    assert np.array_equal(a["out"], np.concatenate([b["out"], c["out"]]))
    assert np.array_equal(a["adj_x"], np.concatenate([b["adj_x"], c["adj_x"]]))
    s = float(np.abs(a["grads"]).max())
    assert_close((b["grads"] + c["grads"]) / s, a["grads"] / s, "additivity of the weight gradients", rel=1e-3, abs_=1e-4)
    t = a["table_grads"][0]
    assert_close(b["table_grads"][0] + c["table_grads"][0], t, "additivity of the grid gradients", rel=1e-3,
                 abs_=1e-4 * float(np.abs(t).max()))


@pytest.mark.parametrize("precision", ["half", "float"])
def test_rows_staged_in_registers_give_the_same_bits_as_rows_staged_in_lds(precision):
    """A multi-level grid with at most 32 encoded channels gets a kernel shape whose encoded rows
    wait in registers (8 tiles per wavefront). It has to agree bit for bit with the shapes that
    stage in LDS (``register_staging: false``): inference, the forward pass whose intermediates
    feed the backward pass, on one pass and on two passes of the resident workgroups, ragged."""
    c = bc.CONFIGS[3]
    cases = []
    for on in (True, False):
        cfg = json.loads(json.dumps(c["cfg"]))
        cfg.setdefault("options", {})["register_staging"] = on
        cfg["encodings"][0]["parameter_precision"] = precision
        rng = np.random.default_rng(5)
        case = Case(cfg, bc.ORACLE_ACTIVATIONS)
        case.set_parameters(bc.make_parameters(3, rng).astype(np.float32))
        case.set_table(0, bc.make_table(3, case.oracle.encodings[0][1].n_params, rng, 1.0))
        cases.append(case)
    reg, lds = cases
    rng = np.random.default_rng(6)
    for N in ((1 << 20) - 37, (1 << 21) - 64 * 700 - 5):
        print("register staging: %d points" % N, flush=True)
        X = bc.make_inputs(3, N, rng)
        a = reg.gpu_inference(X)
        b = lds.gpu_inference(X)
        assert np.abs(a).max() > 0.1 and np.array_equal(a, b)
    N = (1 << 20) - 37
    adj = rng.uniform(-1, 1, (N, 1)).astype(np.float32)
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    ga, gb = reg.gpu_train(X[:N], adj, flags), lds.gpu_train(X[:N], adj, flags)
    for key in ("out", "adj_x", "grads"):
        assert np.array_equal(ga[key], gb[key]), key
    t = gb["table_grads"][0]
    assert_close(ga["table_grads"][0], t, "grid gradients (atomics)", rel=1e-3, abs_=1e-4 * float(np.abs(t).max()))


def test_inference_sorted_by_grid_slab_gives_the_same_bits_as_the_order_given():
    """A network with a dense grid larger than the L2 evaluates large inference batches slab by
    slab of the grid (``sort_points``; a counting sort in front of the fused kernel). Every
    point is evaluated on its own, so the result has to agree bit for bit with the batch
    evaluated as given: uniform points, ragged sizes, points that all fall into one slab,
    points outside the box and NaN coordinates (slab 0), a batch that grows between calls, and
    a small batch against the CPU oracle."""
    c = bc.CONFIGS[5]
    cases = []
    for mode in (1, 0):
        cfg = json.loads(json.dumps(c["cfg"]))
        cfg.setdefault("options", {})["sort_points"] = mode
        rng = np.random.default_rng(11)
        case = Case(cfg, bc.ORACLE_ACTIVATIONS)
        case.set_parameters(bc.make_parameters(5, rng).astype(np.float32))
        case.set_table(0, bc.make_table(5, case.oracle.encodings[0][1].n_params, rng, 1.0))
        cases.append(case)
    sorted_, plain = cases
    rng = np.random.default_rng(12)
    for N in (1, 63, 8191, 8193, (1 << 18) + 77, (1 << 21) - 5):
        print("sorted by slab: %d points" % N, flush=True)
        X = bc.make_inputs(5, N, rng)
        a, b = sorted_.gpu_inference(X), plain.gpu_inference(X)
        assert np.array_equal(a, b)
        assert N < 64 or np.abs(a).max() > 0.01
    N = 50000
    X = bc.make_inputs(5, N, rng)
    X[:, 0] = 0.5                     # one slab of the leading coordinate
    X[:, 1] = X[:, 1] * 0.01 + 0.3    # one or two of the second
    X[::7, 0] = -3.0                  # outside the box: clamped
    X[::11, 1] = 17.0
    assert np.array_equal(sorted_.gpu_inference(X), plain.gpu_inference(X))
    assert_close(sorted_.gpu_inference(X[:4096]), sorted_.oracle.forward(X[:4096]), "sorted inference against the oracle")
    X[::5, 0] = np.nan
    a, b = sorted_.gpu_inference(X), plain.gpu_inference(X)
    assert np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(a[~np.isnan(a)], b[~np.isnan(b)])
    # strided input rows
    wide = torch.rand((70000, 7), device="cuda")
    view = wide[:, 2:6]
    a = sorted_.net.inference(view, sorted_.params, sorted_.encoding_parameters())
    b = plain.net.inference(view.contiguous(), plain.params, plain.encoding_parameters())
    assert torch.equal(a, b)


@pytest.mark.parametrize("dim,slices", [(3, -1), (2, -1), (3, 1)])
def test_hashed_grid_sorted_on_request_gives_the_same_bits(dim, slices):
    """options.sort_points = 1 on a multi-level hashed grid: the batch is ordered by slabs of the grid's second and
    third coordinate (32 x 32 along a Z curve; 1024 slabs of the second one in 2-D) in front of the fused kernel.
    Inference agrees bit for bit with the batch as given (rows of three floats move as one 12-byte load and store),
    a train step gives the same outputs and input gradients and the same sums for the other gradients (slices = 1:
    with the grid gradients summed per slice of the table, in the sorted order as well)."""
    spec = dict(n_in=dim, n_levels=8, n_features_per_level=2, log2_hashmap_size=12, min_resolution=4, max_resolution=128)
    grid = _grid_cfg(spec, "half")
    nets = []
    for mode in (1, 0):
        cfg = {"num_inputs": dim, "num_outputs": 1, "activation_specification": [bc.BUILTIN], "encodings": [dict(grid)],
               "network": [{"n_out": 32, "bias": False, "activation": "celu"}, {"n_out": 1, "bias": False, "activation": "identity"}],
               "options": {"sort_points": mode, "slice_gradients": slices}}
        rng = np.random.default_rng(3)
        case = Case(cfg)
        case.set_parameters(random_parameters(case.oracle, rng))
        case.set_table(0, rng.uniform(-1, 1, case.oracle.encodings[0][1].n_params))
        nets.append(case)
    sorted_, plain = nets
    lo = np.array(grid["bounding_box_min"], np.float32)
    sz = np.array(grid["bounding_box_size"], np.float32)
    rng = np.random.default_rng(4)
    for N in (1, 777, 8193, (1 << 17) + 5):
        X = (lo + sz * rng.uniform(-0.05, 1.05, (N, dim))).astype(np.float32)
        if N > 100:
            X[::13, 1] = np.nan
            X[5::13, 0] = np.inf
        a, b = sorted_.gpu_inference(X), plain.gpu_inference(X)
        assert np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(a[~np.isnan(a)], b[~np.isnan(b)])
    N = 20000
    rng = np.random.default_rng(4)
    X = (lo + sz * rng.uniform(0, 1, (N, dim))).astype(np.float32)
    assert_close(sorted_.gpu_inference(X), sorted_.oracle.forward(X), "sorted inference against the oracle")
    adj = (rng.uniform(-1, 1, (N, 1)) / 16).astype(np.float32)
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    got, ref = sorted_.gpu_train(X, adj, flags), plain.gpu_train(X, adj, flags)
    assert np.array_equal(got["out"], ref["out"]) and np.array_equal(got["adj_x"], ref["adj_x"])
    oracle = sorted_.oracle.backward(X, adj, flags, round_mode=0)
    for name, a, e in (("input", got["adj_x"], oracle["adj_x"]), ("weight", got["grads"], oracle["grads"]),
                       ("grid", got["table_grads"][0], oracle["table_grads"][0])):
        s_ = max(1.0, float(np.abs(e).max()))
        assert_close(a / s_, e / s_, name + " gradients of the sorted batch vs fp32 oracle")
    scale = np.abs(ref["table_grads"][0]).max()
    assert np.allclose(got["table_grads"][0] / scale, ref["table_grads"][0] / scale, rtol=1e-4, atol=1e-6)
    scale = np.abs(ref["grads"]).max()
    assert np.allclose(got["grads"] / scale, ref["grads"] / scale, rtol=1e-3, atol=1e-5)


@pytest.mark.parametrize("slices", [0, 1])
def test_training_sorted_by_grid_slab_matches_the_order_given(slices):
    """The same network trains its large batches in the sorted order too (``sort_training``): the
    forward pass leaves the sorted rows and the order in its temporary memory, the adjoint pass
    reads dL/dy and writes the input gradients through the order. Outputs and input gradients
    belong to single points and have to agree bit for bit with the pass over the batch as given;
    weight and grid gradients are sums over the batch in another order. Ragged sizes, two batch
    sizes in a row on one network, the scatter with atomics and the slice kernels, and a small
    batch against both oracles."""
    c = bc.CONFIGS[5]
    cases = []
    for sort_training in (True, False):
        cfg = json.loads(json.dumps(c["cfg"]))
        cfg.setdefault("options", {}).update({"sort_points": 1, "sort_training": sort_training, "slice_gradients": slices})
        rng = np.random.default_rng(21)
        case = Case(cfg, bc.ORACLE_ACTIVATIONS)
        case.set_parameters(bc.make_parameters(5, rng).astype(np.float32))
        case.set_table(0, bc.make_table(5, case.oracle.encodings[0][1].n_params, rng, 1.0))
        cases.append(case)
    sorted_, plain = cases
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    assert sorted_.net.forward_memory(1000, flags) > plain.net.forward_memory(1000, flags)
    rng = np.random.default_rng(22)
    for N in ((1 << 17) + 77, 8193, 63):
        print("training sorted by slab: %d points" % N, flush=True)
        X = bc.make_inputs(5, N, rng)
        X[::13, 0] = -2.0                 # outside the box
        adj = rng.uniform(-1, 1, (N, 2)).astype(np.float32)
        a, b = sorted_.gpu_train(X, adj, flags), plain.gpu_train(X, adj, flags)
        assert np.array_equal(a["out"], b["out"])
        assert np.array_equal(a["adj_x"], b["adj_x"])
        s = float(np.abs(b["grads"]).max())
        assert s > 0
        assert_close(a["grads"] / s, b["grads"] / s, "weight gradients", rel=1e-3, abs_=1e-4)
        t = b["table_grads"][0]
        assert_close(a["table_grads"][0], t, "grid gradients", rel=1e-3, abs_=1e-4 * float(np.abs(t).max()))
        # input gradients alone (no adjoint memory at all)
        only = sorted_.gpu_train(X, adj, FLAG_INPUT)
        assert np.array_equal(only["adj_x"], b["adj_x"])
    N = 3000
    X = bc.make_inputs(5, N, rng)
    adj = (rng.uniform(-1, 1, (N, 2)) / N).astype(np.float32)
    check_gradients(sorted_, X, adj, flags, sorted_.gpu_train(X, adj, flags), kinks=True)


@pytest.mark.parametrize("n_in,n_out", [(4, 4), (2, 2), (8, 16), (4, 2), (3, 1)])
def test_rows_moved_as_vectors_and_rows_that_cannot_be(n_in, n_out):
    """Input, output, dL/dy and input-gradient rows whose channels lie side by side move 8 or 16
    bytes at a time; rows that start at an address that is not a multiple of that, or whose
    row stride is not, have to take the scalar path and give the same bits. Both against the
    oracle, ragged batch."""
    case = Case(identity_cfg(n_in, [32, n_out], ["relu", "identity"], [True, True]))
    rng = np.random.default_rng(21)
    case.set_parameters(random_parameters(case.oracle, rng))
    N = 64 * 5 + 13
    X = rng.uniform(-1, 1, (N, n_in)).astype(np.float32)
    adj = rng.uniform(-1, 1, (N, n_out)).astype(np.float32)

    def shifted(a, pad):
        """The same rows in memory that starts 4 bytes off and has `pad` more floats per row."""
        n, c = a.shape
        flat = torch.zeros(1 + n * (c + pad), device="cuda")
        view = flat[1:].view(n, c + pad)[:, :c]
        view.copy_(torch.from_numpy(a))
        return view

    x0 = torch.from_numpy(X).cuda()
    a0 = torch.from_numpy(adj).cuda()
    ref_out = case.oracle.forward(X)
    results = []
    for pad in (None, 0, 1):
        x = x0 if pad is None else shifted(X, pad)
        a = a0 if pad is None else shifted(adj, pad)
        assert (x.data_ptr() % 16 == 0) == (pad is None)
        out = case.net.inference(x, case.params, [])
        out2, tmp = case.net.forward_raw(x, case.params, [], 3)
        adj_in = torch.zeros((N, n_in), device="cuda") if pad is None else shifted(np.zeros((N, n_in), np.float32), pad)
        gnet = torch.zeros((case.net.num_network_parameters(),), device="cuda")
        case.net.adjoint_raw(x, a, 3, tmp, case.params, [], grad_network=gnet, adj_input=adj_in)
        torch.cuda.synchronize()
        results.append((out.cpu().numpy(), out2.cpu().numpy(), adj_in.cpu().numpy().copy(), gnet.cpu().numpy()))
    assert_close(results[0][0], ref_out, "inference")
    check_gradients(case, X, adj, 3, dict(adj_x=results[0][2], grads=results[0][3]), kinks=True)
    for other in results[1:]:
        for k in range(3):
            assert np.array_equal(results[0][k], other[k]), k
        s = float(np.abs(results[0][3]).max())
        assert_close(other[3] / s, results[0][3] / s, "weight gradients", rel=1e-3, abs_=1e-5)


def test_sorted_inference_of_a_two_level_dense_grid_in_several_launches():
    """Two dense 3-D levels (8 and 17 MB) are swept one after the other, so a long batch is cut
    into several launches; sorted by slab, every launch takes its stretch of the sorted rows and
    writes through its stretch of the order. Same bits as the batch evaluated as given, and a
    sample against the oracle."""
    grid = {"id": "HashGrid", "start_in": 0, "n_in": 3, "n_levels": 2, "n_features_per_level": 2,
            "log2_hashmap_size": -1, "min_resolution": 128, "max_resolution": 161, "combination_mode": "concat",
            "bounding_box_min": [-1.0, 0.0, 2.0], "bounding_box_size": [2.0, 1.0, 0.5], "parameter_precision": "half"}
    cases = []
    for mode in (1, 0):
        cfg = {"num_inputs": 3, "num_outputs": 1, "activation_specification": ["qmlp/builtin-activations.json"],
               "encodings": [grid], "options": {"sort_points": mode},
               "network": [{"n_out": 16, "bias": True, "activation": "relu"}, {"n_out": 1, "bias": True, "activation": "identity"}]}
        case = Case(cfg)
        rng = np.random.default_rng(31)
        case.set_parameters(random_parameters(case.oracle, rng))
        case.set_table(0, rng.uniform(-1, 1, case.oracle.encodings[0][1].n_params).astype(np.float32))
        cases.append(case)
    sorted_, plain = cases
    rng = np.random.default_rng(32)
    N = (1 << 21) + (1 << 19) + 333
    X = (rng.uniform(0, 1, (N, 3)) * np.array([2.0, 1.0, 0.5]) + np.array([-1.0, 0.0, 2.0])).astype(np.float32)
    print("sorted, several launches: %d points" % N, flush=True)
    a, b = sorted_.gpu_inference(X), plain.gpu_inference(X)
    assert np.array_equal(a, b) and np.abs(a).max() > 0.05
    sample = np.arange(0, N, 5003)
    ref = sorted_.oracle.forward(X[sample])
    assert_close(a[sample], ref, "sampled oracle check", allowed_fraction=2e-3)


def test_position_derivatives_are_kept_when_input_gradients_are_announced():
    """options.input_derivatives (default: when announced): a training pass whose adjoint flags ask for input and
    grid gradients also keeps, per point and level, the derivatives of the level's features with respect to the
    position, and the adjoint pass forms the grid's share of dL/dinput from them instead of gathering every corner
    a second time. Which of the two ran shows in the bits: the gather repeats the operations of the atomic path
    (bit-identical to it), the stored derivatives are halves (2^-11 relative each)."""
    grid = {"id": "HashGrid", "start_in": 0, "n_in": 3, "n_levels": 8, "n_features_per_level": 2,
            "log2_hashmap_size": 12, "min_resolution": 4, "max_resolution": 256, "combination_mode": "concat",
            "bounding_box_min": [-0.5, 0.0, 0.25], "bounding_box_size": [1.0, 2.0, 0.5], "parameter_precision": "half"}
    base = {"num_inputs": 3, "num_outputs": 2, "activation_specification": ["qmlp/builtin-activations.json"],
            "encodings": [grid],
            "network": [{"n_out": 32, "bias": True, "activation": "celu"}, {"n_out": 2, "bias": False, "activation": "identity"}]}
    options = {"auto": {"slice_gradients": 1}, "never": {"slice_gradients": 1, "input_derivatives": 0},
               "always": {"slice_gradients": 1, "input_derivatives": 1}}
    warm_cache(*[dict(base, options=o) for o in options.values()])
    cases = {k: Case(dict(base, options=o)) for k, o in options.items()}
    rng = np.random.default_rng(31)
    params = random_parameters(cases["auto"].oracle, rng)
    table = rng.uniform(-1, 1, cases["auto"].oracle.encodings[0][1].n_params)
    for c in cases.values():
        c.set_parameters(params)
        c.set_table(0, table)
    N = 5000
    lo, sz = np.array(grid["bounding_box_min"], np.float32), np.array(grid["bounding_box_size"], np.float32)
    X = (lo + sz * rng.uniform(0, 1, (N, 3))).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, 2)) * 0.05).astype(np.float32)
    x, a = torch.from_numpy(X).cuda(), torch.from_numpy(adj).cuda()
    gathered = cases["never"].gpu_train(X, adj, 7)["adj_x"]
    sx = float(np.abs(gathered).max())

    def adjoint(case, tmp, flags=7):
        adj_x, _, _ = case.net.adjoint_raw(x, a, flags, tmp, case.params, case.encoding_parameters())
        torch.cuda.synchronize()
        return adj_x.cpu().numpy()

    def from_derivatives(got):
        assert np.allclose(got / sx, gathered / sx, rtol=2e-3, atol=1e-3)
        return not np.array_equal(got, gathered)

    auto, always = cases["auto"], cases["always"]
    # the same size of forward memory whatever the flags: 16 bytes per point and level behind the intermediates
    assert auto.net.forward_memory(N, 6) == auto.net.forward_memory(N, 7) == cases["never"].net.forward_memory(N, 7) + 8 * 16 * 5056
    # announced with the forward memory: stored and used
    _, tmp7 = auto.net.forward_raw(x, auto.params, auto.encoding_parameters(), 7)
    assert from_derivatives(adjoint(auto, tmp7))
    # a pass that announced no input gradients keeps none; an adjoint pass that asks for them anyway gathers
    _, tmp6 = auto.net.forward_raw(x, auto.params, auto.encoding_parameters(), 6)
    assert not from_derivatives(adjoint(auto, tmp6))
    # ... while the memory of the earlier pass still holds its derivatives
    assert from_derivatives(adjoint(auto, tmp7))
    # the flags of the last adjoint pass count as announced too: forward() of the C ABI alone
    out = torch.empty((N, 2), device="cuda")
    tmp = torch.empty(auto.net.forward_memory(N, 0), dtype=torch.uint8, device="cuda")
    import ctypes
    from qmlp import _lib
    _lib.check(_lib.lib.qmlp_network_forward(auto.net._handle, _lib.desc(x), _lib.desc(out), ctypes.c_void_p(tmp.data_ptr()),
                                              _lib.current_stream(x.device)))
    assert from_derivatives(adjoint(auto, tmp))
    # another batch into the same memory, without derivatives: those of the old batch are not taken for it
    M = 3000
    xs, as_ = x[:M].contiguous(), a[:M].contiguous()
    assert auto.net.forward_memory(M, 6) <= tmp7.numel()
    _lib.check(_lib.lib.qmlp_network_forward(auto.net._handle, _lib.desc(xs), _lib.desc(out[:M]), ctypes.c_void_p(tmp7.data_ptr()),
                                              _lib.current_stream(x.device)))
    small, _, _ = auto.net.adjoint_raw(xs, as_, 7, tmp7, auto.params, auto.encoding_parameters())
    assert np.array_equal(small.cpu().numpy(), cases["never"].gpu_train(X[:M], adj[:M], 7)["adj_x"])
    _, tmp7 = auto.net.forward_raw(x, auto.params, auto.encoding_parameters(), 7)
    # always: also when nothing was announced
    _, tmp6 = always.net.forward_raw(x, always.params, always.encoding_parameters(), 6)
    assert from_derivatives(adjoint(always, tmp6))
    # input gradients alone (no grid gradients: no records kernel) come from the backward kernel's own gathers
    only = adjoint(auto, tmp7, flags=1)
    assert np.array_equal(only, cases["never"].gpu_train(X, adj, 1)["adj_x"])
    # against the fp32 oracle, at the tolerance of the target
    ref = auto.oracle.backward(X, adj, FLAG_INPUT, round_mode=0)
    s = max(1.0, float(np.abs(ref["adj_x"]).max()))
    assert_close(adjoint(auto, tmp7) / s, ref["adj_x"] / s, "input gradients from stored derivatives vs fp32 oracle")


@pytest.mark.parametrize("spec,precision", COLUMN_GRIDS)
def test_grid_gradients_summed_by_columns_match_the_records_the_atomic_scatter_and_the_oracle(spec, precision):
    """A single dense level whose batch trains sorted by grid slab (options.sort_points = 1 here, so that small
    batches sort too): the gradients of the table are summed owner by owner of the grid's nodes in LDS, without
    records (kernels/grid_gradient_columns.h; options.column_gradients = 0: records and slices on the same sorted
    batch; options.slice_gradients = 0, sort_points = 0: float atomics on the batch as given). Same entries, same
    weights, another order of the additions; all against the fp32 oracle. Batches: fewer points than slabs; a
    ragged last tile with points outside the box; all points in one small region (one owner, split into parts);
    far outside points and a NaN coordinate (added with atomics by the workgroup of their slab)."""
    d = spec["n_in"]
    grid = _grid_cfg(spec, precision, start=1)
    n_in = d + 1
    base = {"num_inputs": n_in, "num_outputs": 2, "activation_specification": ["qmlp/builtin-activations.json"],
            "encodings": [{"id": "Identity", "start_in": 0, "n_in": 2}, grid],
            "network": [{"n_out": 32, "bias": True, "activation": "celu"},
                        {"n_out": 2, "bias": False, "activation": "identity"}]}
    options = {"columns": {"sort_points": 1, "slice_gradients": 1},
               "records": {"sort_points": 1, "slice_gradients": 1, "column_gradients": 0},
               "atomics": {"sort_points": 0, "slice_gradients": 0}}
    warm_cache(*[dict(base, options=o) for o in options.values()])
    cases = {k: Case(dict(base, options=o)) for k, o in options.items()}
    rng = np.random.default_rng(23)
    params = random_parameters(cases["columns"].oracle, rng)
    table = rng.uniform(-1, 1, cases["columns"].oracle.encodings[1][1].n_params)
    for c in cases.values():
        c.set_parameters(params)
        c.set_table(1, table)
    lo = np.array([0.0] + grid["bounding_box_min"], np.float32)
    sz = np.array([1.0] + grid["bounding_box_size"], np.float32)
    flags = FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC
    for N, clustered in [(500, False), (70001, False), (70001, True)]:
        # (up to one and a half cells outside the box: weights up to 2.5^D; further out the cancelling terms of the
        # extrapolation leave rounding noise in either mode, see below)
        margin = 1.5 / spec["max_resolution"]
        u = rng.uniform(-margin, 1 + margin, (N, n_in)) if not clustered else 0.37 + 2e-3 * rng.uniform(0, 1, (N, n_in))
        X = (lo + sz * u).astype(np.float32)
        if not clustered:
            X[:16, 1:] = lo[1:] + sz[1:] * rng.integers(0, 2, (16, d))        # exact box corners and borders
        adj = (rng.uniform(-1, 1, (N, 2)) * 0.05).astype(np.float32)
        for f in (FLAG_ENC, flags):
            got = {k: c.gpu_train(X, adj, f) for k, c in cases.items()}
            a, b, c = (got[k]["table_grads"][1] for k in ("columns", "records", "atomics"))
            scale = max(1.0, float(np.abs(c).max()))
            what = "N=%d clustered=%s flags=%d" % (N, clustered, f)
            assert np.allclose(a / scale, c / scale, rtol=1e-4, atol=2e-6), what + ": %g" % np.abs(a - c).max()
            assert np.allclose(a / scale, b / scale, rtol=1e-4, atol=2e-6), what + ": %g" % np.abs(a - b).max()
            assert np.array_equal(got["columns"]["out"], got["atomics"]["out"])
            if f & FLAG_INPUT:
                # the same arithmetic for the input gradients in both sorted modes
                assert np.array_equal(got["columns"]["adj_x"], got["records"]["adj_x"]), what
                # (the order of the points inside a slab differs from sort to sort: another order of the fp32 sums)
                sg = float(np.abs(got["records"]["grads"]).max())
                assert np.allclose(got["columns"]["grads"] / sg, got["records"]["grads"] / sg, rtol=1e-4, atol=1e-6), what
                sx = max(1e-30, float(np.abs(got["atomics"]["adj_x"]).max()))
                assert np.allclose(got["columns"]["adj_x"] / sx, got["atomics"]["adj_x"] / sx, rtol=2e-3, atol=1e-3), what
            check_gradients(cases["columns"], X, adj, FLAG_ENC, got["columns"], what="columns, " + what + ": ")
            if N == 500 and f & FLAG_INPUT:
                ref = cases["columns"].oracle.backward(X, adj, FLAG_INPUT, round_mode=0)
                sx = max(1.0, float(np.abs(ref["adj_x"]).max()))
                assert_close(got["columns"]["adj_x"] / sx, ref["adj_x"] / sx, "input gradients vs fp32 oracle")
    # far outside points (weights far above one) and a NaN coordinate: as in the slice kernels' test
    N = 70001
    X = (lo + sz * rng.uniform(0, 1, (N, n_in))).astype(np.float32)
    far = np.arange(7, N, 1000)
    X[far] = (lo + sz * rng.uniform(-3.0, 4.0, (len(far), n_in))).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, 2)) * 0.05).astype(np.float32)
    probe = qmlp.Encoding(json.dumps(grid))
    probe.set_parameter(torch.zeros(probe.num_parameters(), device="cuda", dtype=probe.parameter_dtype()))
    far_idx, far_w = probe.hashgrid_corners(torch.from_numpy(X[far]).cuda())
    touched = np.zeros(probe.num_parameters(), bool)
    for f in range(spec["n_features_per_level"]):
        touched[far_idx.cpu().numpy().astype(np.int64).ravel() + f] = True
    largest = float(far_w.abs().max())
    assert largest > 100
    got = {k: cases[k].gpu_train(X, adj, FLAG_ENC) for k in ("columns", "atomics")}
    a, b = got["atomics"]["table_grads"][1], got["columns"]["table_grads"][1]
    assert np.isfinite(a).all() and np.isfinite(b).all()
    scale = float(np.abs(a[~touched]).max())
    bad = np.where(~np.isclose(a / scale, b / scale, rtol=1e-4, atol=2e-5) & ~touched)[0]
    assert scale > 0 and len(bad) == 0, (len(bad), bad[:8], a[bad[:8]], b[bad[:8]])
    noise = 1.0 + len(far) * largest * 2.0 ** -20
    assert np.abs(a[touched]).max() < noise and np.abs(b[touched]).max() < noise
    X = (lo + sz * rng.uniform(0, 1, (N, n_in))).astype(np.float32)
    X[5, 1] = np.nan
    got = {k: cases[k].gpu_train(X, adj, FLAG_ENC) for k in ("columns", "atomics")}
    a, b = got["atomics"]["table_grads"][1], got["columns"]["table_grads"][1]
    assert np.isnan(a).any() and np.array_equal(np.isnan(a), np.isnan(b))
    ok = ~np.isnan(a)
    scale = float(np.abs(a[ok]).max())
    assert np.allclose(a[ok] / scale, b[ok] / scale, rtol=1e-4, atol=2e-5)


def test_backward_kernel_from_the_offline_compiler_runs_two_wavefronts_per_simd():
    """Where the installed ROCm has an offline compiler (KernelLoader::CompileOffline), the backward kernel that runs
    the layers again is compiled by it for 256 registers and taken if it does not spill: workgroups of four wavefronts,
    two of them resident per compute unit. Its gradients are checked against the oracle like any other kernel's, and
    bit for bit against the kernels that read stored intermediates (from the run-time compiler of the process)."""
    base = identity_cfg(16, [32, 32, 4], ["sine", "celu", "identity"], [False, True, False])
    off = dict(base, options={"recompute_intermediates": 0})
    warm_cache(base, off)
    offline, _ = qmlp._lib.kernel_compiler_stats()
    if not offline:
        pytest.skip("no offline compiler in this installation (or QMLP_COMPILER=hiprtc)")
    cases = {"on": Case(base), "off": Case(off)}
    rng = np.random.default_rng(43)
    params = random_parameters(cases["on"].oracle, rng)
    for c in cases.values():
        c.set_parameters(params)
    full = FLAG_INPUT | FLAG_WEIGHTS
    res = json.loads(cases["on"].net.generated_source("backward_resources", full))
    assert res["recompute"] is True and res["block"] == 256 and res["scratch_bytes"] <= 64 and res["registers"] <= 256
    assert res["full_grid"] == 2 * torch.cuda.get_device_properties(0).multi_processor_count
    N = 4099
    X = rng.uniform(-1, 1, (N, 16)).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, 4)) / 16).astype(np.float32)
    got = {k: c.gpu_train(X, adj, full) for k, c in cases.items()}
    for key in ("out", "adj_x", "grads"):
        assert np.array_equal(got["on"][key], got["off"][key]), key
    # (against the fp32 oracle at rel 1e-2 / abs 1e-3 of the largest entry; the oracle that rounds where the device
    # rounds is matched by the kernels this one equals bit for bit in the tests of the stored intermediates)
    ref = cases["on"].oracle.backward(X, adj, full, round_mode=0)
    for key in ("adj_x", "grads"):
        scale = max(1.0, float(np.abs(ref[key]).max()))
        assert_close(got["on"][key] / scale, ref[key] / scale, key + " vs fp32 oracle")


@pytest.mark.parametrize("which", ["hashgrid", "identity"])
def test_backward_kernel_that_runs_the_layers_again_gives_the_same_bits(which):
    """options.recompute_intermediates (default: when announced): where the backward kernel sums the weight gradients
    of all layers, the training pass keeps the encoded input only and the backward kernel runs the layers again per
    tile (Layer::forwardKeep: the same operations as the forward kernel, so the same pre-activations bit for bit)
    instead of reading 2 x sum(C_out) bytes per point back. Against the same network with the option off: outputs,
    input and weight gradients bit for bit, grid gradients up to the order of their float atomics. An adjoint pass
    with other flags than announced, whose kernels need the stored intermediates, makes the forward pass run again."""
    if which == "hashgrid":
        grid = {"id": "HashGrid", "start_in": 0, "n_in": 3, "n_levels": 8, "n_features_per_level": 2,
                "log2_hashmap_size": 12, "min_resolution": 4, "max_resolution": 256, "combination_mode": "concat",
                "bounding_box_min": [-0.5, 0.0, 0.25], "bounding_box_size": [1.0, 2.0, 0.5], "parameter_precision": "half"}
        base = {"num_inputs": 3, "num_outputs": 3, "activation_specification": ["qmlp/builtin-activations.json"],
                "encodings": [grid],
                "network": [{"n_out": 64, "bias": True, "activation": "celu"}, {"n_out": 48, "bias": False, "activation": "sine"},
                            {"n_out": 3, "bias": True, "activation": "identity"}]}
        options, n_in = {"slice_gradients": 1}, 3
    else:
        base = identity_cfg(7, [32, 64, 5], ["sine", "celu", "identity"], [True, True, False])
        options, n_in = {}, 7
    on, off = dict(base, options=options), dict(base, options=dict(options, recompute_intermediates=0))
    warm_cache(on, off)
    cases = {"on": Case(on), "off": Case(off)}
    rng = np.random.default_rng(41)
    params = random_parameters(cases["on"].oracle, rng)
    for c in cases.values():
        c.set_parameters(params)
        if which == "hashgrid":
            c.set_table(0, rng.uniform(-1, 1, c.oracle.encodings[0][1].n_params) if c is cases["on"] else cases["on"].tables_np[0])
    N = 5003
    if which == "hashgrid":
        lo, sz = np.array(grid["bounding_box_min"], np.float32), np.array(grid["bounding_box_size"], np.float32)
        X = (lo + sz * rng.uniform(0, 1, (N, 3))).astype(np.float32)
    else:
        X = rng.uniform(-1, 1, (N, n_in)).astype(np.float32)
    adj = (rng.uniform(-1, 1, (N, base["num_outputs"])) / 16).astype(np.float32)
    full = (FLAG_INPUT | FLAG_WEIGHTS | FLAG_ENC) if which == "hashgrid" else (FLAG_INPUT | FLAG_WEIGHTS)
    # the kernel that runs for these flags
    kind = "backward_slices_resources" if which == "hashgrid" else "backward_resources"
    assert json.loads(cases["on"].net.generated_source(kind, full))["recompute"] is True
    assert json.loads(cases["off"].net.generated_source(kind, full))["recompute"] is False
    assert "forwardKeep" in cases["on"].net.generated_source("backward_recompute", full)
    got = {k: c.gpu_train(X, adj, full) for k, c in cases.items()}
    assert np.array_equal(got["on"]["out"], got["off"]["out"])
    assert np.array_equal(got["on"]["adj_x"], got["off"]["adj_x"])
    assert np.array_equal(got["on"]["grads"], got["off"]["grads"])
    if which == "hashgrid":
        a, b = got["on"]["table_grads"][0], got["off"]["table_grads"][0]
        s = float(np.abs(b).max())
        assert np.allclose(a / s, b / s, rtol=1e-4, atol=2e-6)
    check_gradients(cases["on"], X, adj, full, got["on"])
    # announced with all gradients, asked for others: input gradients alone, weight gradients alone, ...
    x, a = torch.from_numpy(X).cuda(), torch.from_numpy(adj).cuda()
    on_case, off_case = cases["on"], cases["off"]
    for flags in ([FLAG_INPUT, FLAG_WEIGHTS, FLAG_INPUT | FLAG_WEIGHTS] + ([FLAG_ENC, FLAG_WEIGHTS | FLAG_ENC] if which == "hashgrid" else [])):
        _, tmp = on_case.net.forward_raw(x, on_case.params, on_case.encoding_parameters(), full)
        adj_x, gnet, genc = on_case.net.adjoint_raw(x, a, flags, tmp, on_case.params, on_case.encoding_parameters())
        want = off_case.gpu_train(X, adj, flags)
        torch.cuda.synchronize()
        if flags & FLAG_INPUT:
            assert np.array_equal(adj_x.cpu().numpy(), want["adj_x"]), flags
        if flags & FLAG_WEIGHTS:
            assert np.array_equal(gnet.cpu().numpy(), want["grads"]), flags
        if flags & FLAG_ENC:
            s = float(np.abs(want["table_grads"][0]).max())
            assert np.allclose(genc[0].cpu().numpy() / s, want["table_grads"][0] / s, rtol=1e-4, atol=2e-6), flags
        # ... and once more with the same memory: whatever ran the first time left it complete
        adj_x2, gnet2, _ = on_case.net.adjoint_raw(x, a, flags, tmp, on_case.params, on_case.encoding_parameters())
        torch.cuda.synchronize()
        if flags & FLAG_INPUT:
            assert np.array_equal(adj_x2.cpu().numpy(), want["adj_x"]), flags
        if flags & FLAG_WEIGHTS:
            assert np.array_equal(gnet2.cpu().numpy(), want["grads"]), flags
