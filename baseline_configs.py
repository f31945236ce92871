"""The five benchmark / parity configurations of the fused encoding + MLP path and their
synthetic data: network specifications in the QuickMLP JSON format, parameter
initialisation, inputs and training targets, all generated on the host from
``numpy.random.default_rng(seed)`` so that the CPU check and the GPU see identical values.
"""
import math

import numpy as np

BUILTIN = "qmlp/builtin-activations.json"

SINE30 = {
    "id": "sine30",
    "forward": "z = hsin(__hmul(__float2half(30.0f), x))",
    "adjoint": "adjx = __hmul(__hmul(__float2half(30.0f), hcos(__hmul(__float2half(30.0f), x))), adjz)",
}


def hashgrid3d(precision="half"):
    return {"id": "HashGrid", "start_in": 0, "n_in": 3, "n_levels": 16, "n_features_per_level": 2,
            "log2_hashmap_size": 19, "min_resolution": 16, "max_resolution": 4096,
            "combination_mode": "concat", "bounding_box_min": [0.0, 0.0, 0.0],
            "bounding_box_size": [1.0, 1.0, 1.0], "parameter_precision": precision}


def densegrid4d(precision="half"):
    return {"id": "HashGrid", "start_in": 0, "n_in": 4, "n_levels": 1, "n_features_per_level": 8,
            "log2_hashmap_size": -1, "min_resolution": 32, "max_resolution": 32,
            "combination_mode": "concat", "bounding_box_min": [0.0] * 4, "bounding_box_size": [1.0] * 4,
            "parameter_precision": precision}


def _layers(widths, acts, biases):
    return [{"n_out": w, "bias": b, "activation": a} for w, a, b in zip(widths, acts, biases)]


CONFIGS = {
    # 1: tiny inference, identity(3) -> 16 relu -> 1 relu, no bias
    1: dict(
        cfg={"num_inputs": 3, "num_outputs": 1, "activation_specification": [BUILTIN],
             "encodings": [{"id": "Identity", "start_in": 0, "n_in": 3}],
             "network": _layers([16, 1], ["relu", "relu"], [False, False])},
        points=1 << 16, input_range=(0.0, 1.0), train=False, fan_in=[3, 16], init="linear",
        flop_per_point=2 * (3 * 16 + 16 * 1), gather_bytes_per_point=0, io_bytes_per_point=16),
    # 2: hash grid (16 levels x 2 fp16 features, 2^19 entries) -> 64 relu -> 64 relu -> 1
    2: dict(
        cfg={"num_inputs": 3, "num_outputs": 1, "activation_specification": [BUILTIN],
             "encodings": [hashgrid3d()],
             "network": _layers([64, 64, 1], ["relu", "relu", "identity"], [False] * 3)},
        points=1 << 20, input_range=(0.0, 1.0), train=False, fan_in=[32, 64, 64], init="linear",
        table=("uniform", 1e-4), flop_per_point=2 * (32 * 64 + 64 * 64 + 64 * 1),
        gather_bytes_per_point=16 * 8 * 2 * 2, io_bytes_per_point=16),
    # 3: full train step on the network of 2
    3: dict(
        cfg={"num_inputs": 3, "num_outputs": 1, "activation_specification": [BUILTIN],
             "encodings": [hashgrid3d()],
             "network": _layers([64, 64, 1], ["relu", "relu", "identity"], [False] * 3)},
        points=1 << 18, input_range=(0.0, 1.0), train=True, fan_in=[32, 64, 64], init="linear",
        table=("uniform", 1e-4), flop_per_point=3 * 2 * (32 * 64 + 64 * 64 + 64 * 1),
        gather_bytes_per_point=16 * 8 * 2 * 2 * 2 + 16 * 8 * 2 * 4, io_bytes_per_point=28),
    # 4: SIREN-style heterogeneous widths with biases
    4: dict(
        cfg={"num_inputs": 4, "num_outputs": 4, "activation_specification": [BUILTIN, SINE30],
             "encodings": [{"id": "Identity", "start_in": 0, "n_in": 4}],
             "network": _layers([128, 64, 48, 4], ["sine30", "sine", "celu", "identity"], [True] * 4)},
        points=1 << 20, input_range=(-1.0, 1.0), train=True, fan_in=[4, 128, 64, 48], init="siren",
        flop_per_point=2 * (4 * 128 + 128 * 64 + 64 * 48 + 48 * 4), gather_bytes_per_point=0,
        io_bytes_per_point=32),
    # 5: dense 4-D grid (32^4 x 8 fp16 features) + identity(4) -> 32 -> 32 -> 32 -> 2, relu, bias
    5: dict(
        cfg={"num_inputs": 4, "num_outputs": 2, "activation_specification": [BUILTIN],
             "encodings": [densegrid4d(), {"id": "Identity", "start_in": 0, "n_in": 4}],
             "network": _layers([32, 32, 32, 2], ["relu"] * 4, [True] * 4)},
        points=1 << 21, input_range=(0.0, 1.0), train=True, fan_in=[12, 32, 32, 32], init="linear",
        table=("normal", 0.01), flop_per_point=2 * (12 * 32 + 32 * 32 + 32 * 32 + 32 * 2),
        gather_bytes_per_point=16 * 8 * 2, io_bytes_per_point=24),
}

ORACLE_ACTIVATIONS = {"sine30": (4, 30.0)}   # (qo act id "sin(param*x)", param)


def padded_layout(cfg):
    """[(cin_padded, cout_padded, bias, w_start, b_start)] and the parameter count, following the
    flat layout: all weight matrices (row-major (C_out, C_in)), then the biases."""
    encoded = 0
    for e in cfg["encodings"]:
        if e["id"] == "Identity":
            encoded += e["n_in"]
        else:
            encoded += e["n_features_per_level"] * (e["n_levels"] if e["combination_mode"] != "add" else 1)
    up = lambda v: (v + 15) // 16 * 16
    widths = [encoded] + [l["n_out"] for l in cfg["network"]]
    layers = []
    n = 0
    for i, l in enumerate(cfg["network"]):
        layers.append([up(widths[i]), up(widths[i + 1]), bool(l["bias"]), n, 0])
        n += up(widths[i]) * up(widths[i + 1])
    for layer in layers:
        if layer[2]:
            layer[4] = n
            n += layer[1]
    return [tuple(l) for l in layers], n


# Seed of numpy's default_rng for the parameters of each configuration. Configuration 5 ends in
# a ReLU with bias: with most seeds (0 among them) one or both of its outputs are negative
# before that ReLU for every point, so the output and all gradients are exactly zero; seed 9
# keeps both outputs alive.
PARAMETER_SEED = {1: 0, 2: 0, 3: 0, 4: 0, 5: 9}


def make_parameters(cfg_id, rng):
    """fp16 network parameters in the flat padded layout: U(+-1/sqrt(fan_in)) ("linear") or
    U(+-sqrt(6/fan_in)/30) ("siren") on the real entries, zeros on the padding."""
    c = CONFIGS[cfg_id]
    cfg = c["cfg"]
    layers, n = padded_layout(cfg)
    flat = np.zeros(n, dtype=np.float32)
    real_in = c["fan_in"]
    for i, (cin, cout, bias, ws, bs) in enumerate(layers):
        fan_in = real_in[i]
        real_out = cfg["network"][i]["n_out"]
        bound = 1.0 / math.sqrt(fan_in) if c["init"] == "linear" else math.sqrt(6.0 / fan_in) / 30.0
        W = np.zeros((cout, cin), dtype=np.float32)
        W[:real_out, :fan_in] = rng.uniform(-bound, bound, (real_out, fan_in))
        flat[ws:ws + cin * cout] = W.reshape(-1)
        if bias:
            b = np.zeros(cout, dtype=np.float32)
            b[:real_out] = rng.uniform(-bound, bound, real_out)
            flat[bs:bs + cout] = b
    return flat.astype(np.float16)


def make_table(cfg_id, n_params, rng, scale=None):
    """Grid table values (returned as float32; cast to the storage precision by the caller)."""
    kind, s = CONFIGS[cfg_id]["table"]
    if scale is not None:
        s = scale
    if kind == "uniform":
        return rng.uniform(-s, s, n_params).astype(np.float32)
    return (rng.standard_normal(n_params) * s).astype(np.float32)


def make_inputs(cfg_id, n, rng):
    lo, hi = CONFIGS[cfg_id]["input_range"]
    return rng.uniform(lo, hi, (n, CONFIGS[cfg_id]["cfg"]["num_inputs"])).astype(np.float32)


def make_targets(cfg_id, x):
    """Regression target sin(4 pi x) cos(4 pi y) z, repeated over the output channels."""
    t = np.sin(4 * np.pi * x[:, 0]) * np.cos(4 * np.pi * x[:, 1]) * x[:, 2]
    return np.repeat(t[:, None], CONFIGS[cfg_id]["cfg"]["num_outputs"], axis=1).astype(np.float32)
