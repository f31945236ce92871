"""CPU-only tests of the host side: the C ABI library loads and exports what the headers
declare, the specification layer follows the reference's rules (validated against the
oracle's restatement and the golden level table), and the code generator's output compiles
for gfx950 through hipRTC without a GPU."""
import ctypes
import json
import os
import re
import subprocess
import sys

import numpy as np
import pytest
import torch

import qmlp
import qmlp_oracle as qo
import baseline_configs as bc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qmlp_[a-z0-9_]+)\s*\(", text)))


@pytest.mark.parametrize("header", ["qmlp_hip.h", "qmlp_capi.h"])
def test_library_exports_every_declared_symbol(header):
    lib = ctypes.CDLL(qmlp._lib.LIB_PATH)
    names = _declared_functions(header)
    assert len(names) > 20
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_static_queries_without_gpu():
    assert qmlp.Network.MatrixSize() == 16
    assert qmlp.Network.WarpSize() == 64
    assert qmlp.Network.MaxSharedMemoryBytes() >= 64 * 1024
    assert qmlp.QuickMLP.is_compile_debug_mode() is False


@pytest.mark.parametrize("cfg_id", [1, 2, 3, 4, 5])
def test_parameter_layout_matches_the_oracle(cfg_id):
    cfg = bc.CONFIGS[cfg_id]["cfg"]
    net = qmlp.Network(json.dumps(cfg))
    onet = qo.Network(cfg, bc.ORACLE_ACTIVATIONS)
    assert net.num_network_parameters() == onet.num_parameters
    assert net.channels_in() == cfg["num_inputs"] and net.channels_out() == cfg["num_outputs"]
    assert net.num_layers() == len(cfg["network"])
    layers, n = bc.padded_layout(cfg)
    assert n == onet.num_parameters
    import torch
    flat = torch.zeros(n, dtype=torch.float16)
    for i, l in enumerate(onet.layers):
        w = net.parameter_view(i, False, flat)
        assert tuple(w.shape) == (l["cout"], l["cin"]) and w.stride() == (l["cin"], 1)
        assert (w.data_ptr() - flat.data_ptr()) // 2 == l["w_start"]
        b = net.parameter_view(i, True, flat)
        if l["bias"]:
            assert tuple(b.shape) == (l["cout"],)
            assert (b.data_ptr() - flat.data_ptr()) // 2 == l["b_start"]
        else:
            assert b is None
    assert {1: 512, 2: 7168, 3: 7168, 4: 14336, 5: 3184}[cfg_id] == n


def test_level_table_matches_golden_and_oracle():
    gold = json.load(open(os.path.join(GOLDEN, "cfg2_level_table.json")))
    enc = qmlp.Encoding(json.dumps(gold["spec"]))
    got = [[r, int(h), off] for (r, h, off, _) in enc.hashgrid_levels()]
    assert got == gold["levels"]
    assert enc.num_parameters() == gold["total_parameters"]
    for spec in [bc.densegrid4d("float"),
                 dict(bc.hashgrid3d("float"), n_in=2, bounding_box_min=[0, 0], bounding_box_size=[1, 1],
                      n_levels=5, n_features_per_level=4, log2_hashmap_size=-1, max_resolution=2048),
                 dict(bc.hashgrid3d("float"), n_levels=7, log2_hashmap_size=12, min_resolution=3, max_resolution=300)]:
        e = qmlp.Encoding(json.dumps(spec))
        g = qo.HashGrid(spec)
        assert e.hashgrid_levels() == g.level_table()
        assert e.num_parameters() == g.n_params
        assert e.num_output_channels() == g.num_outputs


def test_encoding_json_round_trip_and_defaults():
    spec = {"id": "HashGrid", "start_in": 1, "n_in": 2, "n_levels": 2, "n_features_per_level": 4,
            "log2_hashmap_size": 8, "min_resolution": 4, "max_resolution": 64, "combination_mode": "add"}
    e = qmlp.Encoding(json.dumps(spec))
    j = json.loads(e.to_json())
    assert j["bounding_box_min"] == [-0.5, -0.5] and j["bounding_box_size"] == [1.0, 1.0]
    assert j["combination_mode"] == "add" and j["parameter_precision"] == "float"
    assert e.max_input_channel() == 2 and e.num_output_channels() == 4 and e.has_parameters()
    e2 = qmlp.Encoding(e.to_json())
    assert json.loads(e2.to_json()) == j
    cat = qmlp.Encoding(json.dumps(dict(spec, combination_mode="cat")))
    assert cat.num_output_channels() == 8
    ident = qmlp.Encoding('{"id": "Identity", "start_in": 2, "n_in": 3}')
    assert ident.max_input_channel() == 4 and ident.num_output_channels() == 3 and not ident.has_parameters()


BASE = bc.CONFIGS[1]["cfg"]


@pytest.mark.parametrize("mutate,code,message", [
    (lambda c: c.update(num_outputs=2), 1, "does not match the number of outputs"),
    (lambda c: c.update(network=[]), 1, "Empty network"),
    (lambda c: c["encodings"][0].update(id="Fourier"), 1, "No encoding with id 'Fourier'"),
    (lambda c: c["encodings"][0].update(n_in=4), 1, "out of bounds"),
    (lambda c: c["network"][0].update(activation="gelu"), 1, "No activation with id 'gelu'"),
    (lambda c: c["network"][0].update(activation=["relu"] * 3), 1, "must match the number of output channels"),
    (lambda c: c["network"][0].update(activation=["relu"] * 15 + [3]), 1, "must be specified as a string"),
    (lambda c: c.pop("num_inputs"), 1, "num_inputs"),
    (lambda c: c.update(activation_specification=["does-not-exist.json"]), 1, "could not be resolved"),
    (lambda c: c.update(activation_specification=[{"id": "1bad", "forward": "z=x", "adjoint": "adjx=adjz"}]), 1,
     "not a valid C.. identifier"),
])
def test_specification_errors(mutate, code, message):
    cfg = json.loads(json.dumps(BASE))
    mutate(cfg)
    with pytest.raises(qmlp.QmlpError, match=message) as ei:
        qmlp.Network(json.dumps(cfg))
    assert ei.value.code == code


def test_malformed_json_and_grid_errors():
    with pytest.raises(qmlp.QmlpError, match="JSON parse error"):
        qmlp.Network('{"num_inputs": 3,')
    bad = dict(bc.hashgrid3d("float"), n_in=7, bounding_box_min=[0] * 7, bounding_box_size=[1] * 7)
    with pytest.raises(qmlp.QmlpError, match=r"to be in \[1,6\]"):
        qmlp.Encoding(json.dumps(bad))
    with pytest.raises(qmlp.QmlpError, match="combination_mode"):
        qmlp.Encoding(json.dumps(dict(bc.hashgrid3d("float"), combination_mode="multiply")))
    with pytest.raises(qmlp.QmlpError, match="Unknown log level"):
        qmlp.set_log_level("chatty")


def test_temporary_memory_of_a_batch_that_trains_in_sorted_order():
    """A network with a dense grid beyond the L2 trains its large batches sorted by grid slab: the forward
    memory also holds the sorted rows, the order, the 1024 slab totals of the sort and every point's place in
    the sorted order, the adjoint memory the rows of the input gradients in that order (256-byte aligned, behind
    everything else; dL/dy is read through the order)."""
    up = lambda v: -(-v // 256) * 256
    cfg = json.loads(json.dumps(bc.CONFIGS[5]["cfg"]))
    cfg.setdefault("options", {})["sort_training"] = False
    given = qmlp.Network(json.dumps(cfg))
    net = qmlp.Network(json.dumps(bc.CONFIGS[5]["cfg"]))
    n = 1 << 21
    assert net.forward_memory(n, 7) == up(given.forward_memory(n, 7)) + up(n * (4 + 1) * 4) + 1024 * 4 + up(n * 4)
    assert net.adjoint_memory(n, 7) == up(given.adjoint_memory(n, 7)) + up(n * 4 * 4)
    assert net.adjoint_memory(n, 6) == given.adjoint_memory(n, 6)
    assert given.adjoint_memory(n, 1) == 0 and net.adjoint_memory(n, 1) == up(n * 4 * 4)
    # below the batch size from which inference sorts, nothing changes
    for m in (1, 1000, (1 << 19) - 1):
        assert net.forward_memory(m, 7) == given.forward_memory(m, 7)
        assert net.adjoint_memory(m, 7) == given.adjoint_memory(m, 7)
    # a hashed grid never sorts (behind its intermediates: 16 bytes per point and level for the derivatives of
    # the level's 2 features with respect to the 3 coordinates)
    hashed = qmlp.Network(json.dumps(bc.CONFIGS[3]["cfg"]))
    assert hashed.forward_memory(n, 7) == (2 * (32 + 64 + 64 + 16) + 16 * 16) * n


def test_temporary_memory_sizes():
    net = qmlp.Network(json.dumps(bc.CONFIGS[3]["cfg"]))
    # intermediates; position derivatives of the grid (3 x 2 halves in one chunk of 16 bytes per level), whatever
    # the flags: a caller may size the memory once for several kinds of passes
    per_fwd = 2 * (32 + 64 + 64 + 16) + 16 * 16
    per_adj = 2 * (64 + 64 + 16)
    plain = json.loads(json.dumps(bc.CONFIGS[3]["cfg"]))
    plain["options"] = {"input_derivatives": 0}
    plain = qmlp.Network(json.dumps(plain))
    assert plain.forward_memory(1 << 18, 7) == 2 * (32 + 64 + 64 + 16) << 18
    assert net.forward_memory(1 << 18, 2) == net.forward_memory(1 << 18, 7)
    # behind the adjoint pre-activations: fp32 partial weight gradients of up to 512 batch
    # slices (one workgroup of 4 wavefronts = 4 tiles each)
    n_params = net.num_network_parameters()
    for n, padded, slices in ((1, 64, 1), (64, 64, 1), (65, 128, 1), (1000, 1024, 4), (1 << 18, 1 << 18, 512)):
        assert net.forward_memory(n, 7) == per_fwd * padded
        # weight gradients alone: the backward kernel sums the tiles of all three layers itself (28 tiles in the
        # accumulation registers of one wavefront per SIMD) and stores no adjoints
        assert net.adjoint_memory(n, 2) == slices * n_params * 4
        # a backward kernel that gathers from the grid for the input gradients has no registers for that
        assert net.adjoint_memory(n, 3) == per_adj * padded + slices * n_params * 4
        assert net.adjoint_memory(n, 1) == 0
        if n < (1 << 15):
            # small batches scatter their grid gradients with atomics and need nothing for it
            assert net.adjoint_memory(n, 7) == per_adj * padded + slices * n_params * 4
            assert net.adjoint_memory(n, 5) == 0
    # From 2^15 points on (a grid of 16 levels; from 2^16 for grids of fewer than 8 levels) the grid gradients are
    # summed slice by slice: the adjoint of the encoded rows
    # (32 halves per point) joins the adjoint pre-activations, and behind everything else come the
    # bucket cursors and the records (4 words each; per level, slices x (1.25 x share + 2048) of them:
    # the table of a level holds 8192 .. 1 048 576 floats, a slice 8192).
    n = 1 << 18
    floats = [8192, 24334, 71874, 221184, 686000] + [1 << 20] * 11
    slices_per_level = [-(-f // 8192) for f in floats]
    records = sum(s * (((5 * n * 4 // 4) // s + 2048) & ~3) for s in slices_per_level)
    cursors = -(-(sum(slices_per_level) + 1) * 4 // 256) * 256
    base = 2 * 32 * n + 512 * n_params * 4       # (all weight gradients are summed in the backward kernel)
    assert net.adjoint_memory(n, 7) == -(-base // 256) * 256 + cursors + -(-records * 16 // 256) * 256
    assert net.adjoint_memory(n, 4) == 2 * 32 * n + cursors + -(-records * 16 // 256) * 256
    assert net.adjoint_memory((1 << 15) - 64, 5) == 0 and net.adjoint_memory(1 << 15, 5) > 0
    few_levels = qmlp.Network(json.dumps(bc.CONFIGS[5]["cfg"]))
    assert few_levels.adjoint_memory((1 << 16) - 64, 4) == 0 and few_levels.adjoint_memory(1 << 16, 4) > 0
    with pytest.raises(qmlp.QmlpError, match="At least one derivative"):
        net.adjoint_memory(10, 0)


def test_temporary_memory_of_networks_whose_backward_kernel_sums_the_weight_gradients():
    """Layers whose gradient tiles the backward kernel keeps in registers (options.fused_weight_update) store no
    adjoint pre-activations: none at all if that holds for every layer, else the layout of all layers stays."""
    def net(widths, mode):
        cfg = {"num_inputs": 16, "num_outputs": widths[-1], "activation_specification": [bc.BUILTIN],
               "encodings": [{"id": "Identity", "start_in": 0, "n_in": 16}],
               "network": [{"n_out": w, "bias": True, "activation": "relu"} for w in widths],
               "options": {"fused_weight_update": mode}}
        return qmlp.Network(json.dumps(cfg))
    n = 4096
    slices = 4096 // 64 // 4
    small = [32, 32, 16]            # gradient tiles, one more each for the bias sums: 2 + 1, 4 + 1, 2 + 1 = 11
    params = net(small, 0).num_network_parameters()
    assert net(small, 0).adjoint_memory(n, 3) == 2 * (32 + 32 + 16) * n + slices * params * 4
    assert net(small, -1).adjoint_memory(n, 3) == slices * params * 4
    assert "::template weightGradient<" not in net(small, 0).generated_source("backward", 3)
    assert net(small, -1).generated_source("backward", 3).count("::template weightGradient<") == 3
    # 4 + 1, 16 + 1, 4 + 1 = 27 tiles: more than the 16 that fit beside two wavefronts per SIMD, so the kernel runs
    # one wavefront per SIMD with 512 registers and sums all of them
    mixed = [64, 64, 16]
    params = net(mixed, 0).num_network_parameters()
    src = net(mixed, -1).generated_source("backward", 3)
    assert src.count("::template weightGradient<") == 3 and "amdgpu_waves_per_eu(1, 1)" in src
    assert net(mixed, -1).adjoint_memory(n, 3) == slices * params * 4
    assert "amdgpu_waves_per_eu(1, 1)" not in net(small, -1).generated_source("backward", 3)
    assert net(mixed, 1).generated_source("backward", 3).count("::template weightGradient<") == 3   # 27 tiles <= 32
    assert "amdgpu_waves_per_eu(1, 1)" not in net(mixed, 1).generated_source("backward", 3)
    assert net(mixed, 1).adjoint_memory(n, 3) == slices * params * 4
    # 61 tiles, and weights that call for workgroups of 8 wavefronts (128 registers each): nothing is summed in the kernel
    deep = net([64, 64, 64, 64, 16], -1).generated_source("backward", 3)
    assert "amdgpu_waves_per_eu(1, 1)" not in deep and "::template weightGradient<" not in deep
    # without weight gradients nothing changes
    assert "::template weightGradient<" not in net(small, -1).generated_source("backward", 1)


def test_generated_source_is_specialised():
    net = qmlp.Network(json.dumps(bc.CONFIGS[2]["cfg"]))
    src = net.generated_source("forward")
    assert "Layer<32, 64, false, activations::relu>" in src
    assert "Layer<64, 16, false, activations::identity>" in src
    assert "static constexpr int resolution[16] = {16, 23, 33, 48, 70, 101, 147, 212, 307, 445, 645, 933, 1351, 1955, 2830, 4095};" in src
    assert "typedef f16 table_t;" in src and not re.search(r"\$\$[A-Z_]+\$\$", src)
    bsrc = net.generated_source("backward", 7)
    assert "stageAdjoint" in bsrc and not re.search(r"\$\$[A-Z_]+\$\$", bsrc)
    wsrc = net.generated_source("weight_update")
    assert "WeightUpdateKernel" in wsrc and not re.search(r"\$\$[A-Z_]+\$\$", wsrc)


def test_kernels_compile_for_gfx950_without_a_gpu_and_are_cached(tmp_path):
    """hipRTC needs no device: generate + compile every kernel of a small fused network, then
    a second network object finds all of them in the disk cache."""
    cache = str(tmp_path / "cache")
    qmlp.set_kernel_cache_dir(cache)
    try:
        grid = dict(bc.hashgrid3d("half"), n_levels=3, log2_hashmap_size=8, max_resolution=64)
        cfg = {"num_inputs": 4, "num_outputs": 3, "activation_specification": [bc.BUILTIN, bc.SINE30],
               "encodings": [grid, {"id": "Identity", "start_in": 3, "n_in": 1}],
               "network": [{"n_out": 48, "bias": True, "activation": "sine30"},
                           {"n_out": 3, "bias": False, "activation": "celu"}]}
        c0, h0 = qmlp._lib.kernel_cache_stats()
        offline, o0 = qmlp._lib.kernel_compiler_stats()
        qmlp.Network(json.dumps(cfg)).precompile(7)
        c1, h1 = qmlp._lib.kernel_cache_stats()
        o1 = qmlp._lib.kernel_compiler_stats()[1]
        # inference and forward in four shapes (4x2, 4x1, 8x4 and 8x8 wavefronts x tiles, the last
        # with its encoded rows in registers), backward with the atomic scatter and backward for the
        # gradient slices, the records kernel of the grid for workgroups of 1024, 512, 256 and 128 points and
        # its slice kernel, 2 weight updates + reduce; for training passes that keep the position derivatives of
        # the grid: forward in the four shapes once more, and the four records kernels that read them; for training
        # passes that keep the encoded input only: the backward kernel that runs the layers again (this network has
        # one behind the slice kernels), and forward in the four shapes with and without the position derivatives;
        # where the installed ROCm has an offline compiler, it compiles that backward kernel, once for two wavefronts per
        # SIMD and once for one (a pass that only fills the cache cannot tell which of the two will be used)
        expected = 35 + (1 if offline else 0)
        assert c1 - c0 == expected and h1 == h0 and o1 - o0 == (2 if offline else 0)
        files = os.listdir(cache)
        assert len(files) == expected and all(f.endswith(".co") for f in files)
        qmlp.Network(json.dumps(cfg)).precompile(7)
        c2, h2 = qmlp._lib.kernel_cache_stats()
        assert c2 == c1                            # nothing recompiled (memory or disk cache)
    finally:
        qmlp.set_kernel_cache_dir(os.environ.get("QMLP_CACHE_DIR", qmlp._lib.DEFAULT_CACHE_DIR))


def test_offline_compiler_can_be_switched_off_and_a_failing_one_falls_back(tmp_path):
    """QMLP_COMPILER=hiprtc keeps every kernel with the run-time compiler of the process; an installed ROCm whose
    hipcc fails (here: a script that exits with an error) costs a warning, and the run-time compiler takes the kernel."""
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = {"num_inputs": 16, "num_outputs": 4, "activation_specification": [bc.BUILTIN],
           "encodings": [{"id": "Identity", "start_in": 0, "n_in": 16}],
           "network": [{"n_out": 16, "bias": False, "activation": "relu"}, {"n_out": 4, "bias": False, "activation": "identity"}]}
    script = ("import sys, json; sys.path[:0] = [%r, %r]; import qmlp; qmlp.set_log_level('off');"
              "net = qmlp.Network(%r); net.precompile(3); print(json.dumps([qmlp._lib.kernel_compiler_stats(), qmlp._lib.kernel_cache_stats()]))"
              % (repo, os.path.join(repo, "quick-mlp_amd"), json.dumps(cfg)))

    def run(env):
        out = subprocess.run([sys.executable, "-c", script], env=dict(os.environ, **env), capture_output=True, text=True, timeout=600)
        assert out.returncode == 0, out.stderr[-2000:]
        return json.loads(out.stdout.strip().splitlines()[-1])

    (offline, count), (compiled, _) = run({"QMLP_COMPILER": "hiprtc", "QMLP_CACHE_DIR": str(tmp_path / "a")})
    assert offline is False and count == 0 and compiled > 0
    # a ROCm directory with the real headers and version file but a hipcc that fails
    fake = tmp_path / "rocm"
    (fake / "bin").mkdir(parents=True)
    (fake / ".info").mkdir()
    (fake / ".info" / "version").write_text("0.0.0-test\n")
    (fake / "bin" / "hipcc").write_text("#!/bin/sh\necho no compiler here >&2\nexit 3\n")
    os.chmod(fake / "bin" / "hipcc", 0o755)
    real = os.environ.get("ROCM_PATH") or "/opt/rocm"
    os.symlink(os.path.join(real, "include"), fake / "include")
    (offline, count), (compiled_with_fallback, _) = run({"ROCM_PATH": str(fake), "QMLP_CACHE_DIR": str(tmp_path / "b")})
    assert offline is True and count == 0
    assert compiled_with_fallback >= compiled      # every kernel was compiled all the same


def test_compile_errors_carry_the_compiler_log(tmp_path):
    qmlp.set_kernel_cache_dir("")
    try:
        cfg = json.loads(json.dumps(BASE))
        cfg["activation_specification"] = [bc.BUILTIN, {"id": "broken", "forward": "z = not_a_function(x)", "adjoint": "adjx = adjz"}]
        cfg["network"][0]["activation"] = "broken"
        net = qmlp.Network(json.dumps(cfg))
        qmlp.set_log_level("off")
        with pytest.raises(qmlp.QmlpError, match="not_a_function") as ei:
            net.precompile(0)
        assert ei.value.code == 3
    finally:
        qmlp.set_log_level("warn")
        qmlp.set_kernel_cache_dir(os.environ.get("QMLP_CACHE_DIR", qmlp._lib.DEFAULT_CACHE_DIR))


def test_weights_beyond_the_lds_are_streamed_or_read_from_global_memory():
    """3 x 256x256 fp16 weights are 384 KB: the layers are staged one after the other into a
    shared LDS buffer. A 512x512 layer alone exceeds the LDS: it is gathered from global
    memory (forward) or from a transposed copy in the adjoint memory (adjoint)."""
    cfg = json.loads(json.dumps(BASE))
    cfg["network"] = [{"n_out": 256, "bias": False, "activation": "relu"}] * 3 + [{"n_out": 1, "bias": False, "activation": "relu"}]
    cfg["num_outputs"] = 1
    net = qmlp.Network(json.dumps(cfg))
    fwd, bwd = net.generated_source("forward"), net.generated_source("backward", 1)
    assert "HAS_STREAMED_LAYERS = true" in fwd and "HAS_STREAMED_LAYERS = true" in bwd
    n_streamed = fwd.count("the stream buffer is free")
    assert n_streamed >= 2 and "forward<STORE, true, " not in fwd
    assert net.adjoint_memory(64, 1) == 0
    cfg["network"] = [{"n_out": 512, "bias": False, "activation": "relu"}] * 2 + [{"n_out": 1, "bias": False, "activation": "relu"}]
    big = qmlp.Network(json.dumps(cfg))
    fwd, bwd = big.generated_source("forward"), big.generated_source("backward", 1)
    assert fwd.count("forward<STORE, true, HAS_STREAMED_LAYERS>(networkParameters +") == 1
    assert bwd.count("true, HAS_STREAMED_LAYERS>(transposedWeights +") == 1
    assert big.adjoint_memory(64, 1) == 512 * 512 * 2                         # the transposed copy
    small = qmlp.Network(json.dumps(BASE))
    assert "HAS_STREAMED_LAYERS = false" in small.generated_source("forward")
    assert small.adjoint_memory(64, 1) == 0


def test_simulated_network_and_weight_copy_shapes():
    import torch
    cfg = json.dumps({"num_inputs": 5, "num_outputs": 3, "activation_specification": [bc.BUILTIN],
                      "encodings": [{"id": "Identity", "start_in": 0, "n_in": 5}],
                      "network": [{"n_out": 20, "bias": True, "activation": "celu"},
                                  {"n_out": 3, "bias": False, "activation": "identity"}]})
    sim = qmlp.SimulatedNetwork(cfg, weight_dtype=torch.float32)
    y = sim(torch.rand(7, 5))
    assert y.shape == (7, 3) and sim.num_layers() == 2 and sim.has_bias(0) and not sim.has_bias(1)
    with pytest.raises(ValueError):
        qmlp.SimulatedNetwork(json.dumps(bc.CONFIGS[2]["cfg"]))


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_activation_objects():
    a = qmlp.Activation("relu")
    assert json.loads(a.to_json())["id"] == "relu"
    b = qmlp.Activation(json.dumps(bc.SINE30))
    assert json.loads(b.to_json())["forward"] == bc.SINE30["forward"]
    with pytest.raises(qmlp.QmlpError, match="No activation with id"):
        qmlp.Activation("swish")


def test_encoding_ids_ignore_case_like_the_reference_samples():
    """network_configs/test1.json:9 and README.md:76 of the reference write "identity"."""
    e = qmlp.Encoding(json.dumps({"id": "identity", "start_in": 1, "n_in": 2}))
    assert json.loads(e.to_json())["id"] == "Identity" and e.max_input_channel() == 2
    g = qmlp.Encoding(json.dumps(dict(bc.hashgrid3d("float"), id="hashgrid")))
    assert json.loads(g.to_json())["id"] == "HashGrid"
    with pytest.raises(qmlp.QmlpError, match="No encoding with id 'Fourier'"):
        qmlp.Encoding(json.dumps({"id": "Fourier", "start_in": 0, "n_in": 3}))


def test_line_integration_host_side():
    child = dict(bc.hashgrid3d("half"), n_levels=2, log2_hashmap_size=8, max_resolution=32, start_in=5, n_in=3,
                 bounding_box_min=[-1, -1, -1], bounding_box_size=[2, 2, 2])
    cfg = {"id": "LineIntegration", "start_in": 2, "n_in": 3, "volume": child, "stepsize": 0.05, "blending": "average"}
    e = qmlp.Encoding(json.dumps(cfg))
    back = json.loads(e.to_json())
    assert back["blending"] == "average" and back["start_in"] == 2 and abs(back["stepsize"] - 0.05) < 1e-7
    assert back["volume"]["start_in"] == 0 and back["volume"]["n_in"] == 3      # the child reads the sample position
    assert e.max_input_channel() == 2 + 6 - 1                                   # ray start + direction
    assert e.num_output_channels() == 4 and e.has_parameters()
    assert e.num_parameters() == qmlp.Encoding(json.dumps(child)).num_parameters()
    assert e.parameter_dtype() == torch.float16
    with pytest.raises(qmlp.QmlpError, match="only defined for 3D"):
        qmlp.Encoding(json.dumps(dict(cfg, n_in=2, volume=dict(child, bounding_box_min=[0, 0], bounding_box_size=[1, 1]))))
    with pytest.raises(qmlp.QmlpError, match="Stepsize must be positive"):
        qmlp.Encoding(json.dumps(dict(cfg, stepsize=0.0)))
    with pytest.raises(qmlp.QmlpError, match="Unknown blending"):
        qmlp.Encoding(json.dumps(dict(cfg, blending="max")))
    with pytest.raises(qmlp.QmlpError, match="volumetric"):
        qmlp.Encoding(json.dumps(dict(cfg, volume={"id": "Identity", "start_in": 0, "n_in": 3})))
    # as part of a network: 6 raw inputs, 4 encoded channels padded to 16
    net = qmlp.Network(json.dumps({"num_inputs": 8, "num_outputs": 1, "activation_specification": [bc.BUILTIN],
                                   "encodings": [cfg], "network": [{"n_out": 1, "bias": False, "activation": "identity"}]}))
    assert net.num_network_parameters() == 16 * 16
    assert "EncodingLineIntegration<2, 3, qmlp::kernel::LineIntegrationBlendingMode::AVERAGE" in net.generated_source("inference")


def test_pullpush_host_side(tmp_path):
    """Kernels for both dtypes compile without a GPU; the argument checks of
    Utils::fractionalPullpush (src_cpp/src/utils.cpp:112-135) fire before any device work."""
    import torch
    from qmlp import pullpush as qpp
    from qmlp._lib import check, desc, lib
    cache = str(tmp_path / "cache")
    qmlp.set_kernel_cache_dir(cache)
    try:
        qpp.precompile(torch.float32)
        qpp.precompile(torch.float64)
        assert len(os.listdir(cache)) == 20    # down, up, 4 adjoint kernels, add and copy for 3 and 4 dimensions; x2 dtypes
        with pytest.raises(qmlp.QmlpError):
            qpp.precompile(torch.float16)
    finally:
        qmlp.set_kernel_cache_dir(os.environ.get("QMLP_CACHE_DIR", qmlp._lib.DEFAULT_CACHE_DIR))

    def call(mask, data, out=None):
        out = torch.empty_like(data) if out is None else out
        check(lib.qmlp_utils_pullpush_forward(desc(mask), desc(data), desc(out), None))

    mask = torch.zeros(1, 4, 4)
    with pytest.raises(qmlp.QmlpError, match="up to 16 channels, but got 16"):
        call(mask, torch.zeros(1, 16, 4, 4))
    with pytest.raises(qmlp.QmlpError, match="mask must have 5 entries at dimension 2"):
        call(mask, torch.zeros(1, 2, 4, 5))
    with pytest.raises(qmlp.QmlpError, match="mask must be of type DOUBLE, but is FLOAT"):
        call(mask, torch.zeros(1, 2, 4, 4, dtype=torch.float64))
    with pytest.raises(qmlp.QmlpError, match="float or double"):
        call(mask.half(), torch.zeros(1, 2, 4, 4, dtype=torch.float16))
    with pytest.raises(qmlp.QmlpError, match="output has the wrong size"):
        call(mask, torch.zeros(1, 2, 4, 4), torch.zeros(1, 3, 4, 4))
    with pytest.raises(qmlp.QmlpError, match="3 dimensions"):
        call(mask[0], torch.zeros(1, 2, 4, 4))
    with pytest.raises(ValueError, match="GPU tensors only"):
        qpp.pullpush(mask, torch.zeros(1, 2, 4, 4))


def test_kernel_cache_key_covers_only_the_headers_a_source_includes(tmp_path):
    """Editing a device header recompiles the kernels that can reach it and no others."""
    import shutil
    import subprocess
    import sys
    kernels = tmp_path / "kernels"
    shutil.copytree(os.path.join(ROOT, "quick-mlp_amd", "csrc", "kernels"), kernels)
    cache = tmp_path / "cache"
    script = (
        "import sys; sys.path.insert(0, %r)\n"
        "import torch, qmlp\n"
        "qmlp.set_log_level('error')\n"
        "qmlp.Activation('relu').precompile()\n"
        "qmlp.pullpush.precompile(torch.float32)\n"
        "print(*qmlp._lib.kernel_cache_stats())\n" % os.path.join(ROOT, "quick-mlp_amd"))
    env = dict(os.environ, QMLP_KERNEL_DIR=str(kernels), QMLP_CACHE_DIR=str(cache))

    def run():
        out = subprocess.run([sys.executable, "-c", script], env=env, capture_output=True, text=True, check=True).stdout
        compiled, hits = (int(v) for v in out.split()[-2:])
        return compiled, hits

    assert run() == (12, 0)                      # 2 activation kernels + 10 pull-push kernels
    assert run() == (0, 12)
    with open(kernels / "qmlp" / "kernels" / "pullpush.h", "a") as f:
        f.write("\n// edited\n")
    assert run() == (10, 2)                      # the activation kernels do not include pullpush.h
    with open(kernels / "qmlp" / "kernels" / "common.h", "a") as f:
        f.write("\n// edited\n")
    assert run() == (12, 0)                      # everything includes common.h


def _two_grid_cfg():
    grid = dict(bc.hashgrid3d("float"), n_levels=2, log2_hashmap_size=8, min_resolution=4, max_resolution=16)
    return {"num_inputs": 3, "num_outputs": 1, "activation_specification": [bc.BUILTIN],
            "encodings": [grid, dict(grid, n_levels=3)],
            "network": [{"n_out": 16, "bias": False, "activation": "relu"},
                        {"n_out": 1, "bias": False, "activation": "identity"}]}


def test_unbound_encoding_tensors_are_refused_before_any_launch():
    """A network call with a grid whose table (or, with encoding gradients, whose gradient
    tensor) is not bound must raise instead of handing a null pointer to the kernel. The
    checks come before compilation and launch, so host tensors stand in for device memory."""
    from qmlp._lib import check, desc, lib
    net = qmlp.Network(json.dumps(_two_grid_cfg()))
    n = 64
    x, y = torch.zeros(n, 3), torch.zeros(n, 1)
    params = torch.zeros(net.num_network_parameters(), dtype=torch.float16)
    tables = [torch.zeros(net.encoding(i).num_parameters()) for i in range(2)]
    tmp = torch.zeros(1 << 20, dtype=torch.uint8)
    check(lib.qmlp_network_set_parameter(net._handle, desc(params), 0))

    def inference():
        check(lib.qmlp_network_inference(net._handle, desc(x), desc(y), None))

    def forward():
        check(lib.qmlp_network_forward(net._handle, desc(x), desc(y), ctypes.c_void_p(tmp.data_ptr()), None))

    def adjoint(flags):
        check(lib.qmlp_network_adjoint(net._handle, desc(x), desc(y), flags, desc(torch.zeros(n, 3)),
                                       ctypes.c_void_p(tmp.data_ptr()), ctypes.c_void_p(tmp.data_ptr()), None))

    for call in (inference, forward, lambda: adjoint(1)):
        with pytest.raises(qmlp.QmlpError, match="Encoding 0 has parameters, but no inference tensor"):
            call()
    net.encoding(0).set_parameter(tables[0])
    with pytest.raises(qmlp.QmlpError, match="Encoding 1 has parameters, but no inference tensor"):
        inference()
    net.encoding(1).set_parameter(tables[1])
    # one grid trainable, one frozen: the kernel adds into both gradient tables
    net.encoding(0).set_parameter(torch.zeros_like(tables[0]), gradients=True)
    with pytest.raises(qmlp.QmlpError, match="encoding 1 has no gradient tensor"):
        adjoint(4)
    with pytest.raises(qmlp.QmlpError, match="encoding 1 has no gradient tensor"):
        adjoint(5)

    # standalone encoding: no table bound or passed
    enc = qmlp.Encoding(json.dumps(_two_grid_cfg()["encodings"][0]))
    out = torch.zeros(n, enc.num_output_channels())
    with pytest.raises(qmlp.QmlpError, match="no inference tensor is bound or passed"):
        check(lib.qmlp_encoding_forward(enc._handle, desc(x), desc(out), None, None))
    with pytest.raises(qmlp.QmlpError, match="no gradient tensor is bound or passed"):
        check(lib.qmlp_encoding_adjoint(enc._handle, desc(x), desc(out), desc(torch.zeros(n, 3)), None,
                                        desc(tables[0]), None, 3))


def test_the_python_binding_cache_forgets_a_table_the_standalone_call_unbound():
    """Encoding.set_parameter skips binding the same memory twice; the standalone
    *_with_parameter calls leave the native encoding unbound, so they must reset that memory."""
    enc = qmlp.Encoding(json.dumps(_two_grid_cfg()["encodings"][0]))
    t = torch.zeros(enc.num_parameters())
    enc.set_parameter(t)
    assert enc._bound_inference is not None
    src = open(os.path.join(ROOT, "quick-mlp_amd", "qmlp", "classes.py")).read()
    for name in ("inference_with_parameter", "adjoint_with_parameter_and_flags"):
        body = src.split("def %s(" % name)[1].split("\n    def ")[0]
        assert "self._bound_inference = None" in body, name


def test_rows_in_registers_shape_is_not_offered_to_single_table_or_gather_heavy_grids():
    """The forward shape that keeps the encoded rows of 8 tiles in registers pays through fewer
    sweeps over the tables of a multi-level grid. A grid with one table has nothing to sweep, and
    a cell whose gathers need more than 128 registers for 8 points spills by the kilobyte: a
    dense 4-D grid with 8 features (BASELINE config 5) is both, and its kernel of that shape
    once ended in a GPU memory fault. Such networks must never be given the shape."""
    def shapes(cfg):
        return {(s["pass"], s["shape"]) for s in json.loads(qmlp.Network(json.dumps(cfg)).generated_source("shapes"))}

    assert ("inference", "registers") in shapes(bc.CONFIGS[2]["cfg"])
    for cfg_id in (1, 4, 5):
        assert not any(shape == "registers" for _, shape in shapes(bc.CONFIGS[cfg_id]["cfg"])), cfg_id
    base = bc.CONFIGS[5]["cfg"]
    for change in ({"n_features_per_level": 2}, {"n_features_per_level": 4, "n_levels": 1},
                   {"n_levels": 2, "min_resolution": 16, "max_resolution": 32}):      # 2 levels, but 16 corners x 8 features
        cfg = json.loads(json.dumps(base))
        cfg["encodings"][0].update(change)
        got = shapes(cfg)
        if cfg["encodings"][0]["n_levels"] < 2:
            assert not any(shape == "registers" for _, shape in got), change
        else:
            # 8 points x 16 corners x 8 fp16 features = 512 registers in flight: beyond the limit of 128
            assert not any(shape == "registers" for _, shape in got), change
    # and the option switches the shape off for a network that would get it
    cfg = json.loads(json.dumps(bc.CONFIGS[2]["cfg"]))
    cfg["options"] = {"register_staging": False}
    assert not any(shape == "registers" for _, shape in shapes(cfg))


@pytest.mark.parametrize("option,value,flags,kind", [
    ("overwrite_blocksize_inference", 96, 0, "inference"),
    ("overwrite_blocksize_inference", 2048, 0, "inference"),
    ("overwrite_blocksize_forward", 100, 1, "forward"),
    ("overwrite_blocksize_backward", 32, 1, "backward"),
    ("overwrite_blocksize_backward", 1088, 3, "backward"),
    ("overwrite_blocksize_weight_update", 100, 2, "weight_update"),
    ("overwrite_blocksize_weight_update", 4096, 2, "weight_update"),
])
def test_launch_options_out_of_range_are_refused(option, value, flags, kind):
    """Workgroups are whole wavefronts of 64 lanes, at most 16 of them (the reference takes any
    multiple of its warp size up to the device limit, src_cpp/src/fused_network.cpp:472-485)."""
    cfg = json.loads(json.dumps(BASE))
    cfg["options"] = {option: value}
    net = qmlp.Network(json.dumps(cfg))          # options are parsed here, applied when a kernel is generated
    message = "multiple of 64 and at most 1024, but is %d" % value
    with pytest.raises(qmlp.QmlpError, match=message) as ei:
        net.precompile(flags)
    assert ei.value.code == 1                    # configuration_error
    with pytest.raises(qmlp.QmlpError, match=message):
        net.generated_source(kind, flags) if kind == "backward" else net.generated_source(kind)
    # the kernels the option does not concern still generate
    other = "backward" if kind != "backward" else "forward"
    assert "__launch_bounds__(256)" in (net.generated_source(other, 1) if other == "backward" else net.generated_source(other))


def test_launch_options_shape_the_generated_kernels():
    cfg = json.loads(json.dumps(BASE))
    cfg["options"] = {"overwrite_blocksize_inference": 64, "overwrite_blocksize_forward": 512,
                      "overwrite_blocksize_backward": 1024, "overwrite_blocksize_weight_update": 128,
                      "skew_shared_memory": True, "parallel_weight_update": False}
    net = qmlp.Network(json.dumps(cfg))
    assert "__launch_bounds__(64)" in net.generated_source("inference")
    assert "__launch_bounds__(512)" in net.generated_source("forward")
    assert "__launch_bounds__(1024)" in net.generated_source("backward", 3)
    assert "__launch_bounds__(128)" in net.generated_source("weight_update")
    shapes = json.loads(net.generated_source("shapes"))
    assert {(s["pass"], s["block"]) for s in shapes} == {("inference", 64), ("forward", 512)}
    # zero and negative values mean "not overwritten", as in the reference (values > 0 are taken)
    cfg["options"] = {"overwrite_blocksize_inference": -1, "overwrite_blocksize_backward": 0}
    net = qmlp.Network(json.dumps(cfg))
    assert "__launch_bounds__(256)" in net.generated_source("inference")
    assert "__launch_bounds__(256)" in net.generated_source("backward", 3)


def test_staging_rows_beyond_the_lds_are_a_configuration_error():
    """A workgroup shrinks until the staging rows of its wavefronts fit into the LDS beside the
    weights; a network whose one staging tile does not fit is refused (the reference shrinks its
    blocks the same way, src_cpp/src/fused_network.cpp:476-485, and then fails at the launch)."""
    wide = {"num_inputs": 2048, "num_outputs": 16, "activation_specification": [bc.BUILTIN],
            "encodings": [{"id": "Identity", "start_in": 0, "n_in": 2048}],
            "network": [{"n_out": 16, "bias": False, "activation": "relu"}]}
    net = qmlp.Network(json.dumps(wide))
    with pytest.raises(qmlp.QmlpError, match="too large for the fused kernels") as ei:
        net.generated_source("backward", 1)
    assert ei.value.code == 1
    # 1024 asked for, but 16 wavefronts x 64 rows x 264 halves exceed the LDS beside the weights
    mid = json.loads(json.dumps(wide))
    mid["num_inputs"] = 256
    mid["encodings"][0]["n_in"] = 256
    mid["options"] = {"overwrite_blocksize_backward": 1024}
    src = qmlp.Network(json.dumps(mid)).generated_source("backward", 1)
    m = re.search(r"__launch_bounds__\((\d+)\) [^;]*NetworkKernelBackward", src)
    assert m and int(m.group(1)) % 64 == 0 and 64 <= int(m.group(1)) < 1024
