#!/usr/bin/env python3
"""Benchmark of the fused hash-grid + MLP path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2-inference]

A step is one pass of the hot path over one batch of synthetic input that already
resides in HBM: by default the fused inference kernel of the hash-grid(16 levels, 2 fp16
features, 2^19 entries) -> 64 -> 64 -> 1 network on 2^20 points. Prints ONE JSON line;
`value` is points per second of that workload, `roofline` prices the kernel against the
HBM peak with its algorithmic bytes (gathered table entries + input + output), and
`cpu_baseline` is the CPU oracle timed on this machine's host cores on the same workload.
The train step of the same network (2^18 points: forward with stored intermediates,
adjoint with grid scatter, weight update) is reported under "train_step".
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (os.path.join(ROOT, "quick-mlp_amd"), os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 matrix, published

# HBM bytes one launch moves, from hardware counters (two profiler runs of this script:
# FETCH_SIZE and WRITE_SIZE per dispatch, each scaled by what the same counter reads for the
# 256 MiB device copy of --copy-calibration: x2.000 and x1.000 on MI355X). The summary
# with the commands is kept under profiles/. The figures belong to one version of the device
# code: "kernels" is device_code_hash() at the time of the counter runs, and a workload whose
# device code has changed since (or that has no counter run) reports traffic null.
MEASURED_TRAFFIC_BYTES = {
    "cfg2-inference": {"points": 1 << 20, "fetch": 105163.0 * 1024 * 2.0, "write": 4096.0 * 1024 * 1.0,
                       "kernels": "6abc8c19b03aa50d"},
}


def device_code_hash(net):
    """Hash of everything the fused forward kernel of `net` is compiled from: the generated
    source and the device headers it includes, directly or through other headers."""
    import hashlib
    import re
    source = net.generated_source("forward")
    kernel_dir = os.path.join(ROOT, "quick-mlp_amd", "csrc", "kernels")
    seen, todo = {}, [source]
    while todo:
        text = todo.pop()
        for name in re.findall(r'#include\s*[<"]([^>"]+)[>"]', text):
            path = os.path.join(kernel_dir, name)
            if name not in seen and os.path.isfile(path):
                seen[name] = open(path, "rb").read()
                todo.append(seen[name].decode())
    h = hashlib.sha256(source.encode())
    for name in sorted(seen):
        h.update(name.encode() + b"\0" + seen[name] + b"\0")
    return h.hexdigest()[:16]

WORKLOADS = {
    "cfg1-inference": (1, False),
    "cfg2-inference": (2, False),
    "cfg3-train": (3, True),
    "cfg4-inference": (4, False),
    "cfg4-train": (4, True),
    "cfg5-inference": (5, False),
    "cfg5-train": (5, True),
}


def build_case(cfg_id, n_points, device):
    import numpy as np
    import torch
    import qmlp
    import baseline_configs as bc
    c = bc.CONFIGS[cfg_id]
    rng = np.random.default_rng(bc.PARAMETER_SEED[cfg_id])
    net = qmlp.Network(json.dumps(c["cfg"]))
    params_np = bc.make_parameters(cfg_id, rng)
    tables_np = []
    enc_params = []
    for i in range(net.num_encodings()):
        e = net.encoding(i)
        if e.has_parameters():
            t = bc.make_table(cfg_id, e.num_parameters(), rng)
            tables_np.append(t)
            enc_params.append(torch.from_numpy(t).to(e.parameter_dtype()).to(device))
        else:
            tables_np.append(None)
            enc_params.append(None)
    X = bc.make_inputs(cfg_id, n_points, rng)
    return dict(cfg_id=cfg_id, cfg=c, net=net, params_np=params_np, tables_np=tables_np, X_np=X,
                params=torch.from_numpy(params_np).to(device), enc_params=enc_params,
                x=torch.from_numpy(X).to(device))


def time_steps(step, steps, warmup, warmup_seconds=0.0):
    """W untimed steps, then exactly K timed ones between two synchronisations. Every timed
    step is also bracketed by HIP events on the launch stream for the per-launch duration.
    warmup_seconds > 0 (secondary measurements only): untimed steps go on until that much time
    has passed as well, so that the device is back at its clocks after host-side set-up."""
    import torch
    t_warm = time.perf_counter()
    done = 0
    while done < warmup or (warmup_seconds > 0 and time.perf_counter() - t_warm < warmup_seconds):
        step()
        done += 1
        if warmup_seconds > 0 and done % 4 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        step()
        stops[i].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    per_launch_ms = [a.elapsed_time(b) for a, b in zip(starts, stops)]
    return elapsed, sum(per_launch_ms) / len(per_launch_ms)


def run_inference(case, steps, warmup):
    import torch
    net, x, params, enc = case["net"], case["x"], case["params"], case["enc_params"]
    out_holder = {}

    def step():
        out_holder["out"] = net.inference(x, params, enc)

    step()   # compiles (or loads from the kernel cache) outside of any timing
    torch.cuda.synchronize()
    return time_steps(step, steps, warmup)


def ordered_batch_report(cfg_id, n, device, steps, warmup):
    """The inference launch of a hash-grid network on the same batch in three orders: as given; ordered by the
    library in front of the kernel (options.sort_points = 1: slabs of the grid's second and third coordinate,
    the sort inside the timed step); and arriving in that order (sorted beforehand with torch, nothing for the
    library to do: what a caller with coherent batches, e.g. rays of an image tile, gets)."""
    import torch
    import baseline_configs as bc
    base = bc.CONFIGS[cfg_id]["cfg"]
    out = {}
    results = {}
    try:
        for name, mode in (("as_given", 0), ("sorted_by_the_library", 1), ("arrives_in_slab_order", 0)):
            bc.CONFIGS[cfg_id]["cfg"] = json.loads(json.dumps(base))
            bc.CONFIGS[cfg_id]["cfg"].setdefault("options", {})["sort_points"] = mode
            case = build_case(cfg_id, n, device)
            if name == "arrives_in_slab_order":
                x = case["x"]
                q = (x.clamp(0, 1 - 1e-7) * 32).long()
                key = torch.zeros_like(q[:, 0])
                for b in range(5):
                    key |= ((q[:, 1] >> b) & 1) << (2 * b + 1) | ((q[:, 2] >> b) & 1) << (2 * b)
                order = torch.argsort(key * n + torch.randperm(n, device=device))
                case["x"] = x[order].contiguous()
                results[name] = (case["net"].inference(case["x"], case["params"], case["enc_params"]), order)
            else:
                results[name] = (case["net"].inference(case["x"], case["params"], case["enc_params"]), None)
            elapsed, launch_ms = run_inference(case, steps, warmup)
            out[name] = {"ms_per_step": 1e3 * elapsed / steps, "launch_ms": launch_ms}
            del case
    finally:
        bc.CONFIGS[cfg_id]["cfg"] = base
    ref = results["as_given"][0]
    out["same_bits"] = bool(torch.equal(ref, results["sorted_by_the_library"][0])
                            and torch.equal(ref[results["arrives_in_slab_order"][1]], results["arrives_in_slab_order"][0]))
    return out


LOSS_SCALE = 65536.0


def run_train(case, steps, warmup, input_gradients=True, warmup_seconds=0.0):
    import torch
    import baseline_configs as bc
    net, x, params, enc = case["net"], case["x"], case["params"], case["enc_params"]
    cfg_id = case["cfg_id"]
    n = x.shape[0]
    target = torch.from_numpy(bc.make_targets(cfg_id, case["X_np"])).to(x.device)
    flags = (1 if input_gradients else 0) | 2 | (4 if any(e is not None for e in enc) else 0)
    grad_net = torch.zeros((net.num_network_parameters(),), dtype=torch.float32, device=x.device)
    grad_enc = [None if e is None else torch.zeros(e.shape, dtype=torch.float32, device=x.device) for e in enc]
    adj_in = torch.zeros_like(x)

    def step():
        # one full train step without the optimizer: forward with stored intermediates,
        # L2-loss adjoint, backward to inputs + grid, weight update (gradients re-zeroed)
        grad_net.zero_()
        adj_in.zero_()
        for g in grad_enc:
            if g is not None:
                g.zero_()
        out, tmp = net.forward_raw(x, params, enc, flags)
        # (mean squared error with the loss scaled by 2^16, as fp16 training does: 2 / numel alone is 5e-7 for 2^21
        # points with two outputs, and the adjoints of the layers, which are halves, underflow to zero -- a step whose
        # gradients vanish is not the work of a train step: kernels that skip zeros would look faster than they are)
        adj_out = (out - target) * (2.0 * LOSS_SCALE / out.numel())
        net.adjoint_raw(x, adj_out, flags, tmp, params, enc, grad_network=grad_net, grad_encodings=grad_enc,
                        adj_input=adj_in if input_gradients else None)

    step()
    torch.cuda.synchronize()
    return time_steps(step, steps, warmup, warmup_seconds)


def cpu_baseline(case, train, min_seconds=10.0):
    """The CPU oracle (an fp32 port of the reference's Eigen test evaluation, OpenMP over
    points) on the same workload, repeated until at least min_seconds of CPU work."""
    import numpy as np
    import qmlp_oracle as qo
    import baseline_configs as bc
    cfg_id = case["cfg_id"]
    oracle = qo.Network(case["cfg"]["cfg"], bc.ORACLE_ACTIVATIONS)
    oracle.set_parameters(case["params_np"].astype(np.float32))
    for i, t in enumerate(case["tables_np"]):
        if t is not None:
            oracle.set_table(i, qo.round_half(t))
    X = case["X_np"]
    n = X.shape[0]
    adj = np.full((n, oracle.n_out), 1.0 / n, dtype=np.float32)
    times = []
    t_all = time.perf_counter()
    while True:
        t0 = time.perf_counter()
        if train:
            oracle.backward(X, adj, 7 if any(t is not None for t in case["tables_np"]) else 3)
        else:
            oracle.forward(X)
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_all >= min_seconds and len(times) >= 2:
            break
    best = sorted(times)[len(times) // 2]
    return {"value": n / best, "unit": "points/s", "cores": qo.lib().qo_num_threads(), "kind": "port",
            "sample": "%d repetitions of the full workload (%d points), median; fp32 C oracle with OpenMP"
                      % (len(times), n)}


# ------------------------------------------------------------------ layer GEMMs alone
def mlp_cfg(n_in, widths, activation="relu", last="identity"):
    import baseline_configs as bc
    acts = [activation] * (len(widths) - 1) + [last]
    return {"num_inputs": n_in, "num_outputs": widths[-1], "activation_specification": [bc.BUILTIN],
            "encodings": [{"id": "Identity", "start_in": 0, "n_in": n_in}],
            "network": [{"n_out": w, "bias": False, "activation": a} for w, a in zip(widths, acts)]}


def mlp_flops(n_in, widths, padded):
    up = (lambda v: (v + 15) // 16 * 16) if padded else (lambda v: v)
    chain = [up(n_in)] + [up(w) for w in widths]
    return 2 * sum(a * b for a, b in zip(chain[:-1], chain[1:]))


def run_mlp(n_in, widths, n, device, steps, warmup, cached_input=False, train=False, seed=0, back_to_back=1):
    """The layers of an identity-encoded network on n points. cached_input: every point reads the
    same input row (a tensor with stride 0 along the batch), so the input comes from cache and
    the launch is bound by the layers; otherwise the fp32 rows stream from HBM (4*n_in bytes per
    point, which bounds narrow networks before the matrix cores do). Returns ms per launch."""
    import numpy as np
    import torch
    import qmlp
    cfg = mlp_cfg(n_in, widths)
    net = qmlp.Network(json.dumps(cfg))
    rng = np.random.default_rng(seed)
    params = torch.from_numpy((rng.uniform(-1, 1, net.num_network_parameters()) / 8).astype(np.float16)).to(device)
    if cached_input:
        x = torch.from_numpy(rng.uniform(-1, 1, (1, n_in)).astype(np.float32)).to(device).expand(n, n_in)
    else:
        x = torch.from_numpy(rng.uniform(-1, 1, (n, n_in)).astype(np.float32)).to(device)
    if not train:
        def step():
            net.inference(x, params, [])
    else:
        adj = torch.from_numpy(rng.uniform(-1, 1, (n, widths[-1])).astype(np.float32)).to(device)
        grad_net = torch.zeros((net.num_network_parameters(),), dtype=torch.float32, device=device)
        adj_in = torch.zeros((n, n_in), dtype=torch.float32, device=device)

        def step():
            # the reference's "forward + backward": gradients for the input and the weights
            out, tmp = net.forward_raw(x, params, [], 3)
            net.adjoint_raw(x, adj, 3, tmp, params, [], grad_network=grad_net, adj_input=adj_in)
    step()
    torch.cuda.synchronize()
    elapsed, launch_ms = time_steps(step, steps, warmup)
    if back_to_back > 1 and not train:
        # the same launch 16 times in one captured graph: the kernels then follow each other without the gap
        # that the host leaves between two launches of a kernel this short (the call path neither allocates
        # nor synchronises, so it can be captured)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(back_to_back):
                step()
        _, graph_ms = time_steps(graph.replay, max(3, steps // 4), 2)
        return launch_ms, 1e3 * elapsed / steps, graph_ms / back_to_back
    return launch_ms, 1e3 * elapsed / steps


LAYER_GEMM_NETWORKS = (("cfg2_mlp", 32, [64, 64, 1]), ("mlp_64x4", 64, [64, 64, 64, 64, 4]))
REFERENCE_GRID = [(width, [width] * hidden + [4]) for hidden in (2, 4) for width in (16, 32, 64)]


def precompile_networks():
    """Compiles the kernels of the identity-encoded benchmark networks into the kernel cache
    (no GPU needed); the build step calls this."""
    import qmlp
    for n_in, widths in [(n, w) for _, n, w in LAYER_GEMM_NETWORKS] + REFERENCE_GRID:
        qmlp.Network(json.dumps(mlp_cfg(n_in, widths))).precompile(3)


def layer_gemm_report(device, steps, warmup, only="", n=1 << 20):
    """MFMA fraction of the layer GEMMs of the hash-grid network (32 -> 64 -> 64 -> 1) run on their
    own on 2^20 points, and of a deeper 64-wide network."""
    out = {}
    for name, n_in, widths in LAYER_GEMM_NETWORKS:
        for cached in (False, True):
            if only and only != name + ("_cached_input" if cached else ""):
                continue
            ms, _, kernel_ms = run_mlp(n_in, widths, n, device, steps, warmup, cached_input=cached, back_to_back=16)
            key = name + ("_cached_input" if cached else "")
            frac = lambda t, padded: mlp_flops(n_in, widths, padded) * n / (t * 1e-3) / 1e12 / MFMA_FP16_PEAK_TFLOPS
            out[key] = {"launch_ms": ms, "points": n, "frac": frac(ms, False), "frac_padded_flop": frac(ms, True),
                        # 16 launches back to back in one graph: the duration of the kernel without the host's gap
                        "back_to_back_ms": kernel_ms, "frac_back_to_back": frac(kernel_ms, False),
                        "frac_padded_flop_back_to_back": frac(kernel_ms, True),
                        "input_hbm_bound_ms": None if cached else 4.0 * (n_in + widths[-1]) * n / (HBM_PEAK_GBS * 1e9) * 1e3}
            if cached and n == 1 << 20:
                # the same kernel on 2^23 points: eight times the tiles per wavefront, the ramp at both ends counts less
                big, _ = run_mlp(n_in, widths, 1 << 23, device, max(3, steps // 4), 2, cached_input=True)
                out[key]["launch_ms_8M_points"] = big
                out[key]["frac_8M_points"] = mlp_flops(n_in, widths, False) * (1 << 23) / (big * 1e-3) / 1e12 / MFMA_FP16_PEAK_TFLOPS
    return out


def torch_baseline(width, widths, n, device, half, trials=10, startup=2):
    """The reference's own comparison on the same device (tests_py/qmlp_tests/profile_network.py:27-60,
    149-177): a stack of torch.nn.Linear layers without bias, ReLU between them, in fp32 or (input cast to half,
    output cast back) in fp16; wall clock of a call between two synchronisations, 10 trials of which the first
    two are dropped; inference under no_grad, then forward + backward with the gradient of the input."""
    import numpy as np
    import torch
    layers, last = [], width
    for i, w in enumerate(widths):
        layers.append(torch.nn.Linear(last, w, bias=False))
        if i + 1 < len(widths):
            layers.append(torch.nn.ReLU())
        last = w
    net = torch.nn.Sequential(*layers).to(device)
    if half:
        net = net.half()
    run = (lambda x: net(x.half()).float()) if half else net
    x = torch.randn((n, width), device=device, dtype=torch.float32, requires_grad=True)
    grad_out = torch.randn((n, widths[-1]), device=device, dtype=torch.float32)
    times = [[], []]
    with torch.no_grad():
        for _ in range(trials):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            run(x)
            torch.cuda.synchronize()
            times[0].append(time.perf_counter() - t0)
    for _ in range(trials):
        x.grad = None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = run(x)
        torch.autograd.backward(out, grad_out)
        torch.cuda.synchronize()
        times[1].append(time.perf_counter() - t0)
    return [1e3 * float(np.mean(t[startup:])) for t in times]


def reference_grid(device, steps, warmup, only=""):
    """The benchmark grid of the reference (tests_py/qmlp_tests/profile_network.py:107-190):
    10^6 points, 2 or 4 hidden layers of 16, 32 or 64 neurons (as many inputs), ReLU, 4 outputs,
    no bias, identity encoding; inference and forward + backward (input and weight gradients), next to the
    PyTorch-32 and PyTorch-16 networks that the reference times beside its own."""
    n = 1000 * 1000
    rows = []
    for width, widths in REFERENCE_GRID:
        hidden = len(widths) - 1
        if not only or only == "%d x %d" % (width, hidden):
            inf_ms, inf_wall = run_mlp(width, widths, n, device, steps, warmup)
            trn_ms, trn_wall = run_mlp(width, widths, n, device, max(3, steps // 2), min(warmup, 3), train=True)
            flop = mlp_flops(width, widths, False)
            t32, t16 = torch_baseline(width, widths, n, device, False), torch_baseline(width, widths, n, device, True)
            rows.append({"network": "%d x %d" % (width, hidden), "points": n,
                         # stated baselines on the same device, not targets: torch.nn.Linear stacks, wall clock per call
                         "torch_fp32_inference_ms": t32[0], "torch_fp32_forward_backward_ms": t32[1],
                         "torch_fp16_inference_ms": t16[0], "torch_fp16_forward_backward_ms": t16[1],
                         "inference_ms": inf_ms, "inference_wall_ms": inf_wall,
                         "forward_backward_ms": trn_ms, "forward_backward_wall_ms": trn_wall,
                         "inference_mfma_frac": flop * n / (inf_ms * 1e-3) / 1e12 / MFMA_FP16_PEAK_TFLOPS,
                         "inference_hbm_frac": 4.0 * (width + 4) * n / (inf_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                         "forward_backward_mfma_frac": 3 * flop * n / (trn_ms * 1e-3) / 1e12 / MFMA_FP16_PEAK_TFLOPS})
    return rows


# ------------------------------------------------------------------ the request rate of random gathers
GATHER_SOURCE = r"""
#include <hip/hip_runtime.h>
// Random 8-byte gathers, one 128-byte line per lane and load, eight loads in flight per lane:
// what the grid encodings do. The indices are hashed in the kernel, nothing else touches memory.
__device__ __forceinline__ unsigned mix(unsigned x)
{
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}
extern "C" __global__ void __launch_bounds__(256) GatherCeiling(const unsigned long long* __restrict__ table,
                                                                unsigned entries, float* __restrict__ out, int iters)
{
    const unsigned gid = blockIdx.x * blockDim.x + threadIdx.x;
    unsigned long long acc = 0;
    for (int it = 0; it < iters; it += 8) {
        unsigned e[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) e[k] = mix(gid * 977u + (it + k) * 0x9e3779b9u) % entries;
#pragma unroll
        for (int k = 0; k < 8; ++k) acc += table[e[k]];
    }
    if (acc == 0x123456789abcdefull) out[gid] = 1.f;
}
"""


def gather_ceiling(device, repeats=5):
    """Lane-loads per second of random 8-byte gathers from a table that stays in the L2 of every
    die (2 MiB) and from one that does not (64 MiB), through the loader's C ABI (qmlp_hip.h).
    Every load of a lane is a 128-byte line of its own, as in a hashed grid level."""
    import ctypes
    import torch
    import qmlp
    lib = qmlp._lib.lib
    lib.qmlp_hip_last_error.restype = ctypes.c_char_p

    def ok(rc):
        if rc != 0:
            raise RuntimeError(lib.qmlp_hip_last_error().decode())

    module, fn, lowered = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_char_p()
    names = (ctypes.c_char_p * 1)(b"GatherCeiling")
    opts = (ctypes.c_char_p * 6)(b"-O3", b"-I/opt/rocm/include", b"-Xclang", b"-target-feature", b"-Xclang", b"-packed-fp32-ops")
    ok(lib.qmlp_hip_module_compile(GATHER_SOURCE.encode(), b"gather_ceiling.hip", None, None, 0, names, 1, opts, 6,
                                   None, ctypes.byref(module), None))
    ok(lib.qmlp_hip_module_load(module))
    ok(lib.qmlp_hip_module_lowered_name(module, b"GatherCeiling", ctypes.byref(lowered)))
    ok(lib.qmlp_hip_module_get_function(module, lowered, ctypes.byref(fn)))
    props = torch.cuda.get_device_properties(device)
    cus, clock_hz = props.multi_processor_count, 2.4e9
    blocks, threads, iters = 2048, 256, 64
    table = torch.ones((64 << 20) // 8, dtype=torch.int64, device=device)
    out = torch.zeros(blocks * threads, dtype=torch.float32, device=device)
    stream = qmlp._lib.current_stream(device)
    result = {}
    for name, nbytes in (("l2_hit", 2 << 20), ("l2_miss", 64 << 20)):
        a_table, a_entries = ctypes.c_void_p(table.data_ptr()), ctypes.c_uint32(nbytes // 8)
        a_out, a_iters = ctypes.c_void_p(out.data_ptr()), ctypes.c_int(iters)
        args = (ctypes.c_void_p * 4)(ctypes.addressof(a_table), ctypes.addressof(a_entries), ctypes.addressof(a_out),
                                     ctypes.addressof(a_iters))
        ok(lib.qmlp_hip_launch(fn, blocks, threads, 0, stream, args))
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(repeats):
            ok(lib.qmlp_hip_launch(fn, blocks, threads, 0, stream, args))
        stop.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(stop) / repeats
        loads = float(blocks) * threads * iters
        result[name] = {"table_bytes": nbytes, "requests_per_s": loads / (ms * 1e-3),
                        "requests_per_clock_and_cu": loads / (ms * 1e-3) / cus / clock_hz, "launch_ms": ms}
    ok(lib.qmlp_hip_module_destroy(module))
    result["compute_units"] = cus
    result["clock_hz_assumed"] = clock_hz
    return result


PATTERN_SOURCE = r"""
#include <hip/hip_runtime.h>
// What one gather instruction of a wavefront costs, by the cache lines its 64 lanes ask for. Every lane has a line
// number and a word in that line that stay fixed over the loop; every iteration adds an offset that is the same for
// the whole wavefront (so the per-load arithmetic is three vector instructions), eight loads are in flight per lane.
__device__ __forceinline__ unsigned mix(unsigned x)
{
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}
template <int W>
__device__ void body(const unsigned* __restrict__ table, unsigned lineMask, const unsigned* __restrict__ laneLine,
                     const unsigned* __restrict__ laneWord, float* out, int iters)
{
    const unsigned gid = blockIdx.x * blockDim.x + threadIdx.x;
    const unsigned lane = threadIdx.x & 63;
    const unsigned myLine = laneLine[lane], myWord = laneWord[lane];
    unsigned acc = 0, h = mix(gid >> 6);
    typedef unsigned vec __attribute__((ext_vector_type(W)));
    for (int it = 0; it < iters; it += 8) {
        vec v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            h = h * 1664525u + 1013904223u;
            const unsigned line = (myLine + (h >> 8)) & lineMask;
            v[j] = *reinterpret_cast<const vec*>(table + line * 32u + myWord);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
            for (int w = 0; w < W; ++w) acc += v[j][w];
    }
    if (acc == 0x12345678u) out[gid] = 1.f;
}
extern "C" __global__ void __launch_bounds__(256) GatherPattern4(const unsigned* t, unsigned m, const unsigned* l, const unsigned* w, float* o, int n) { body<1>(t, m, l, w, o, n); }
extern "C" __global__ void __launch_bounds__(256) GatherPattern8(const unsigned* t, unsigned m, const unsigned* l, const unsigned* w, float* o, int n) { body<2>(t, m, l, w, o, n); }
"""


def gather_patterns(device, repeats=3):
    """Cycles of one compute unit per gather instruction of a wavefront, by the number of distinct 128-byte lines its
    lanes ask for (1, 16 or 64), by how the lanes that share a line are placed (neighbours or spread), and by
    whether the lines are found in the L1 (a region of 8 KiB) or come from the L2 (a region of 2 MiB, which is
    the table of one level of the hash grid). The clock is taken as 2.4 GHz."""
    import ctypes
    import numpy as np
    import torch
    import qmlp
    lib = qmlp._lib.lib
    lib.qmlp_hip_last_error.restype = ctypes.c_char_p

    def ok(rc):
        if rc != 0:
            raise RuntimeError(lib.qmlp_hip_last_error().decode())

    kernels = [b"GatherPattern4", b"GatherPattern8"]
    module = ctypes.c_void_p()
    names = (ctypes.c_char_p * len(kernels))(*kernels)
    opts = (ctypes.c_char_p * 6)(b"-O3", b"-I/opt/rocm/include", b"-Xclang", b"-target-feature", b"-Xclang", b"-packed-fp32-ops")
    ok(lib.qmlp_hip_module_compile(PATTERN_SOURCE.encode(), b"gather_patterns.hip", None, None, 0, names, len(kernels), opts, 6,
                                   None, ctypes.byref(module), None))
    ok(lib.qmlp_hip_module_load(module))
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    blocks, threads, iters = 8 * cus, 256, 512
    table = torch.ones((4 << 20) // 4, dtype=torch.int32, device=device)
    out = torch.zeros(blocks * threads, dtype=torch.float32, device=device)
    stream = qmlp._lib.current_stream(device)
    rng = np.random.default_rng(1)
    rows = []
    for kernel, width in zip(kernels, (1, 2)):
        fn, lowered = ctypes.c_void_p(), ctypes.c_char_p()
        ok(lib.qmlp_hip_module_lowered_name(module, kernel, ctypes.byref(lowered)))
        ok(lib.qmlp_hip_module_get_function(module, lowered, ctypes.byref(fn)))
        for region in (8 << 10, 2 << 20):
            for lines, placement in ((1, "neighbours"), (16, "neighbours"), (16, "spread"), (64, "neighbours")):
                lane = np.arange(64)
                line = (lane // (64 // lines) if placement == "neighbours" else lane % lines) * 7919
                word = rng.integers(0, 32 // width, 64) * width
                d_line = torch.from_numpy(line.astype(np.int32)).to(device)
                d_word = torch.from_numpy(word.astype(np.int32)).to(device)
                a = [ctypes.c_void_p(table.data_ptr()), ctypes.c_uint32(region // 128 - 1), ctypes.c_void_p(d_line.data_ptr()),
                     ctypes.c_void_p(d_word.data_ptr()), ctypes.c_void_p(out.data_ptr()), ctypes.c_int(iters)]
                args = (ctypes.c_void_p * len(a))(*[ctypes.addressof(v) for v in a])
                ok(lib.qmlp_hip_launch(fn, blocks, threads, 0, stream, args))
                torch.cuda.synchronize()
                start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                for _ in range(repeats):
                    ok(lib.qmlp_hip_launch(fn, blocks, threads, 0, stream, args))
                stop.record()
                torch.cuda.synchronize()
                ms = start.elapsed_time(stop) / repeats
                instructions_per_cu = blocks * threads / 64 * iters / cus
                rows.append({"bytes_per_lane": 4 * width, "region_bytes": region, "lines_per_instruction": lines,
                             "lanes_of_a_line": placement, "launch_ms": ms,
                             "clocks_per_instruction_and_cu": ms * 1e-3 * 2.4e9 / instructions_per_cu})
    ok(lib.qmlp_hip_module_destroy(module))
    return rows


OVERLAP_SOURCE = r"""
#include <hip/hip_runtime.h>
// Do the matrix cores and the vector ALUs of a SIMD work side by side? Per iteration 32 matrix instructions on
// 8 independent accumulator tiles (MODE & 1) and 320 packed fp16 vector instructions on 16 independent registers
// (MODE & 2); nothing one stream computes is used by the other.
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int MODE>
__device__ void body(float* out, int iters)
{
    f16x8 a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(threadIdx.x * 0.001f + i); b[i] = (_Float16)(threadIdx.x * 0.002f - i); }
    f32x4 acc[8];
    for (int i = 0; i < 8; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    f16x2 v[16];
    for (int i = 0; i < 16; ++i) { v[i][0] = (_Float16)(threadIdx.x + i); v[i][1] = (_Float16)(i); }
    const f16x2 lim = {(_Float16)0.5f, (_Float16)0.25f};
    for (int it = 0; it < iters; ++it) {
        if (MODE & 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[i], 0, 0, 0);
        }
        if (MODE & 2) {
#pragma unroll
            for (int r = 0; r < 10; ++r)
#pragma unroll
                for (int i = 0; i < 16; ++i) v[i] = __builtin_elementwise_max(v[i] + lim, lim);
        }
    }
    float s = 0.f;
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][3];
    for (int i = 0; i < 16; ++i) s += (float)v[i][0] + (float)v[i][1];
    if (s == 12345.678f) out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}
extern "C" __global__ void __launch_bounds__(256) OverlapMatrix(float* out, int iters) { body<1>(out, iters); }
extern "C" __global__ void __launch_bounds__(256) OverlapVector(float* out, int iters) { body<2>(out, iters); }
extern "C" __global__ void __launch_bounds__(256) OverlapBoth(float* out, int iters) { body<3>(out, iters); }
"""


def mfma_valu_overlap(device, iters=2000):
    """Cycles per v_mfma_f32_16x16x32_f16 and per packed vector instruction of a SIMD that runs only the one or the
    other, and the time of both streams together against their sum: what a layer of the fused kernels, whose matrix
    results pass through conversions and activations on the vector ALUs, can at best overlap. 4 wavefronts per SIMD."""
    import ctypes
    import torch
    import qmlp
    lib = qmlp._lib.lib
    lib.qmlp_hip_last_error.restype = ctypes.c_char_p

    def ok(rc):
        if rc != 0:
            raise RuntimeError(lib.qmlp_hip_last_error().decode())

    kernels = [b"OverlapMatrix", b"OverlapVector", b"OverlapBoth"]
    module = ctypes.c_void_p()
    names = (ctypes.c_char_p * len(kernels))(*kernels)
    opts = (ctypes.c_char_p * 6)(b"-O3", b"-I/opt/rocm/include", b"-Xclang", b"-target-feature", b"-Xclang", b"-packed-fp32-ops")
    ok(lib.qmlp_hip_module_compile(OVERLAP_SOURCE.encode(), b"mfma_valu_overlap.hip", None, None, 0, names, len(kernels), opts, 6,
                                   None, ctypes.byref(module), None))
    ok(lib.qmlp_hip_module_load(module))
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    waves_per_simd = 4
    blocks = cus * waves_per_simd
    out = torch.zeros(blocks * 256, dtype=torch.float32, device=device)
    stream = qmlp._lib.current_stream(device)
    ms = {}
    for name in kernels:
        fn, lowered = ctypes.c_void_p(), ctypes.c_char_p()
        ok(lib.qmlp_hip_module_lowered_name(module, name, ctypes.byref(lowered)))
        ok(lib.qmlp_hip_module_get_function(module, lowered, ctypes.byref(fn)))
        a_out, a_iters = ctypes.c_void_p(out.data_ptr()), ctypes.c_int(iters)
        args = (ctypes.c_void_p * 2)(ctypes.addressof(a_out), ctypes.addressof(a_iters))
        ok(lib.qmlp_hip_launch(fn, blocks, 256, 0, stream, args))
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        ok(lib.qmlp_hip_launch(fn, blocks, 256, 0, stream, args))
        stop.record()
        torch.cuda.synchronize()
        ms[name.decode()] = start.elapsed_time(stop)
    ok(lib.qmlp_hip_module_destroy(module))
    per_simd = lambda t, n: t * 1e-3 * 2.4e9 / iters / waves_per_simd / n
    return {"waves_per_simd": waves_per_simd, "launch_ms": ms,
            "clocks_per_mfma_16x16x32_f16": per_simd(ms["OverlapMatrix"], 32),
            "clocks_per_packed_valu": per_simd(ms["OverlapVector"], 320),
            "both_over_sum": ms["OverlapBoth"] / (ms["OverlapMatrix"] + ms["OverlapVector"]),
            "both_over_larger": ms["OverlapBoth"] / max(ms["OverlapMatrix"], ms["OverlapVector"]),
            # what the matrix cores of the device deliver with this instruction when nothing else runs
            "mfma_only_tflops": 16384.0 * 32 * iters * blocks * 4 / (ms["OverlapMatrix"] * 1e-3) / 1e12,
            "clock_hz_assumed": 2.4e9}


LDS_SOURCE = r"""
#include <hip/hip_runtime.h>
// Reference patterns for reading the LDS bank-conflict counter: every kernel issues the same number
// of LDS read instructions per wavefront; only the addresses differ.
//   0: 16 bytes per lane at consecutive addresses (how the layer weights are read as matrix-core operands)
//   1:  4 bytes per lane at consecutive addresses (no conflicts by construction)
//   2:  4 bytes per lane, 128 bytes apart (every lane on the same bank)
//   3:  8 bytes per lane, rows of 64 bytes rotated as the staging rows of 32 channels are (arrays.h)
//   4:  8 bytes per lane at consecutive addresses
template <int KIND>
__device__ void body(float* out, int iters)
{
    __shared__ __attribute__((aligned(16))) float s[16384];
    for (int i = threadIdx.x; i < 16384; i += blockDim.x) s[i] = 1.f;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float acc = 0.f;
    for (int it = 0; it < iters; ++it) {
        int base = ((it * 4 + wave) & 7) * 2048;
        asm volatile("" : "+v"(base));                     // keeps the read inside the loop
        if (KIND == 0) { const float4 v = reinterpret_cast<const float4*>(s)[(base >> 2) + lane]; acc += v.x + v.y + v.z + v.w; }
        if (KIND == 4) { const float2 v = reinterpret_cast<const float2*>(s)[(base >> 1) + lane]; acc += v.x + v.y; }
        if (KIND == 1) acc += s[base + lane];
        if (KIND == 2) acc += s[(base + lane * 32) & 16383];
        if (KIND == 3) {
            const int r = lane & 15, g = lane >> 4;          // 16 rows x 4 chunks of 8 bytes, as one operand read
            const int row = r, chunk = (g + 2 * (row / 4) + (row >> 4)) & 7;
            const float2 v = *reinterpret_cast<const float2*>(s + base + row * 16 + chunk * 2);
            acc += v.x + v.y;
        }
    }
    if (acc == 12345.f) out[blockIdx.x * blockDim.x + threadIdx.x] = acc;
}
extern "C" __global__ void __launch_bounds__(256) LdsRead16Consecutive(float* out, int iters) { body<0>(out, iters); }
extern "C" __global__ void __launch_bounds__(256) LdsRead4Consecutive(float* out, int iters) { body<1>(out, iters); }
extern "C" __global__ void __launch_bounds__(256) LdsRead4SameBank(float* out, int iters) { body<2>(out, iters); }
extern "C" __global__ void __launch_bounds__(256) LdsRead8RotatedRows(float* out, int iters) { body<3>(out, iters); }
extern "C" __global__ void __launch_bounds__(256) LdsRead8Consecutive(float* out, int iters) { body<4>(out, iters); }
"""


def lds_calibration(device, repeats=3):
    """Launches the reference LDS read patterns (for a profiler run that collects
    SQ_LDS_BANK_CONFLICT and SQ_ACTIVE_INST_LDS next to the kernels of the library)."""
    import ctypes
    import torch
    import qmlp
    lib = qmlp._lib.lib
    lib.qmlp_hip_last_error.restype = ctypes.c_char_p

    def ok(rc):
        if rc != 0:
            raise RuntimeError(lib.qmlp_hip_last_error().decode())

    kernels = [b"LdsRead16Consecutive", b"LdsRead4Consecutive", b"LdsRead4SameBank", b"LdsRead8RotatedRows",
               b"LdsRead8Consecutive"]
    module = ctypes.c_void_p()
    names = (ctypes.c_char_p * len(kernels))(*kernels)
    opts = (ctypes.c_char_p * 6)(b"-O3", b"-I/opt/rocm/include", b"-Xclang", b"-target-feature", b"-Xclang", b"-packed-fp32-ops")
    ok(lib.qmlp_hip_module_compile(LDS_SOURCE.encode(), b"lds_calibration.hip", None, None, 0, names, len(kernels), opts, 6,
                                   None, ctypes.byref(module), None))
    ok(lib.qmlp_hip_module_load(module))
    out = torch.zeros(1024 * 256, dtype=torch.float32, device=device)
    stream = qmlp._lib.current_stream(device)
    result = {}
    for name in kernels:
        fn, lowered = ctypes.c_void_p(), ctypes.c_char_p()
        ok(lib.qmlp_hip_module_lowered_name(module, name, ctypes.byref(lowered)))
        ok(lib.qmlp_hip_module_get_function(module, lowered, ctypes.byref(fn)))
        a_out, a_iters = ctypes.c_void_p(out.data_ptr()), ctypes.c_int(4096)
        args = (ctypes.c_void_p * 2)(ctypes.addressof(a_out), ctypes.addressof(a_iters))
        ok(lib.qmlp_hip_launch(fn, 1024, 256, 0, stream, args))
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(repeats):
            ok(lib.qmlp_hip_launch(fn, 1024, 256, 0, stream, args))
        stop.record()
        torch.cuda.synchronize()
        result[name.decode()] = {"launch_ms": start.elapsed_time(stop) / repeats, "lds_reads_per_wave": 4096}
    ok(lib.qmlp_hip_module_destroy(module))
    return result


def request_ceiling(gather, points, requests_per_point, l2_miss_fraction, launch_ms):
    """Prices the line requests of a gathering launch with the two measured rates."""
    hit = points * requests_per_point * (1.0 - l2_miss_fraction) / gather["l2_hit"]["requests_per_s"]
    miss = points * requests_per_point * l2_miss_fraction / gather["l2_miss"]["requests_per_s"]
    bound_ms = 1e3 * (hit + miss)
    return {"requests_per_point": requests_per_point, "l2_miss_fraction": l2_miss_fraction,
            "l2_hit_requests_per_s": gather["l2_hit"]["requests_per_s"],
            "l2_miss_requests_per_s": gather["l2_miss"]["requests_per_s"],
            "bound_ms": bound_ms, "frac_of_bound": bound_ms / launch_ms}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg2-inference",
                    choices=sorted(WORKLOADS) + ["layer-gemm", "reference-grid", "gather-ceiling", "gather-patterns", "mfma-valu-overlap",
                                              "lds-calibration", "all"],
                    help="layer-gemm: the layers of the hash-grid network on their own; reference-grid: the reference's "
                         "own benchmark networks; gather-ceiling: request rate of random gathers; all: every workload")
    ap.add_argument("--points", type=int, default=0, help="override the number of points")
    ap.add_argument("--case", default="", help="layer-gemm / reference-grid: only the case of this name "
                                               "(e.g. cfg2_mlp_cached_input, '64 x 4')")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-train", action="store_true", help="skip the secondary train-step measurement")
    ap.add_argument("--no-ordered", action="store_true", help="skip the secondary measurements on ordered batches")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy a few times (reference kernel for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path shards by points and nothing here uses a second "
                 "device; run with --gpus 1")

    import torch
    import qmlp
    import baseline_configs as bc
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    qmlp.set_log_level("error")
    device = torch.device("cuda:0")

    if args.copy_calibration:
        src = torch.empty((256 << 20) // 4, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    head = {"metric": "points/sec fused hashgrid+MLP inference & train step; % MFMA/HBM roofline", "unit": "points/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f16", "data": "synthetic"}
    if args.workload == "layer-gemm":
        report = layer_gemm_report(device, args.steps, args.warmup, args.case, args.points or (1 << 20))
        ms = next(iter(report.values()))["launch_ms"]
        print(json.dumps(dict(head, value=(args.points or (1 << 20)) / (ms * 1e-3), ms_per_step=ms,
                              config={"workload": "layer-gemm", "points": args.points or (1 << 20),
                                      "case": args.case or "all (value: the first)"},
                              mfma=dict(peak_tflops=MFMA_FP16_PEAK_TFLOPS, layer_gemm=report))))
        return
    if args.workload == "reference-grid":
        rows = reference_grid(device, args.steps, args.warmup, args.case)
        print(json.dumps(dict(head, value=rows[-1]["points"] / (rows[-1]["inference_ms"] * 1e-3),
                              ms_per_step=rows[-1]["inference_ms"],
                              config={"workload": "reference-grid", "points": rows[-1]["points"],
                                      "network": rows[-1]["network"] + " (value); all six under networks"},
                              networks=rows)))
        return
    if args.workload == "gather-ceiling":
        g = gather_ceiling(device)
        print(json.dumps(dict(head, value=g["l2_hit"]["requests_per_s"], unit="line requests/s",
                              ms_per_step=g["l2_hit"]["launch_ms"],
                              config={"workload": "gather-ceiling", "loads": 2048 * 256 * 64}, gather=g)))
        return
    if args.workload == "gather-patterns":
        rows = gather_patterns(device)
        print(json.dumps(dict(head, value=1.0 / (rows[0]["launch_ms"] * 1e-3), unit="launches/s", ms_per_step=rows[0]["launch_ms"],
                              config={"workload": "gather-patterns"}, patterns=rows)))
        return
    if args.workload == "mfma-valu-overlap":
        r = mfma_valu_overlap(device)
        print(json.dumps(dict(head, value=r["mfma_only_tflops"], unit="TFLOP/s", ms_per_step=r["launch_ms"]["OverlapMatrix"],
                              config={"workload": "mfma-valu-overlap"}, overlap=r)))
        return
    if args.workload == "lds-calibration":
        r = lds_calibration(device)
        print(json.dumps(dict(head, value=1.0 / (r["LdsRead16Consecutive"]["launch_ms"] * 1e-3), unit="launches/s",
                              ms_per_step=r["LdsRead16Consecutive"]["launch_ms"],
                              config={"workload": "lds-calibration"}, lds=r)))
        return
    if args.workload == "all":
        g = gather_ceiling(device)
        summary = {"gather": g, "layer_gemm": layer_gemm_report(device, args.steps, args.warmup),
                   "reference_grid": reference_grid(device, args.steps, args.warmup), "workloads": {}}
        for name, (cid, trn) in sorted(WORKLOADS.items()):
            cc = bc.CONFIGS[cid]
            cs = build_case(cid, cc["points"], device)
            el, lms = (run_train if trn else run_inference)(cs, args.steps, args.warmup)
            bpp = cc["gather_bytes_per_point"] + cc["io_bytes_per_point"]
            summary["workloads"][name] = {
                "points": cc["points"], "ms_per_step": 1e3 * el / args.steps, "launch_ms": lms,
                "points_per_s": args.steps * cc["points"] / el,
                "hbm_frac": bpp * cc["points"] / (lms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                "mfma_frac": cc["flop_per_point"] * cc["points"] / (lms * 1e-3) / 1e12 / MFMA_FP16_PEAK_TFLOPS}
            del cs
        w = summary["workloads"]["cfg2-inference"]
        print(json.dumps(dict(head, value=w["points_per_s"], ms_per_step=w["ms_per_step"],
                              config={"workload": "all (value: cfg2-inference)"}, **summary)))
        return

    cfg_id, train = WORKLOADS[args.workload]
    c = bc.CONFIGS[cfg_id]
    n = args.points or c["points"]
    case = build_case(cfg_id, n, device)
    elapsed, launch_ms = (run_train if train else run_inference)(case, args.steps, args.warmup)
    value = args.steps * n / elapsed

    # algorithmic bytes of one launch: table entries gathered (and scattered) + input + output
    bytes_per_point = c["gather_bytes_per_point"] + c["io_bytes_per_point"]
    achieved_gbs = bytes_per_point * n / (launch_ms * 1e-3) / 1e9
    flops = c["flop_per_point"] * n / (launch_ms * 1e-3)
    traffic = None
    m = MEASURED_TRAFFIC_BYTES.get(args.workload)
    if m is not None and m["points"] == n and m["kernels"] == device_code_hash(case["net"]):
        # same form as "achieved": bytes of one launch over the launch duration measured now
        traffic = (m["fetch"] + m["write"]) / (launch_ms * 1e-3) / 1e9
    result = {
        "metric": "points/sec fused hashgrid+MLP inference & train step; % MFMA/HBM roofline",
        "value": value, "unit": "points/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": 1e3 * elapsed / args.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": args.workload, "points": n, "spec": "BASELINE config %d" % cfg_id,
                   "network": "x".join(str(l["n_out"]) for l in c["cfg"]["network"]),
                   "encodings": [e["id"] for e in c["cfg"]["encodings"]]},
        "roofline": {"bound": "hbm", "achieved": achieved_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved_gbs / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_bytes_per_launch": None if traffic is None else m["fetch"] + m["write"],
                     "algorithmic_bytes_per_launch": bytes_per_point * n,
                     "kernel": "NetworkKernelInferenceAndForward" if not train else "train step (4-5 kernels)",
                     "launch_ms": launch_ms, "algorithmic_bytes_per_point": bytes_per_point},
        "mfma": {"achieved_tflops": flops / 1e12, "peak_tflops": MFMA_FP16_PEAK_TFLOPS,
                 "frac": flops / 1e12 / MFMA_FP16_PEAK_TFLOPS, "flop_per_point": c["flop_per_point"]},
        "kernel_cache": dict(zip(("compiled", "disk_hits"), qmlp._lib.kernel_cache_stats())),
        "device_code": device_code_hash(case["net"]),
    }
    if not train and cfg_id == 2:
        # the two north-star fractions of the hash-grid network: its layer GEMMs on their own, and
        # the launch against the request rate of random gathers measured in this same run (64 line
        # requests per point: 16 levels x 4 pairs of corners; 3% of them miss the L2, see profiles/)
        result["mfma"]["layer_gemm"] = layer_gemm_report(device, max(10, args.steps // 2), args.warmup)
        # (the duration of the kernel as a profiler's kernel trace sees it: launches back to back)
        result["mfma"]["layer_gemm_frac"] = result["mfma"]["layer_gemm"]["cfg2_mlp_cached_input"]["frac_back_to_back"]
        result["roofline"]["request_ceiling"] = request_ceiling(gather_ceiling(device), n, 64.0, 0.03, launch_ms)
        # What binds the launch: every gather instruction of a level with more cells than the batch has points brings
        # 64 lines of 128 bytes from the L2 (4 pairs of corners per point and level, 16 levels), of which 8 bytes
        # each are used. Between the L2 of a die and a compute unit pass 64 bytes per clock (a published figure of the
        # architecture: 2 KiB per clock and die over its 32 compute units); the clock is taken as 2.4 GHz.
        cus = torch.cuda.get_device_properties(device).multi_processor_count
        l2_bytes = 64.0 * 128.0 * n
        l2_peak_gbs = cus * 64.0 * 2.4e9 / 1e9
        result["roofline"]["l2_lines"] = {"bound": "l2", "lines_per_point": 64, "line_bytes": 128,
                                          "achieved": l2_bytes / (launch_ms * 1e-3) / 1e9, "peak": l2_peak_gbs, "unit": "GB/s",
                                          "frac": l2_bytes / (launch_ms * 1e-3) / 1e9 / l2_peak_gbs,
                                          "used_bytes_per_line": 8}
    if not train and cfg_id == 2 and not args.no_ordered:
        # the same launch on a batch that the library orders first, and on one that arrives ordered
        result["ordered_batch"] = ordered_batch_report(cfg_id, n, device, max(10, args.steps // 2), args.warmup)
    if not train and cfg_id == 2 and not args.no_train:
        # the train step of the same network at its own batch size
        c3 = bc.CONFIGS[3]
        case3 = build_case(3, c3["points"], device)
        # at least 20 timed steps after at least 10 untimed ones and 50 ms: the tables of this case were just
        # generated on the host, and a device that idled that long starts its first launches below its clocks
        steps3 = max(20, args.steps // 2)
        e3, l3 = run_train(case3, steps3, max(10, args.warmup), warmup_seconds=0.05)
        b3 = c3["gather_bytes_per_point"] + c3["io_bytes_per_point"]
        # (the same step without the gradients with respect to the input points, which training the network and
        # the grid does not need: no second gather)
        e3p, _ = run_train(case3, steps3, max(10, args.warmup), input_gradients=False, warmup_seconds=0.05)
        result["train_step"] = {"workload": "cfg3-train", "points": c3["points"], "steps": steps3,
                                "launch_ms": l3,
                                "ms_per_step_without_input_gradients": 1e3 * e3p / steps3,
                                "value": steps3 * c3["points"] / e3, "unit": "points/s", "ms_per_step": 1e3 * e3 / steps3,
                                "hbm_frac": b3 * c3["points"] / (l3 * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                "mfma_frac": c3["flop_per_point"] * c3["points"] / (l3 * 1e-3) / 1e12 / MFMA_FP16_PEAK_TFLOPS}
        del case3
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(case, train)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
