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
# with the commands is kept under profiles/. Workloads without a counter run report null.
MEASURED_TRAFFIC_BYTES = {
    "cfg2-inference": {"points": 1 << 20, "fetch": 106149.0 * 1024 * 2.0, "write": 8192.0 * 1024 * 1.0},
}

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
    from qmlp import baseline_configs as bc
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


def time_steps(step, steps, warmup):
    """W untimed steps, then exactly K timed ones between two synchronisations. Every timed
    step is also bracketed by HIP events on the launch stream for the per-launch duration."""
    import torch
    for _ in range(warmup):
        step()
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


def run_train(case, steps, warmup):
    import torch
    from qmlp import baseline_configs as bc
    net, x, params, enc = case["net"], case["x"], case["params"], case["enc_params"]
    cfg_id = case["cfg_id"]
    n = x.shape[0]
    target = torch.from_numpy(bc.make_targets(cfg_id, case["X_np"])).to(x.device)
    flags = 1 | 2 | (4 if any(e is not None for e in enc) else 0)
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
        adj_out = (out - target) * (2.0 / out.numel())
        net.adjoint_raw(x, adj_out, flags, tmp, params, enc, grad_network=grad_net, grad_encodings=grad_enc,
                        adj_input=adj_in)

    step()
    torch.cuda.synchronize()
    return time_steps(step, steps, warmup)


def cpu_baseline(case, train, min_seconds=10.0):
    """The CPU oracle (an fp32 port of the reference's Eigen test evaluation, OpenMP over
    points) on the same workload, repeated until at least min_seconds of CPU work."""
    import numpy as np
    import qmlp_oracle as qo
    from qmlp import baseline_configs as bc
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg2-inference", choices=sorted(WORKLOADS))
    ap.add_argument("--points", type=int, default=0, help="override the number of points")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-train", action="store_true", help="skip the secondary train-step measurement")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy a few times (reference kernel for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path shards by points and nothing here uses a second "
                 "device; run with --gpus 1")

    import torch
    import qmlp
    from qmlp import baseline_configs as bc
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
    if m is not None and m["points"] == n:
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
    }
    if not train and cfg_id == 2 and not args.no_train:
        # the train step of the same network at its own batch size
        c3 = bc.CONFIGS[3]
        case3 = build_case(3, c3["points"], device)
        steps3 = max(5, args.steps // 2)
        e3, l3 = run_train(case3, steps3, min(args.warmup, 3))
        b3 = c3["gather_bytes_per_point"] + c3["io_bytes_per_point"]
        result["train_step"] = {"workload": "cfg3-train", "points": c3["points"], "steps": steps3,
                                "value": steps3 * c3["points"] / e3, "unit": "points/s", "ms_per_step": 1e3 * e3 / steps3,
                                "hbm_frac": b3 * c3["points"] / (l3 * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                "mfma_frac": c3["flop_per_point"] * c3["points"] / (l3 * 1e-3) / 1e12 / MFMA_FP16_PEAK_TFLOPS}
        del case3
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(case, train)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
