"""Shared pieces of the parity tests: run a specification through the C ABI on the GPU and
through the CPU oracle on the same seeded inputs, and compare."""
import json
import os

import numpy as np
import pytest
import torch

import qmlp
import qmlp_oracle as qo
import baseline_configs as bc

REL, ABS = 1e-2, 1e-3          # tolerance of the fp16 path against the fp32 oracle
FLAG_INPUT, FLAG_WEIGHTS, FLAG_ENC = 1, 2, 4


def require_gpu(encoding_cfg=None, adjoint_modes=(3,)):
    """For tests that do not go through Case. In a CPU cache-warming pass the standalone
    kernels of encoding_cfg are compiled into the in-tree kernel cache, then the test stops."""
    if os.environ.get("QMLP_WARM_CACHE") and encoding_cfg is not None:
        import json
        import qmlp
        enc = qmlp.Encoding(json.dumps(encoding_cfg))
        enc.precompile(0)
        for m in adjoint_modes:
            enc.precompile(m)
        pytest.skip("kernel cache warmed")
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")


def warm_cache(*cfgs):
    """In a CPU cache-warming pass: compiles the kernels of all these specifications into the
    in-tree kernel cache and stops the test (a test that builds several networks calls this first,
    because the first Case of a warming pass ends the test)."""
    if os.environ.get("QMLP_WARM_CACHE"):
        for cfg in cfgs:
            qmlp.Network(json.dumps(cfg)).precompile(7)
        pytest.skip("kernel cache warmed")


def identity_cfg(n_in, widths, acts, biases, extra_acts=()):
    return {"num_inputs": n_in, "num_outputs": widths[-1],
            "activation_specification": ["qmlp/builtin-activations.json", *extra_acts],
            "encodings": [{"id": "Identity", "start_in": 0, "n_in": n_in}],
            "network": [{"n_out": w, "bias": b, "activation": a} for w, a, b in zip(widths, acts, biases)]}


def random_parameters(onet, rng, scale=None):
    """fp16-representable parameters: U(+-1/sqrt(C_in padded)) like initializeInferenceParameters."""
    flat = np.zeros(onet.num_parameters, dtype=np.float32)
    for l in onet.layers:
        bound = scale if scale is not None else 1.0 / np.sqrt(l["cin"])
        n = l["cin"] * l["cout"]
        flat[l["w_start"]:l["w_start"] + n] = rng.uniform(-bound, bound, n)
        if l["bias"]:
            flat[l["b_start"]:l["b_start"] + l["cout"]] = rng.uniform(-bound, bound, l["cout"])
    return qo.round_half(flat)


class Case:
    """One network on both sides."""

    def __init__(self, cfg, oracle_activations=None):
        self.cfg = cfg
        self.cfg_json = json.dumps(cfg)
        self.oracle = qo.Network(cfg, oracle_activations)
        self.net = qmlp.Network(self.cfg_json)
        assert self.net.num_network_parameters() == self.oracle.num_parameters
        if os.environ.get("QMLP_WARM_CACHE"):
            # CPU-only pass over the GPU tests: compile this network's kernels into the
            # in-tree kernel cache (hipRTC needs no GPU) and stop there
            self.net.precompile(7)
            pytest.skip("kernel cache warmed")
        self.tables_np = [None] * len(self.oracle.encodings)
        self.params_np = None

    def set_parameters(self, flat_f32):
        self.params_np = np.asarray(flat_f32, dtype=np.float32)
        self.oracle.set_parameters(self.params_np)
        self.params = torch.from_numpy(self.params_np.astype(np.float16)).cuda()

    def set_table(self, i, table_f32):
        enc = self.net.encoding(i)
        dt = enc.parameter_dtype(False)
        t = torch.from_numpy(np.asarray(table_f32, dtype=np.float32)).to(dt)
        self.tables_np[i] = t.to(torch.float32).numpy()          # what the device really stores
        self.oracle.set_table(i, self.tables_np[i])
        self._tables = getattr(self, "_tables", {})
        self._tables[i] = t.cuda()

    def encoding_parameters(self):
        out = []
        for i in range(self.net.num_encodings()):
            out.append(getattr(self, "_tables", {}).get(i))
        return out

    def gpu_inference(self, X):
        x = torch.from_numpy(X).cuda()
        out = self.net.inference(x, self.params, self.encoding_parameters())
        torch.cuda.synchronize()
        return out.cpu().numpy()

    def gpu_train(self, X, adj, flags):
        x = torch.from_numpy(X).cuda()
        a = torch.from_numpy(adj).cuda()
        out, tmp = self.net.forward_raw(x, self.params, self.encoding_parameters(), flags)
        adj_x, gnet, genc = self.net.adjoint_raw(x, a, flags, tmp, self.params, self.encoding_parameters())
        torch.cuda.synchronize()
        return dict(out=out.cpu().numpy(),
                    adj_x=None if adj_x is None else adj_x.cpu().numpy(),
                    grads=None if gnet is None else gnet.cpu().numpy(),
                    table_grads=[None if g is None else g.cpu().numpy() for g in genc])


def assert_close(actual, expected, what, rel=REL, abs_=ABS, allowed_fraction=0.0):
    frac, worst = qo.compare(actual, expected, rel, abs_)
    assert frac <= allowed_fraction, (
        "%s: %.4f%% of the entries exceed rel %g / abs %g (worst ratio %.2f)" % (what, 100 * frac, rel, abs_, worst))


def check_gradients(case, X, adj, flags, got, kinks=False, what="", kink_fraction=0.02):
    """Gradients of the fp16 device path against both oracles.

    fp32 oracle: rel 1e-2 / abs 1e-3, the absolute part relative to the largest entry when
    that exceeds one (gradients are sums over the batch). Networks with ReLU have kinks: an
    fp16 rounding of a pre-activation next to zero switches a whole unit for that point, so a
    small fraction of entries (2%; with only 35 points one point is already 3%) may exceed. The oracle that rounds where the device rounds
    (round_mode 1) has to be matched twice as tightly (rel 5e-3 / abs 5e-4) in every case;
    what remains there is the last-bit difference of the half-precision sin/exp intrinsics."""
    ref0 = case.oracle.backward(X, adj, flags, round_mode=0)
    ref1 = case.oracle.backward(X, adj, flags, round_mode=1)
    pairs = []
    if flags & FLAG_INPUT:
        pairs.append(("input gradients", got["adj_x"], ref0["adj_x"], ref1["adj_x"]))
    if flags & FLAG_WEIGHTS:
        pairs.append(("weight gradients", got["grads"], ref0["grads"], ref1["grads"]))
    if flags & FLAG_ENC:
        for i, g in enumerate(got["table_grads"]):
            if g is not None:
                pairs.append(("grid gradients %d" % i, g, ref0["table_grads"][i], ref1["table_grads"][i]))
    for name, a, e0, e1 in pairs:
        s = max(1.0, float(np.abs(e0).max()))
        assert_close(a / s, e0 / s, what + name + " vs fp32 oracle", allowed_fraction=kink_fraction if kinks else 0.0)
        assert_close(a / s, e1 / s, what + name + " vs rounding oracle", rel=5e-3, abs_=5e-4,
                     allowed_fraction=2e-3 if kinks else 0.0)
    return ref0


def baseline_case(cfg_id, table_scale=None, seed=None, options=None):
    """A Case for BASELINE config cfg_id with its seeded parameters (and tables); options are
    added to the "options" of the specification."""
    c = bc.CONFIGS[cfg_id]
    seed = bc.PARAMETER_SEED[cfg_id] if seed is None else seed
    rng = np.random.default_rng(seed)
    cfg = json.loads(json.dumps(c["cfg"]))
    if options:
        cfg.setdefault("options", {}).update(options)
    case = Case(cfg, bc.ORACLE_ACTIVATIONS)
    case.set_parameters(bc.make_parameters(cfg_id, rng).astype(np.float32))
    for i, e in enumerate(case.oracle.encodings):
        if e[0] == "hashgrid":
            case.set_table(i, bc.make_table(cfg_id, e[1].n_params, rng, table_scale))
    return case, rng
