"""Pins the CPU oracle against things it does not itself define: hand-computed known
answers, torch library routines (linear + autograd, grid_sample), an independent
float64 brute-force interpolator written from the hashing formula, invariants, and
finite differences. Runs without a GPU."""
import itertools
import json
import os

import numpy as np
import pytest
import torch

import qmlp_oracle as qo

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
PRIMES = [1, 43857811, 83857661, 73856093, 19349663, 834927]


# ------------------------------------------------------------------ helpers
def grid_spec(dim, levels=1, feat=4, log2=-1, rmin=2, rmax=16, mode="concat", bmin=None, bsize=None,
              start=0):
    return {"id": "HashGrid", "start_in": start, "n_in": dim, "n_levels": levels,
            "n_features_per_level": feat, "log2_hashmap_size": log2, "min_resolution": rmin,
            "max_resolution": rmax, "combination_mode": mode,
            "bounding_box_min": bmin if bmin is not None else [0.0] * dim,
            "bounding_box_size": bsize if bsize is not None else [1.0] * dim}


def brute_force_grid(g, table, x):
    """Independent float64 multilinear interpolation over itertools corners."""
    table = np.asarray(table, dtype=np.float64)
    N, D, F = x.shape[0], g.dim, g.n_feat
    lt = g.level_table()
    out = np.zeros((N, g.num_outputs))
    bmin = np.array(g.cfg["bounding_box_min"], dtype=np.float32)
    binv = (np.float32(1) / np.array(g.cfg["bounding_box_size"], dtype=np.float32))
    for n in range(N):
        pos = ((x[n, g.start_in:g.start_in + D].astype(np.float32) - bmin) * binv).astype(np.float32)
        for l, (R, hashed, off, hsize) in enumerate(lt):
            p = (pos * np.float32(R - 1)).astype(np.float32)
            lo = np.clip(np.trunc(p).astype(np.int64), 0, R - 1)
            hi = np.clip(np.trunc(p).astype(np.int64) + 1, 0, R - 1)
            fr = p.astype(np.float64) - lo
            feat = np.zeros(F)
            for bits in itertools.product((0, 1), repeat=D):
                c = [hi[d] if bits[d] else lo[d] for d in range(D)]
                w = np.prod([fr[d] if bits[d] else 1 - fr[d] for d in range(D)])
                if hashed:
                    h = 0
                    for d in range(D):
                        h ^= (int(c[d]) * PRIMES[d]) & 0xFFFFFFFF
                    idx = h % hsize
                else:
                    idx = 0
                    for d in range(D):
                        idx = idx * R + int(c[d])
                feat += w * table[off + idx * F: off + idx * F + F]
            if g.combination == qo.CONCAT:
                out[n, l * F:(l + 1) * F] = feat
            else:
                out[n, :F] += feat
    return out


# ------------------------------------------------------------------ fp16 rounding
def test_round_half_matches_numpy():
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.uniform(-70000, 70000, 2000), rng.uniform(-1, 1, 2000), rng.uniform(-1e-4, 1e-4, 2000),
        rng.uniform(-1e-7, 1e-7, 500), [0.0, -0.0, 65504.0, 65519.9, 65520.0, 6.1035e-5, 6.0e-8,
                                         2.98e-8, 2.9802322e-8, 1.0009765625, 1.00048828125]
    ]).astype(np.float32)
    mine = np.array([qo.lib().qo_round_half(float(v)) for v in vals], dtype=np.float32)
    with np.errstate(over="ignore"):
        ref = vals.astype(np.float16).astype(np.float32)
    assert np.array_equal(mine, ref)


# ------------------------------------------------------------------ level table
def test_level_table_golden_cfg2():
    gold = json.load(open(os.path.join(GOLDEN, "cfg2_level_table.json")))
    g = qo.HashGrid(gold["spec"])
    got = [[r, int(h), off] for (r, h, off, _) in g.level_table()]
    assert got == gold["levels"]
    assert g.n_params == gold["total_parameters"]
    assert all(hs == (1 << 19) for (_, h, _, hs) in g.level_table() if h)


@pytest.mark.parametrize("dim,levels,feat,log2,rmin,rmax", [
    (3, 16, 2, 19, 16, 4096), (2, 5, 4, -1, 16, 2048), (4, 1, 8, -1, 32, 32), (1, 3, 1, 4, 2, 64),
    (6, 4, 2, 10, 2, 9)])
def test_level_table_invariants(dim, levels, feat, log2, rmin, rmax):
    g = qo.HashGrid(grid_spec(dim, levels, feat, log2, rmin, rmax))
    lt = g.level_table()
    assert lt[0][0] == rmin
    assert lt[-1][0] in (rmax, rmax - 1) or levels == 1   # floor of an inexact pow
    assert all(a[0] <= b[0] for a, b in zip(lt, lt[1:]))
    off = 0
    for (R, hashed, o, hs) in lt:
        assert o == off
        dense_ok = log2 <= 0 or R ** dim <= (1 << log2)
        assert hashed == (not dense_ok)
        off += (hs if hashed else R ** dim) * feat
    assert g.n_params == off


def test_default_bounding_box_is_centered_unit_cube():
    cfg = grid_spec(2)
    del cfg["bounding_box_min"], cfg["bounding_box_size"]
    g = qo.HashGrid(cfg)
    assert list(g.s.bb_min)[:2] == [-0.5, -0.5] and list(g.s.bb_inv)[:2] == [1.0, 1.0]


# ------------------------------------------------------------------ indices
def _u32(vals):
    import ctypes
    return (ctypes.c_uint32 * len(vals))(*vals)


def test_hash_known_answers():
    L = qo.lib()
    assert L.qo_index_hash(3, _u32([0, 0, 0])) == 0
    assert L.qo_index_hash(3, _u32([1, 1, 1])) == (1 ^ 43857811 ^ 83857661)
    assert L.qo_index_hash(1, _u32([12345])) == 12345
    assert L.qo_index_hash(2, _u32([7, 3])) == (7 ^ ((3 * 43857811) & 0xFFFFFFFF))
    # uint32 wrap-around of the product
    assert L.qo_index_hash(3, _u32([4094, 4094, 4094])) == \
        (4094 ^ ((4094 * 43857811) & 0xFFFFFFFF) ^ ((4094 * 83857661) & 0xFFFFFFFF))
    v = [5, 6, 7, 8, 9, 10]
    h = 0
    for d in range(6):
        h ^= (v[d] * PRIMES[d]) & 0xFFFFFFFF
    assert L.qo_index_hash(6, _u32(v)) == h


def test_dense_index_last_coordinate_fastest_and_bijective():
    L = qo.lib()
    assert L.qo_index_dense(3, _u32([2, 1, 0]), 5) == (2 * 5 + 1) * 5 + 0
    assert L.qo_index_dense(3, _u32([0, 0, 1]), 5) == 1
    seen = {L.qo_index_dense(3, _u32(list(c)), 3) for c in itertools.product(range(3), repeat=3)}
    assert seen == set(range(27))
    seen4 = {L.qo_index_dense(4, _u32(list(c)), 2) for c in itertools.product(range(2), repeat=4)}
    assert seen4 == set(range(16))


def test_corner_indices_in_range_and_match_brute_force_formula():
    g = qo.HashGrid(grid_spec(3, 6, 2, 8, 4, 64))
    rng = np.random.default_rng(3)
    x = rng.uniform(0, 1, (200, 3)).astype(np.float32)
    idx, w = g.corners(x)
    lt = g.level_table()
    for l, (R, hashed, off, hs) in enumerate(lt):
        size = (hs if hashed else R ** 3) * 2
        assert idx[:, l].min() >= off and idx[:, l].max() < off + size
        assert np.all((idx[:, l] - off) % 2 == 0)
    assert np.allclose(w.sum(axis=2), 1.0, atol=1e-6)            # partition of unity
    # spot-check corner 0 and corner 7 of every level against the formula
    for n in range(20):
        for l, (R, hashed, off, hs) in enumerate(lt):
            p = (x[n] * np.float32(R - 1)).astype(np.float32)
            lo = np.clip(np.trunc(p).astype(int), 0, R - 1)
            hi = np.clip(np.trunc(p).astype(int) + 1, 0, R - 1)
            for c, pos in ((0, lo), (7, hi), (1, [hi[0], lo[1], lo[2]]), (4, [lo[0], lo[1], hi[2]])):
                if hashed:
                    h = 0
                    for d in range(3):
                        h ^= (int(pos[d]) * PRIMES[d]) & 0xFFFFFFFF
                    e = h % hs
                else:
                    e = (int(pos[0]) * R + int(pos[1])) * R + int(pos[2])
                assert idx[n, l, c] == off + 2 * e


# ------------------------------------------------------------------ interpolation vs grid_sample
def _grid_sample_ref(table, x, R, C, dim):
    """torch grid_sample on params.reshape(R,..,R,C) (first coordinate slowest)."""
    t = torch.from_numpy(table.reshape(*([R] * dim), C))
    xt = torch.from_numpy(x)
    if dim == 1:
        inp = t.reshape(1, R, 1, C).permute(0, 3, 2, 1)            # (1,C,1,R)
        grid = torch.stack([xt[:, 0], torch.zeros_like(xt[:, 0])], dim=-1).reshape(1, -1, 1, 2)
        out = torch.nn.functional.grid_sample(inp, grid, mode="bilinear", align_corners=True,
                                              padding_mode="border")
        return out[0, :, :, 0].t().numpy()
    if dim == 2:
        inp = t.permute(2, 1, 0).unsqueeze(0)                       # (1,C,H=y,W=x)
        grid = xt.reshape(1, -1, 1, 2)
        out = torch.nn.functional.grid_sample(inp, grid, mode="bilinear", align_corners=True,
                                              padding_mode="border")
        return out[0, :, :, 0].t().numpy()
    inp = t.permute(3, 2, 1, 0).unsqueeze(0)                        # (1,C,D=z,H=y,W=x)
    grid = xt.reshape(1, -1, 1, 1, 3)
    out = torch.nn.functional.grid_sample(inp, grid, mode="bilinear", align_corners=True,
                                          padding_mode="border")
    return out[0, :, :, 0, 0].t().numpy()


@pytest.mark.parametrize("dim,R", [(1, 2), (2, 2), (1, 7), (2, 5), (3, 4)])
def test_dense_grid_matches_grid_sample(dim, R):
    C = 4
    g = qo.HashGrid(grid_spec(dim, 1, C, -1, R, 16, "add", [-1.0] * dim, [2.0] * dim))
    rng = np.random.default_rng(dim * 10 + R)
    table = rng.standard_normal(g.n_params).astype(np.float32)
    x = rng.uniform(-1, 1, (64, dim)).astype(np.float32)
    got = g.forward(table, x)
    want = _grid_sample_ref(table, x, R, C, dim)
    assert np.allclose(got, want, atol=2e-5)


@pytest.mark.parametrize("dim,R", [(2, 5), (3, 4)])
def test_dense_grid_gradients_match_grid_sample_autograd(dim, R):
    C = 3
    g = qo.HashGrid(grid_spec(dim, 1, C, -1, R, 16, "add", [-1.0] * dim, [2.0] * dim))
    rng = np.random.default_rng(5)
    table = rng.standard_normal(g.n_params).astype(np.float32)
    x = rng.uniform(-0.95, 0.95, (40, dim)).astype(np.float32)
    v = rng.standard_normal((40, C)).astype(np.float32)
    adj_x, grad = g.adjoint(table, x, v, res_factor=1)
    tt = torch.from_numpy(table.copy()).requires_grad_(True)
    xt = torch.from_numpy(x.copy()).requires_grad_(True)
    t = tt.reshape(*([R] * dim), C)
    if dim == 2:
        inp = t.permute(2, 1, 0).unsqueeze(0)
        out = torch.nn.functional.grid_sample(inp, xt.reshape(1, -1, 1, 2), mode="bilinear",
                                              align_corners=True, padding_mode="border")[0, :, :, 0].t()
    else:
        inp = t.permute(3, 2, 1, 0).unsqueeze(0)
        out = torch.nn.functional.grid_sample(inp, xt.reshape(1, -1, 1, 1, 3), mode="bilinear",
                                              align_corners=True, padding_mode="border")[0, :, :, 0, 0].t()
    (out * torch.from_numpy(v)).sum().backward()
    assert np.allclose(grad, tt.grad.numpy(), atol=1e-5)
    assert np.allclose(adj_x, xt.grad.numpy(), atol=1e-4)
    # the reference's formula (no (R-1) factor) is smaller by exactly (R-1)
    adj_ref, _ = g.adjoint(table, x, v, res_factor=0)
    assert np.allclose(adj_ref * (R - 1), adj_x, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("spec", [
    grid_spec(4, 1, 8, -1, 5, 5), grid_spec(3, 5, 2, 6, 3, 40), grid_spec(2, 4, 3, 5, 4, 100, "add"),
    grid_spec(5, 2, 1, 7, 2, 6), grid_spec(3, 3, 2, 6, 3, 20, "concat", [-1, 0, 2], [2, 0.5, 4], 1)])
def test_grid_matches_float64_brute_force(spec):
    g = qo.HashGrid(spec)
    rng = np.random.default_rng(11)
    table = rng.standard_normal(g.n_params).astype(np.float32)
    ncols = g.start_in + g.dim
    lo = np.array(([0] * g.start_in) + list(spec["bounding_box_min"]), dtype=np.float32)
    sz = np.array(([1] * g.start_in) + list(spec["bounding_box_size"]), dtype=np.float32)
    x = (lo + sz * rng.uniform(0, 1, (30, ncols))).astype(np.float32)
    assert np.allclose(g.forward(table, x), brute_force_grid(g, table, x), atol=3e-5)


def test_grid_constant_table_and_corner_inputs():
    g = qo.HashGrid(grid_spec(3, 3, 2, 7, 4, 30))
    rng = np.random.default_rng(2)
    x = rng.uniform(0, 1, (50, 3)).astype(np.float32)
    const = np.full(g.n_params, 0.37, dtype=np.float32)
    assert np.allclose(g.forward(const, x), 0.37, atol=1e-6)
    # inputs exactly on cell corners of the (dense) level 0 return table rows
    R = g.level_table()[0][0]
    table = rng.standard_normal(g.n_params).astype(np.float32)
    cells = rng.integers(0, R, (20, 3))
    xc = (cells / (R - 1)).astype(np.float32)
    out = g.forward(table, xc)
    rows = np.stack([table[2 * ((c[0] * R + c[1]) * R + c[2]):][:2] for c in cells])
    assert np.allclose(out[:, :2], rows, atol=2e-5)


def test_grid_extrapolates_below_and_clamps_above():
    g = qo.HashGrid(grid_spec(1, 1, 1, -1, 3, 3))
    table = np.array([1.0, 2.0, 4.0], dtype=np.float32)
    x = np.array([[-0.25], [1.5], [0.0], [1.0]], dtype=np.float32)
    # p = 2x. x=-0.25: (int)p=0 -> lo=0, hi=1, f=-0.5 -> 1*(1.5)+2*(-0.5) = 0.5 (extrapolates)
    # x=1.5: p=3 -> lo=hi=2, f=1 -> 4*(0)+4*1 = 4
    assert np.allclose(g.forward(table, x)[:, 0], [0.5, 4.0, 1.0, 4.0])


# ------------------------------------------------------------------ adjoint of the grid
def test_grid_gradient_is_the_transpose_of_forward():
    g = qo.HashGrid(grid_spec(3, 4, 2, 6, 3, 40))
    rng = np.random.default_rng(8)
    x = rng.uniform(0, 1, (100, 3)).astype(np.float32)
    theta = rng.standard_normal(g.n_params).astype(np.float32)
    dtheta = rng.standard_normal(g.n_params).astype(np.float32)
    v = rng.standard_normal((100, g.num_outputs)).astype(np.float32)
    _, grad = g.adjoint(theta, x, v, input_grads=False)
    lhs = float((g.forward(dtheta, x).astype(np.float64) * v).sum())
    rhs = float((dtheta.astype(np.float64) * grad).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs))
    # weights sum to one: per level the scattered mass equals the summed adjoint
    for l, (R, hashed, off, hs) in enumerate(g.level_table()):
        size = (hs if hashed else R ** 3) * 2
        mass = grad[off:off + size].reshape(-1, 2).sum(0)
        assert np.allclose(mass, v[:, 2 * l:2 * l + 2].sum(0), atol=1e-3)


@pytest.mark.parametrize("spec", [grid_spec(3, 3, 2, 6, 3, 20), grid_spec(4, 1, 4, -1, 6, 6),
                                  grid_spec(2, 3, 2, 5, 4, 50, "add", [-1, -2], [2, 4])])
def test_grid_input_gradient_matches_finite_differences(spec):
    g = qo.HashGrid(spec)
    rng = np.random.default_rng(13)
    table = rng.standard_normal(g.n_params).astype(np.float32)
    lo = np.array(spec["bounding_box_min"], dtype=np.float64)
    sz = np.array(spec["bounding_box_size"], dtype=np.float64)
    Rmax = g.level_table()[-1][0]
    # keep every point away from cell boundaries of the finest level so FD stays in one cell
    cell = rng.integers(0, Rmax - 1, (25, g.dim))
    u = (cell + rng.uniform(0.3, 0.7, (25, g.dim))) / (Rmax - 1)
    ok = np.ones(25, dtype=bool)
    for (R, _, _, _) in g.level_table():
        fr = (u * (R - 1)) % 1.0
        ok &= np.all((fr > 0.05) & (fr < 0.95), axis=1)
    u = u[ok]
    assert len(u) >= 5
    x = (lo + sz * u).astype(np.float32)
    v = rng.standard_normal((len(x), g.num_outputs)).astype(np.float32)
    adj_x, _ = g.adjoint(table, x, v, param_grads=False, res_factor=1)
    eps = 1e-4 * sz
    fd = np.zeros_like(adj_x, dtype=np.float64)
    for d in range(g.dim):
        xp, xm = x.astype(np.float64).copy(), x.astype(np.float64).copy()
        xp[:, d] += eps[d]
        xm[:, d] -= eps[d]
        # brute force keeps float64 fractional parts; cell selection uses fp32 like the kernel
        fp = brute_force_grid_f64(g, table, xp)
        fm = brute_force_grid_f64(g, table, xm)
        fd[:, d] = ((fp - fm) * v).sum(1) / (2 * eps[d])
    assert np.allclose(adj_x, fd, rtol=2e-3, atol=2e-3)


def brute_force_grid_f64(g, table, x):
    """Same as brute_force_grid but entirely in float64 (for finite differences)."""
    table = np.asarray(table, dtype=np.float64)
    N, D, F = x.shape[0], g.dim, g.n_feat
    out = np.zeros((N, g.num_outputs))
    bmin = np.array(g.cfg["bounding_box_min"], dtype=np.float64)
    bsz = np.array(g.cfg["bounding_box_size"], dtype=np.float64)
    for n in range(N):
        pos = (x[n, g.start_in:g.start_in + D] - bmin) / bsz
        for l, (R, hashed, off, hsize) in enumerate(g.level_table()):
            p = pos * (R - 1)
            lo = np.clip(np.trunc(p).astype(np.int64), 0, R - 1)
            hi = np.clip(np.trunc(p).astype(np.int64) + 1, 0, R - 1)
            fr = p - lo
            feat = np.zeros(F)
            for bits in itertools.product((0, 1), repeat=D):
                c = [hi[d] if bits[d] else lo[d] for d in range(D)]
                w = np.prod([fr[d] if bits[d] else 1 - fr[d] for d in range(D)])
                if hashed:
                    h = 0
                    for d in range(D):
                        h ^= (int(c[d]) * PRIMES[d]) & 0xFFFFFFFF
                    idx = h % hsize
                else:
                    idx = 0
                    for d in range(D):
                        idx = idx * R + int(c[d])
                feat += w * table[off + idx * F: off + idx * F + F]
            if g.combination == qo.CONCAT:
                out[n, l * F:(l + 1) * F] = feat
            else:
                out[n, :F] += feat
    return out


# ------------------------------------------------------------------ activations
def test_activations_match_torch():
    xs = np.linspace(-4, 4, 161).astype(np.float32)
    L = qo.lib()
    t = torch.from_numpy(xs).requires_grad_(True)
    for act, fn in ((qo.ACT_RELU, torch.relu), (qo.ACT_CELU, torch.nn.functional.celu),
                    (qo.ACT_SINE, torch.sin), (qo.ACT_IDENTITY, lambda z: z * 1.0),
                    (qo.ACT_SINE_FREQ, lambda z: torch.sin(30.0 * z))):
        if t.grad is not None:
            t.grad = None
        y = fn(t)
        y.backward(torch.full_like(y, 0.7))
        mine = np.array([L.qo_act_forward(act, 30.0, float(v)) for v in xs])
        mine_adj = np.array([L.qo_act_adjoint(act, 30.0, float(v), 0.7) for v in xs])
        assert np.allclose(mine, y.detach().numpy(), atol=1e-5)
        keep = np.abs(xs) > 1e-6       # relu/celu kink at 0 is convention
        assert np.allclose(mine_adj[keep], t.grad.numpy()[keep], atol=2e-4)


# ------------------------------------------------------------------ MLP vs torch linear + autograd
def mlp_cfg(n_in, widths, acts, biases):
    return {"num_inputs": n_in, "num_outputs": widths[-1],
            "activation_specification": ["qmlp/builtin-activations.json"],
            "encodings": [{"id": "Identity", "start_in": 0, "n_in": n_in}],
            "network": [{"n_out": w, "bias": b, "activation": a}
                        for w, a, b in zip(widths, acts, biases)]}


TORCH_ACT = {"relu": torch.relu, "celu": torch.nn.functional.celu, "sine": torch.sin,
             "identity": lambda z: z}


def torch_mlp(net, X, adj, params):
    """Plain torch evaluation on the padded parameter layout; returns out, dX, dParams."""
    p = torch.from_numpy(params.copy()).requires_grad_(True)
    x = torch.from_numpy(X.copy()).requires_grad_(True)
    h = torch.nn.functional.pad(x, (0, net.layers[0]["cin"] - X.shape[1]))
    for i, l in enumerate(net.layers):
        W = p[l["w_start"]: l["w_start"] + l["cin"] * l["cout"]].reshape(l["cout"], l["cin"])
        b = p[l["b_start"]: l["b_start"] + l["cout"]] if l["bias"] else None
        h = torch.nn.functional.linear(h, W, b)
        a = net.cfg["network"][i]["activation"]
        if isinstance(a, str):
            h = TORCH_ACT[a](h)
        else:   # one activation per channel; the padding takes the last one
            a = list(a) + [a[-1]] * (l["cout"] - len(a))
            h = torch.stack([TORCH_ACT[a[c]](h[:, c]) for c in range(l["cout"])], dim=1)
    out = h[:, :net.n_out]
    (out * torch.from_numpy(adj)).sum().backward()
    return out.detach().numpy(), x.grad.numpy(), p.grad.numpy()


@pytest.mark.parametrize("n_in,widths,acts,biases,N", [
    (16, [16], ["celu"], [False], 35), (48, [32], ["sine"], [False], 35),
    (19, [16, 16], ["identity", "identity"], [False, False], 32),
    (16, [16, 23], ["identity", "identity"], [False, False], 32),
    (20, [16, 24], ["identity", "identity"], [False, False], 32),
    (3, [16, 1], ["relu", "relu"], [True, True], 513),
    (4, [128, 64, 48, 4], ["sine", "sine", "celu", "identity"], [True, True, True, True], 128),
    (5, [32, 48, 16], ["celu", "relu", "identity"], [False, True, False], 16),
    (7, [20, 5], [["relu", "sine", "celu", "identity"] * 5, ["sine", "identity", "relu", "relu", "celu"]], [True, False], 64)])
def test_mlp_matches_torch_linear_autograd(n_in, widths, acts, biases, N):
    net = qo.Network(mlp_cfg(n_in, widths, acts, biases))
    rng = np.random.default_rng(42)
    params = rng.uniform(-0.4, 0.4, net.num_parameters).astype(np.float32)
    net.set_parameters(params)
    X = rng.uniform(-1, 1, (N, n_in)).astype(np.float32)
    adj = rng.standard_normal((N, widths[-1])).astype(np.float32)
    out = net.forward(X)
    res = net.backward(X, adj, qo.GRAD_INPUT | qo.GRAD_WEIGHTS)
    t_out, t_dx, t_dp = torch_mlp(net, X, adj, params)
    assert np.allclose(out, t_out, atol=1e-4)
    assert np.allclose(res["adj_x"], t_dx, atol=1e-4)
    assert np.allclose(res["grads"], t_dp, rtol=1e-4, atol=1e-3)


def test_parameter_layout_counts_from_reference_configs():
    # padded shapes: all weights first (row-major (C_out, C_in)), then biases
    assert qo.Network(mlp_cfg(3, [16, 1], ["relu", "relu"], [False, False])).num_parameters == 512
    n4 = qo.Network(mlp_cfg(4, [128, 64, 48, 4], ["sine", "sine", "celu", "identity"], [True] * 4))
    assert n4.num_parameters == 14080 + 256
    assert n4.layers[0]["w_start"] == 0 and n4.layers[1]["w_start"] == 16 * 128
    assert n4.layers[0]["b_start"] == 14080 and n4.layers[3]["b_start"] == 14080 + 128 + 64 + 48
    n = qo.Network(mlp_cfg(19, [23, 5], ["identity", "identity"], [False, False]))
    assert [(l["cin"], l["cout"]) for l in n.layers] == [(32, 32), (32, 16)]


def test_padding_invariants():
    net = qo.Network(mlp_cfg(5, [19, 3], ["celu", "identity"], [True, False]))
    rng = np.random.default_rng(0)
    params = rng.uniform(-0.5, 0.5, net.num_parameters).astype(np.float32)
    X = rng.uniform(-1, 1, (40, 5)).astype(np.float32)
    net.set_parameters(params)
    base = net.forward(X)
    # weights on padded input columns multiply zeros
    p2 = params.copy()
    p2[:net.layers[0]["cin"] * net.layers[0]["cout"]].reshape(32, 16)[:, 5:] += 3.0
    net.set_parameters(p2)
    assert np.array_equal(net.forward(X), base)
    # padded rows of the last layer never reach the output
    p3 = params.copy()
    l1 = net.layers[1]
    p3[l1["w_start"]:l1["w_start"] + 16 * 32].reshape(16, 32)[3:, :] = 9.0
    net.set_parameters(p3)
    assert np.array_equal(net.forward(X), base)


# ------------------------------------------------------------------ fused = encoding o MLP
def test_fused_network_is_the_composition():
    cfg = {"num_inputs": 4, "num_outputs": 2, "activation_specification": [],
           "encodings": [grid_spec(3, 4, 2, 6, 3, 30, start=1), {"id": "Identity", "start_in": 0, "n_in": 4}],
           "network": [{"n_out": 32, "bias": True, "activation": "relu"},
                       {"n_out": 2, "bias": False, "activation": "identity"}]}
    net = qo.Network(cfg)
    assert net.encoded_channels == 12 and net.layers[0]["cin"] == 16
    rng = np.random.default_rng(4)
    g = net.encodings[0][1]
    table = rng.standard_normal(g.n_params).astype(np.float32)
    params = rng.uniform(-0.3, 0.3, net.num_parameters).astype(np.float32)
    net.set_parameters(params)
    net.set_table(0, table)
    X = rng.uniform(0, 1, (64, 4)).astype(np.float32)
    out, enc, pre = net.forward(X, store=True)
    feats = np.concatenate([g.forward(table, X), X, np.zeros((64, 4), np.float32)], axis=1)
    assert np.allclose(enc, feats, atol=1e-6)
    W0, b0, W1 = net.weight(0), net.bias(0), net.weight(1)
    h = np.maximum(feats @ W0.T + b0, 0)
    assert np.allclose(out, (h @ W1.T)[:, :2], atol=1e-4)
    # gradients: chain rule through both halves
    adj = rng.standard_normal((64, 2)).astype(np.float32)
    res = net.backward(X, adj, qo.GRAD_INPUT | qo.GRAD_WEIGHTS | qo.GRAD_ENCODINGS)
    dpre1 = np.pad(adj, ((0, 0), (0, 14)))
    dh = dpre1 @ W1
    dpre0 = dh * (pre[0] > 0)
    dfeat = dpre0 @ W0
    ax, gt = g.adjoint(table, X, dfeat[:, :8])
    assert np.allclose(res["table_grads"][0], gt, atol=1e-4)
    assert np.allclose(res["adj_x"], ax + dfeat[:, 8:12], atol=1e-3)
    assert np.allclose(net.weight(0, res["grads"]), dpre0.T @ feats, atol=1e-3)
    assert np.allclose(net.bias(0, res["grads"]), dpre0.sum(0), atol=1e-3)
    assert np.allclose(net.weight(1, res["grads"]), dpre1.T @ h, atol=1e-3)


def test_round_mode_one_stays_close_to_fp32():
    net = qo.Network(mlp_cfg(8, [32, 32, 4], ["relu", "celu", "identity"], [True, True, True]))
    rng = np.random.default_rng(6)
    net.set_parameters(qo.round_half(rng.uniform(-0.3, 0.3, net.num_parameters)))
    X = rng.uniform(-1, 1, (256, 8)).astype(np.float32)
    a, b = net.forward(X, 0), net.forward(X, 1)
    frac, worst = qo.compare(b, a, 1e-2, 1e-3)
    assert frac == 0.0
    assert not np.array_equal(a, b)


def test_round_mode_one_rounds_at_every_point_of_the_half_precision_pipeline():
    """Known answer for the oracle mode that rounds to fp16 where the device does. One point
    through identity(1) -> 16 sine -> 1 identity with two live hidden units; the numbers are
    worked out by hand (exact binary fractions, sine / cosine from tables to 16 digits), every value
    in front of a rounding sits at least 1/8 fp16 ulp away from a tie, and every rounding changes
    its value, so a rounding that is missing or sits elsewhere changes one of the results below.

      x = 1.0006103515625          -> encoded row   x^ = 1.0009765625      (1 + 0.625 ulp -> 1 + 1 ulp)
      pre0 = 0.8125  * x^ = 0.81329345703125 -> 0.8134765625 ; pre1 = 0.5625 * x^ = 0.56304931640625 -> 0.56298828125
      h0 = sin(pre0) = 0.72667986... -> 0.7265625            ; h1 = sin(pre1) = 0.53371566... -> 0.53369140625
      y  = 0.6875 h0 - 1.4375 h1 = -0.267669677734375 -> -0.267578125
      g = dL/dy = 0.30010986328125 -> g^ = 0.300048828125
      dW1 = g^ * (h0, h1) = (0.21800422668457031, 0.16013348102569580)   (fp32 products of fp16 values: exact)
      dh = (0.6875 g^, -1.4375 g^) = (0.2062835693359375, -0.4313201904296875) -> (0.206298828125, -0.431396484375)
      dpre0 = cos(pre) * dh = (0.14172239..., -0.36481648...) -> (0.1417236328125, -0.36474609375)
      dW0 = dpre0 * x^ = (0.14186203479766846, -0.36510229110717773)
      dx = 0.8125 dpre0[0] + 0.5625 dpre0[1] = -0.09001922607421875 -> -0.09002685546875
    """
    net = qo.Network(mlp_cfg(1, [2, 1], ["sine", "identity"], [False, False]))
    params = np.zeros(net.num_parameters, np.float32)
    w0, w1 = net.weight(0, params), net.weight(1, params)
    w0[0, 0], w0[1, 0] = 0.8125, 0.5625
    w1[0, 0], w1[0, 1] = 0.6875, -1.4375
    net.set_parameters(params)
    X = np.array([[1.0006103515625]], np.float32)
    g = np.array([[0.30010986328125]], np.float32)
    out, enc, pre = net.forward(X, round_mode=1, store=True)
    assert enc[0, 0] == np.float32(1.0009765625)
    assert pre[0][0, 0] == np.float32(0.8134765625) and pre[0][0, 1] == np.float32(0.56298828125)
    assert pre[1][0, 0] == np.float32(-0.267578125) and out[0, 0] == np.float32(-0.267578125)
    res = net.backward(X, g, qo.GRAD_INPUT | qo.GRAD_WEIGHTS, round_mode=1, return_dpre=True)
    assert res["dpre"][1][0, 0] == np.float32(0.300048828125)
    assert res["dpre"][0][0, 0] == np.float32(0.1417236328125) and res["dpre"][0][0, 1] == np.float32(-0.36474609375)
    dw0, dw1 = net.weight(0, res["grads"]), net.weight(1, res["grads"])
    assert dw1[0, 0] == np.float32(0.21800422668457031) and dw1[0, 1] == np.float32(0.16013348102569580)
    assert dw0[0, 0] == np.float32(0.14186203479766846) and dw0[1, 0] == np.float32(-0.36510229110717773)
    assert res["adj_x"][0, 0] == np.float32(-0.09002685546875)
    # everything else of the padded matrices stays zero
    assert np.count_nonzero(res["grads"]) == 4
    # the fp32 mode rounds nowhere: the same chain without the arrows
    out0 = net.forward(X, round_mode=0)
    assert abs(float(out0[0, 0]) - (-0.26767468)) < 1e-7 and out0[0, 0] != out[0, 0]
    res0 = net.backward(X, g, qo.GRAD_INPUT | qo.GRAD_WEIGHTS, round_mode=0)
    assert abs(float(res0["adj_x"][0, 0]) - (-0.09001060)) < 1e-7
    assert np.allclose(net.weight(1, res0["grads"])[0, :2], [0.21798468, 0.16013654], rtol=0, atol=1e-7)
    assert np.allclose(net.weight(0, res0["grads"])[:2, 0], [0.14189935, -0.36508220], rtol=0, atol=1e-7)


# ------------------------------------------------------------------ line integration
def line_spec(child, stepsize=0.25, blending="additive", start=0):
    return {"id": "LineIntegration", "start_in": start, "n_in": 3, "volume": child, "stepsize": stepsize,
            "blending": blending}


def slab_interval(start, direction, bmin, bsize):
    """Independent float64 slab test (zero direction components: the slab does not bound t)."""
    lo, hi = -np.inf, np.inf
    for d in range(3):
        if direction[d] == 0:
            assert bmin[d] <= start[d] <= bmin[d] + bsize[d]
            continue
        ta = (bmin[d] - start[d]) / direction[d]
        tb = (bmin[d] + bsize[d] - start[d]) / direction[d]
        lo, hi = max(lo, min(ta, tb)), min(hi, max(ta, tb))
    return lo, hi


def test_line_integration_known_answer_axis_aligned_ray():
    """Box [-1,1]^3, ray from (-2,0.1,0.2) along +x: inside for t in [1,3); with a step of 0.25
    the march samples t = 1, 1.25, .., 2.75: 8 samples, floor(2/0.25) = 8 steps. A constant
    table c (partition of unity) therefore gives 8c when summing and c when averaging."""
    child = grid_spec(3, levels=2, feat=2, log2=6, rmin=3, rmax=9, bmin=[-1.0] * 3, bsize=[2.0] * 3)
    x = np.array([[-2.0, 0.1, 0.2, 1.0, 0.0, 0.0]], np.float32)
    for blending, want in (("additive", 8 * 0.375), ("average", 0.375)):
        li = qo.LineIntegration(line_spec(child, 0.25, blending))
        table = np.full(li.n_params, 0.375, np.float32)
        out = li.forward(table, x)
        assert out.shape == (1, 4)
        assert np.allclose(out, want, rtol=1e-6, atol=0)


def test_line_integration_misses_and_rays_starting_inside():
    child = grid_spec(3, levels=1, feat=1, rmin=4, rmax=4, bmin=[-1.0] * 3, bsize=[2.0] * 3)
    li = qo.LineIntegration(line_spec(child, 0.3, "additive"))
    table = np.full(li.n_params, 2.0, np.float32)
    # passes beside the box: no sample
    miss = np.array([[-2.0, 3.0, 0.0, 1.0, 0.0, 0.0]], np.float32)
    assert np.all(li.forward(table, miss) == 0)
    # starts at the centre: the march begins at the (negative) entry parameter, as in the reference
    inside = np.array([[0.0, 0.0, 0.0, 0.0, 0.0, 1.0]], np.float32)
    lo, hi = slab_interval(inside[0, :3].astype(np.float64), inside[0, 3:].astype(np.float64), [-1.0] * 3, [2.0] * 3)
    assert (lo, hi) == (-1.0, 1.0)
    count = len([k for k in range(100) if lo + k * 0.3 < hi])      # 7 samples: -1, -0.7, .., 0.8
    assert count == 7
    assert np.allclose(li.forward(table, inside), 2.0 * count, rtol=1e-6)


def test_line_integration_of_a_linear_field_has_a_closed_form():
    """A dense level whose node values are an affine function of the node position interpolates
    that function exactly, so the sum over the samples t_k = tmin + k h is
    n (a.start + b) + (a.dir) sum t_k."""
    R = 5
    bmin, bsize = np.array([-1.0, -0.5, 0.0]), np.array([2.0, 1.5, 1.0])
    child = grid_spec(3, levels=1, feat=1, rmin=R, rmax=R, bmin=list(bmin), bsize=list(bsize))
    h = 0.07
    a, b = np.array([0.3, -0.7, 1.1]), 0.25
    li = qo.LineIntegration(line_spec(child, h, "additive", start=1))
    nodes = np.stack(np.meshgrid(*[np.arange(R)] * 3, indexing="ij"), -1).reshape(-1, 3)   # last coordinate fastest
    table = (bmin + bsize * nodes / (R - 1)) @ a + b
    rng = np.random.default_rng(5)
    rays = []
    while len(rays) < 20:
        start = bmin + bsize * rng.uniform(-0.5, 1.5, 3)
        target = bmin + bsize * rng.uniform(0.2, 0.8, 3)
        d = (target - start) / np.linalg.norm(target - start)
        lo, hi = slab_interval(start, d, bmin, bsize)
        frac = ((hi - lo) / h) % 1.0
        if hi > lo and 0.2 < frac < 0.8:        # the number of samples is not a rounding matter
            rays.append(np.concatenate([[9.0], start, d]))
    X = np.array(rays, np.float32)
    out = li.forward(table.astype(np.float32), X)[:, 0]
    for n, ray in enumerate(X.astype(np.float64)):
        start, d = ray[1:4], ray[4:7]
        lo, hi = slab_interval(start, d, bmin, bsize)
        t = lo + h * np.arange(int(np.ceil((hi - lo) / h)))
        want = len(t) * (a @ start + b) + (a @ d) * t.sum()
        assert abs(out[n] - want) < 2e-4 * max(1.0, abs(want)), (n, out[n], want)


def _line_samples(li, cfg_child, ray):
    """The sample parameters and positions of one ray in the fp32 arithmetic of the march
    (entry parameter by an fp32 slab test, t += h in fp32, fused multiply-add positions)."""
    f = np.float32
    start, d = ray[li.start_in:li.start_in + 3].astype(f), ray[li.start_in + 3:li.start_in + 6].astype(f)
    bmin, bsize = np.array(cfg_child["bounding_box_min"], f), np.array(cfg_child["bounding_box_size"], f)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = f(1) / d
        ta, tb = (bmin - start) * inv, ((bmin + bsize) - start) * inv
    tmin, tmax = np.fmax.reduce(np.fmin(ta, tb)), np.fmin.reduce(np.fmax(ta, tb))
    ts, t = [], tmin
    while t < tmax:
        ts.append(t)
        t = f(t + f(li.stepsize))
    ts = np.array(ts, f)
    pos = (ts.astype(np.float64)[:, None] * d.astype(np.float64) + start.astype(np.float64)).astype(f)  # one rounding = fma
    steps = int(np.floor(f(f(tmax - tmin) / f(li.stepsize)))) if len(ts) else 0
    return ts, pos, steps


@pytest.mark.parametrize("blending", ["additive", "average"])
def test_line_integration_is_the_sum_of_the_pinned_grid_over_the_samples(blending):
    """Forward, input gradients (tmin/tmax constant, as in the reference) and table gradients
    equal the sums over explicitly generated sample positions of the separately pinned grid
    forward / adjoint."""
    child = grid_spec(3, levels=3, feat=2, log2=9, rmin=4, rmax=32, bmin=[-1.0, -1.0, -1.0], bsize=[2.0, 2.0, 2.0])
    li = qo.LineIntegration(line_spec(child, 0.11, blending, start=1))
    g = qo.HashGrid(child)
    rng = np.random.default_rng(11)
    table = rng.standard_normal(g.n_params).astype(np.float32)
    N = 40
    start = rng.uniform(-2, 2, (N, 3))
    target = rng.uniform(-0.8, 0.8, (N, 3))
    d = target - start
    d /= np.linalg.norm(d, axis=1, keepdims=True)
    X = np.concatenate([np.zeros((N, 1)), start, d], 1).astype(np.float32)
    X[0, 4:7] = [0.0, 1.0, 0.0]; X[0, 1:4] = [0.3, -2.0, 0.1]       # a zero direction component
    adj = rng.standard_normal((N, g.num_outputs)).astype(np.float32)
    out = li.forward(table, X)
    adj_x, grad = li.adjoint(table, X, adj)
    want_grad = np.zeros(g.n_params, np.float64)
    for n in range(N):
        ts, pos, steps = _line_samples(li, child, X[n])
        scale = 1.0 / steps if (blending == "average" and steps > 0) else 1.0
        assert len(ts) > 3
        feats = g.forward(table, pos).astype(np.float64)
        assert np.allclose(out[n], feats.sum(0) * scale, rtol=2e-5, atol=2e-5)
        a_rep = np.repeat((adj[n] * np.float32(scale))[None], len(ts), 0)
        ap, gp = g.adjoint(table, pos, a_rep)
        assert np.allclose(adj_x[n, 1:4], ap.astype(np.float64).sum(0), rtol=1e-4, atol=1e-3)
        assert np.allclose(adj_x[n, 4:7], (ap.astype(np.float64) * ts[:, None]).sum(0), rtol=1e-4, atol=1e-3)
        assert adj_x[n, 0] == 0
        want_grad += gp
    assert np.allclose(grad, want_grad, rtol=1e-4, atol=1e-4)


def test_line_integration_table_gradient_is_the_transpose_of_forward():
    child = grid_spec(3, levels=2, feat=2, log2=8, rmin=3, rmax=20, bmin=[0.0] * 3, bsize=[1.0] * 3)
    li = qo.LineIntegration(line_spec(child, 0.05, "average"))
    rng = np.random.default_rng(2)
    N = 64
    start = rng.uniform(-0.5, 1.5, (N, 3))
    d = rng.uniform(0.2, 0.8, (N, 3)) - start
    X = np.concatenate([start, d / np.linalg.norm(d, axis=1, keepdims=True)], 1).astype(np.float32)
    theta = rng.standard_normal(li.n_params).astype(np.float32)
    v = rng.standard_normal((N, li.num_outputs)).astype(np.float32)
    lhs = float((li.forward(theta, X).astype(np.float64) * v).sum())
    _, grad = li.adjoint(np.zeros_like(theta), X, v, input_grads=False)
    rhs = float((grad.astype(np.float64) * theta).sum())
    assert abs(lhs - rhs) < 1e-4 * max(1.0, abs(lhs))


def test_fused_network_with_line_integration_is_the_composition():
    child = grid_spec(3, levels=2, feat=2, log2=8, rmin=3, rmax=20, bmin=[-1.0] * 3, bsize=[2.0] * 3)
    line = line_spec(child, 0.2, "average")
    cfg = {"num_inputs": 6, "num_outputs": 2, "activation_specification": [],
           "encodings": [line],
           "network": [{"n_out": 16, "bias": True, "activation": "relu"},
                       {"n_out": 2, "bias": False, "activation": "identity"}]}
    net = qo.Network(cfg)
    li = qo.LineIntegration(line)
    rng = np.random.default_rng(4)
    table = rng.standard_normal(li.n_params).astype(np.float32)
    params = (rng.standard_normal(net.num_parameters) * 0.3).astype(np.float32)
    net.set_parameters(params)
    net.set_table(0, table)
    N = 30
    start = rng.uniform(-2, 2, (N, 3))
    d = rng.uniform(-0.5, 0.5, (N, 3)) - start
    X = np.concatenate([start, d / np.linalg.norm(d, axis=1, keepdims=True)], 1).astype(np.float32)
    enc = li.forward(table, X)
    W0, b0, W1 = net.weight(0)[:, :4], net.bias(0), net.weight(1)[:2]
    pre0 = enc @ W0.T + b0
    want = np.maximum(pre0, 0) @ W1.T
    assert np.allclose(net.forward(X), want, rtol=1e-4, atol=1e-5)
    # backward: the adjoint of the encoded input goes through the march's own (pinned) adjoint
    adj = rng.standard_normal((N, 2)).astype(np.float32)
    res = net.backward(X, adj, 7)
    d_enc = ((adj @ W1) * (pre0 > 0)) @ W0
    want_ax, want_gt = li.adjoint(table, X, d_enc.astype(np.float32))
    assert np.allclose(res["adj_x"], want_ax, rtol=1e-3, atol=1e-4)
    assert np.allclose(res["table_grads"][0], want_gt, rtol=1e-3, atol=1e-4)


def test_line_integration_takes_no_sample_on_unbounded_or_endless_rays():
    """Where the reference's march would never end (zero direction: tmin = -inf; a step far
    below the float spacing at t) the ray takes no sample; the result is zero, not a hang."""
    child = grid_spec(3, levels=1, feat=1, rmin=4, rmax=4, bmin=[-1.0] * 3, bsize=[2.0] * 3)
    table = np.full(64, 2.0, np.float32)
    X = np.array([[0.0, 0.0, 0.0, 0.0, 0.0, 0.0],          # no direction at all, start inside the box
                  [0.0, 0.0, 0.0, 1e-30, 0.0, 0.0],        # interval of 2e30 length
                  [0.0, 0.0, 0.0, 0.0, 0.0, 1.0]], np.float32)
    li = qo.LineIntegration(line_spec(child, 0.3, "additive"))
    out = li.forward(table, X)
    assert out[0, 0] == 0 and out[1, 0] == 0 and out[2, 0] == 14.0
    ax, gp = li.adjoint(table, X[:2], np.ones((2, 1), np.float32))
    assert not ax.any() and not gp.any()
    tiny = qo.LineIntegration(line_spec(child, 1e-9, "additive"))      # 2e9 steps: refused
    assert tiny.forward(table, X[2:])[0, 0] == 0
