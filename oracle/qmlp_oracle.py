"""ctypes front end of the CPU oracle (test infrastructure only).

The shipped library never imports this module; tests, the smoke check and the
benchmark's CPU-baseline leg do. The spec handling below restates the padding and
flat-parameter layout rules of the reference (src_cpp/src/fused_network.cpp:147-206,
314-346): every layer width is rounded up to a multiple of 16, all weight matrices
come first (row-major (C_out, C_in)), then the biases of the biased layers. One
deliberate divergence: the fan-in of layer 0 is the number of encoded channels, not
``num_inputs`` (fused_network.cpp:95 uses num_inputs, which only works for
encodings that keep the channel count).
"""
import ctypes
import json
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libqmlp_oracle.so")

MAX_LEVELS, MAX_DIM, MAX_ENC, MAX_LAYERS = 32, 6, 8, 16
ACT_RELU, ACT_CELU, ACT_SINE, ACT_IDENTITY, ACT_SINE_FREQ = 0, 1, 2, 3, 4
CONCAT, ADD = 0, 1
ENC_IDENTITY, ENC_HASHGRID, ENC_LINE = 0, 1, 2
GRAD_INPUT, GRAD_WEIGHTS, GRAD_ENCODINGS = 1, 2, 4

BUILTIN_ACTIVATIONS = {
    "relu": (ACT_RELU, 0.0),
    "celu": (ACT_CELU, 0.0),
    "sine": (ACT_SINE, 0.0),
    "identity": (ACT_IDENTITY, 0.0),
}

_fp = ctypes.POINTER(ctypes.c_float)
_u32p = ctypes.POINTER(ctypes.c_uint32)


class HashGridStruct(ctypes.Structure):
    _fields_ = [
        ("start_in", ctypes.c_int), ("dim", ctypes.c_int), ("n_levels", ctypes.c_int),
        ("n_feat", ctypes.c_int), ("combination", ctypes.c_int), ("n_params", ctypes.c_int),
        ("mem_offset", ctypes.c_int * MAX_LEVELS), ("resolution", ctypes.c_int * MAX_LEVELS),
        ("hash_size", ctypes.c_int * MAX_LEVELS), ("hashed", ctypes.c_int * MAX_LEVELS),
        ("bb_min", ctypes.c_float * MAX_DIM), ("bb_inv", ctypes.c_float * MAX_DIM),
    ]


class LineStruct(ctypes.Structure):
    _fields_ = [
        ("start_in", ctypes.c_int), ("blending", ctypes.c_int), ("stepsize", ctypes.c_float),
        ("bb_min", ctypes.c_float * 3), ("bb_size", ctypes.c_float * 3),
    ]


class NetworkStruct(ctypes.Structure):
    _fields_ = [
        ("n_in", ctypes.c_int), ("n_enc", ctypes.c_int),
        ("enc_kind", ctypes.c_int * MAX_ENC), ("enc_start", ctypes.c_int * MAX_ENC),
        ("enc_nin", ctypes.c_int * MAX_ENC),
        ("enc_grid", ctypes.POINTER(HashGridStruct) * MAX_ENC),
        ("enc_table", _fp * MAX_ENC), ("enc_grad", _fp * MAX_ENC),
        ("enc_line", ctypes.POINTER(LineStruct) * MAX_ENC),
        ("n_layers", ctypes.c_int),
        ("cin", ctypes.c_int * MAX_LAYERS), ("cout", ctypes.c_int * MAX_LAYERS),
        ("act", ctypes.c_int * MAX_LAYERS), ("act_param", ctypes.c_float * MAX_LAYERS),
        ("act_channel", ctypes.POINTER(ctypes.c_int) * MAX_LAYERS), ("act_param_channel", _fp * MAX_LAYERS),
        ("W", _fp * MAX_LAYERS), ("b", _fp * MAX_LAYERS),
        ("dW", _fp * MAX_LAYERS), ("db", _fp * MAX_LAYERS),
        ("round_mode", ctypes.c_int), ("res_factor", ctypes.c_int),
    ]


def build():
    """Compile the oracle's C restatement (gcc + make)."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "libqmlp_oracle.so"],
                          stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.qo_round_half.restype = ctypes.c_float
        L.qo_round_half.argtypes = [ctypes.c_float]
        L.qo_hashgrid_init.restype = ctypes.c_int
        L.qo_hashgrid_init.argtypes = [ctypes.POINTER(HashGridStruct)] + [ctypes.c_int] * 8 + [_fp, _fp]
        L.qo_hashgrid_num_outputs.argtypes = [ctypes.POINTER(HashGridStruct)]
        L.qo_index_dense.restype = ctypes.c_uint32
        L.qo_index_dense.argtypes = [ctypes.c_int, _u32p, ctypes.c_uint32]
        L.qo_index_hash.restype = ctypes.c_uint32
        L.qo_index_hash.argtypes = [ctypes.c_int, _u32p]
        L.qo_hashgrid_corners.restype = None
        L.qo_hashgrid_corners.argtypes = [ctypes.POINTER(HashGridStruct), _fp, ctypes.c_long,
                                          ctypes.c_long, _u32p, _fp]
        L.qo_hashgrid_forward.restype = None
        L.qo_hashgrid_forward.argtypes = [ctypes.POINTER(HashGridStruct), _fp, _fp, ctypes.c_long,
                                          ctypes.c_long, _fp, ctypes.c_long]
        L.qo_hashgrid_adjoint.restype = None
        L.qo_hashgrid_adjoint.argtypes = [ctypes.POINTER(HashGridStruct), _fp, _fp, ctypes.c_long,
                                          ctypes.c_long, _fp, ctypes.c_long, _fp, ctypes.c_long,
                                          _fp, ctypes.c_int]
        L.qo_line_forward.argtypes = [ctypes.POINTER(LineStruct), ctypes.POINTER(HashGridStruct), _fp, _fp,
                                      ctypes.c_long, ctypes.c_long, _fp, ctypes.c_long]
        L.qo_line_adjoint.argtypes = [ctypes.POINTER(LineStruct), ctypes.POINTER(HashGridStruct), _fp, _fp,
                                      ctypes.c_long, ctypes.c_long, _fp, ctypes.c_long, _fp, ctypes.c_long,
                                      _fp, ctypes.c_int]
        L.qo_act_forward.restype = ctypes.c_float
        L.qo_act_forward.argtypes = [ctypes.c_int, ctypes.c_float, ctypes.c_float]
        L.qo_act_adjoint.restype = ctypes.c_float
        L.qo_act_adjoint.argtypes = [ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_float]
        L.qo_network_forward.restype = None
        L.qo_network_forward.argtypes = [ctypes.POINTER(NetworkStruct), _fp, ctypes.c_long,
                                         ctypes.c_long, _fp, ctypes.c_int, _fp,
                                         ctypes.POINTER(_fp)]
        L.qo_network_backward.restype = None
        L.qo_network_backward.argtypes = [ctypes.POINTER(NetworkStruct), _fp, ctypes.c_long,
                                          ctypes.c_long, _fp, ctypes.c_int, ctypes.c_int, _fp,
                                          ctypes.POINTER(_fp), _fp, ctypes.POINTER(_fp)]
        L.qo_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a):
    return a.ctypes.data_as(_fp) if a is not None else ctypes.cast(None, _fp)


def round_half(a):
    """Round to fp16 and back with numpy (an independent route to qo_round_half)."""
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)


def round_up(x, m):
    return (x + m - 1) // m * m


class HashGrid:
    """Level table + encoding of one HashGrid spec (encoding_hashgrid.cpp:99-112 keys)."""

    def __init__(self, cfg):
        self.cfg = dict(cfg)
        mode = cfg["combination_mode"]
        # nlohmann's enum macro maps unknown strings to the first entry (concat)
        self.combination = ADD if mode == "add" else CONCAT
        dim = int(cfg["n_in"])
        bmin = cfg.get("bounding_box_min") or [-0.5] * dim
        bsize = cfg.get("bounding_box_size") or [1.0] * dim
        if len(bmin) != dim or len(bsize) != dim:
            raise ValueError("bounding box dimension mismatch")
        self.s = HashGridStruct()
        bm = (ctypes.c_float * dim)(*bmin)
        bs = (ctypes.c_float * dim)(*bsize)
        rc = lib().qo_hashgrid_init(ctypes.byref(self.s), int(cfg["start_in"]), dim,
                                    int(cfg["n_levels"]), int(cfg["n_features_per_level"]),
                                    int(cfg["log2_hashmap_size"]), int(cfg["min_resolution"]),
                                    int(cfg["max_resolution"]), self.combination, bm, bs)
        if rc != 0:
            raise ValueError("invalid HashGrid configuration (code %d)" % rc)

    dim = property(lambda self: self.s.dim)
    n_levels = property(lambda self: self.s.n_levels)
    n_feat = property(lambda self: self.s.n_feat)
    n_params = property(lambda self: self.s.n_params)
    start_in = property(lambda self: self.s.start_in)

    @property
    def num_outputs(self):
        return lib().qo_hashgrid_num_outputs(ctypes.byref(self.s))

    def level_table(self):
        L = self.n_levels
        return [(self.s.resolution[l], bool(self.s.hashed[l]), self.s.mem_offset[l],
                 self.s.hash_size[l]) for l in range(L)]

    def corners(self, x):
        x = _f32(x)
        N = x.shape[0]
        nc = 1 << self.dim
        idx = np.zeros((N, self.n_levels, nc), dtype=np.uint32)
        w = np.zeros((N, self.n_levels, nc), dtype=np.float32)
        lib().qo_hashgrid_corners(ctypes.byref(self.s), _ptr(x), N, x.shape[1],
                                  idx.ctypes.data_as(_u32p), _ptr(w))
        return idx, w

    def forward(self, table, x):
        table, x = _f32(table), _f32(x)
        assert table.size == self.n_params
        N = x.shape[0]
        out = np.zeros((N, self.num_outputs), dtype=np.float32)
        lib().qo_hashgrid_forward(ctypes.byref(self.s), _ptr(table), _ptr(x), N, x.shape[1],
                                  _ptr(out), out.shape[1])
        return out

    def adjoint(self, table, x, adj_out, input_grads=True, param_grads=True, res_factor=1):
        table, x, adj_out = _f32(table), _f32(x), _f32(adj_out)
        N = x.shape[0]
        adj_x = np.zeros_like(x) if input_grads else None
        grad = np.zeros(self.n_params, dtype=np.float32) if param_grads else None
        lib().qo_hashgrid_adjoint(ctypes.byref(self.s), _ptr(table), _ptr(x), N, x.shape[1],
                                  _ptr(adj_out), adj_out.shape[1], _ptr(adj_x),
                                  x.shape[1], _ptr(grad), int(res_factor))
        return adj_x, grad


class LineIntegration:
    """Fixed-step ray march through a child HashGrid (encoding_line_integration.cpp:43-51 keys:
    start_in, n_in, volume, stepsize, blending)."""

    def __init__(self, cfg):
        if int(cfg["n_in"]) != 3:
            raise ValueError("LineIntegration is only defined for 3D volumes")
        child = dict(cfg["volume"], start_in=0, n_in=3)
        self.child = HashGrid(child)
        self.start_in = int(cfg["start_in"])
        self.stepsize = float(cfg["stepsize"])
        if not self.stepsize > 0:
            raise ValueError("Stepsize must be positive")
        self.blending = {"additive": 0, "average": 1}[cfg["blending"]]
        self.num_outputs = self.child.num_outputs
        self.n_params = self.child.n_params
        self.s = LineStruct()
        self.s.start_in, self.s.blending, self.s.stepsize = self.start_in, self.blending, self.stepsize
        bb_min = child.get("bounding_box_min") or [-0.5] * 3
        bb_size = child.get("bounding_box_size") or [1.0] * 3
        for d in range(3):
            self.s.bb_min[d], self.s.bb_size[d] = bb_min[d], bb_size[d]

    def forward(self, table, x):
        x, table = _f32(x), _f32(table)
        out = np.zeros((x.shape[0], self.num_outputs), np.float32)
        lib().qo_line_forward(ctypes.byref(self.s), ctypes.byref(self.child.s), _ptr(table), _ptr(x),
                              x.shape[0], x.shape[1], _ptr(out), out.shape[1])
        return out

    def adjoint(self, table, x, adj_out, input_grads=True, param_grads=True, res_factor=1):
        x, table, adj_out = _f32(x), _f32(table), _f32(adj_out)
        adj_x = np.zeros_like(x) if input_grads else None
        grad = np.zeros_like(table) if param_grads else None
        lib().qo_line_adjoint(ctypes.byref(self.s), ctypes.byref(self.child.s), _ptr(table), _ptr(x),
                              x.shape[0], x.shape[1], _ptr(adj_out), adj_out.shape[1],
                              _ptr(adj_x) if input_grads else None, x.shape[1],
                              _ptr(grad) if param_grads else None, int(res_factor))
        return adj_x, grad


class Network:
    """The fused network of a JSON spec, evaluated on the CPU in fp32."""

    def __init__(self, cfg, activations=None):
        if isinstance(cfg, str):
            cfg = json.loads(cfg)
        self.cfg = cfg
        acts = dict(BUILTIN_ACTIVATIONS)
        acts.update(activations or {})
        self.n_in = int(cfg["num_inputs"])
        self.n_out = int(cfg["num_outputs"])
        self.encodings = []
        encoded = 0
        for e in cfg["encodings"]:
            if e["id"] == "Identity":
                enc = ("identity", int(e["start_in"]), int(e["n_in"]))
                encoded += enc[2]
                top = enc[1] + enc[2] - 1
            elif e["id"] == "HashGrid":
                g = HashGrid(e)
                enc = ("hashgrid", g)
                encoded += g.num_outputs
                top = g.start_in + g.dim - 1
            elif e["id"] == "LineIntegration":
                li = LineIntegration(e)
                enc = ("line", li)
                encoded += li.num_outputs
                top = li.start_in + 5
            else:
                raise ValueError("No encoding with id '%s' found" % e["id"])
            if top >= self.n_in:
                raise ValueError("encoding input channels out of bounds")
            self.encodings.append(enc)
        self.encoded_channels = encoded
        self.layers = []
        prev = encoded
        for l in cfg["network"]:
            a = l["activation"]
            per_channel = None
            if not isinstance(a, str):
                # one activation per output channel (fused_network.cpp:112-125); channels of
                # the padding take the last one
                if len(a) != int(l["n_out"]):
                    raise ValueError("the number of activations must match the number of output channels")
                per_channel = [acts[x] for x in a]
                a = a[-1]
            self.layers.append(dict(cin=prev, cout=int(l["n_out"]), bias=bool(l["bias"]),
                                    act=acts[a], act_channels=per_channel))
            prev = int(l["n_out"])
        if prev != self.n_out:
            raise ValueError("last layer width does not match num_outputs")
        for i, l in enumerate(self.layers):
            p = round_up(l["cin"], 16)
            l["cin"] = p
            if i > 0:
                self.layers[i - 1]["cout"] = p
        self.layers[-1]["cout"] = round_up(self.layers[-1]["cout"], 16)
        n = 0
        for l in self.layers:
            l["w_start"] = n
            n += l["cin"] * l["cout"]
        for l in self.layers:
            if l["bias"]:
                l["b_start"] = n
                n += l["cout"]
            else:
                l["b_start"] = 0
        self.num_parameters = n
        self.params = None
        self.tables = [None] * len(self.encodings)

    # -- parameters ------------------------------------------------------------
    def set_parameters(self, flat):
        flat = _f32(flat)
        assert flat.shape == (self.num_parameters,)
        self.params = flat

    def set_table(self, enc_index, table):
        g = self.encodings[enc_index][1]
        table = _f32(table)
        assert table.shape == (g.n_params,)
        self.tables[enc_index] = table

    def weight(self, layer, flat=None):
        flat = self.params if flat is None else flat
        l = self.layers[layer]
        return flat[l["w_start"]: l["w_start"] + l["cin"] * l["cout"]].reshape(l["cout"], l["cin"])

    def bias(self, layer, flat=None):
        flat = self.params if flat is None else flat
        l = self.layers[layer]
        if not l["bias"]:
            return None
        return flat[l["b_start"]: l["b_start"] + l["cout"]]

    # -- evaluation ------------------------------------------------------------
    def _struct(self, round_mode, res_factor, grads=None, table_grads=None):
        s = NetworkStruct()
        keep = []
        s.n_in = self.n_in
        s.n_enc = len(self.encodings)
        for i, e in enumerate(self.encodings):
            if e[0] == "identity":
                s.enc_kind[i] = ENC_IDENTITY
                s.enc_start[i], s.enc_nin[i] = e[1], e[2]
            else:
                if e[0] == "line":
                    s.enc_kind[i] = ENC_LINE
                    s.enc_line[i] = ctypes.pointer(e[1].s)
                    s.enc_grid[i] = ctypes.pointer(e[1].child.s)
                else:
                    s.enc_kind[i] = ENC_HASHGRID
                    s.enc_grid[i] = ctypes.pointer(e[1].s)
                assert self.tables[i] is not None, "encoding table not set"
                s.enc_table[i] = _ptr(self.tables[i])
                if table_grads is not None and table_grads[i] is not None:
                    s.enc_grad[i] = _ptr(table_grads[i])
        s.n_layers = len(self.layers)
        for i, l in enumerate(self.layers):
            s.cin[i], s.cout[i] = l["cin"], l["cout"]
            s.act[i], s.act_param[i] = l["act"]
            if l["act_channels"] is not None:
                chans = list(l["act_channels"]) + [l["act_channels"][-1]] * (l["cout"] - len(l["act_channels"]))
                kinds = np.array([c[0] for c in chans], dtype=np.int32)
                prms = np.array([c[1] for c in chans], dtype=np.float32)
                keep += [kinds, prms]
                s.act_channel[i] = kinds.ctypes.data_as(ctypes.POINTER(ctypes.c_int))
                s.act_param_channel[i] = _ptr(prms)
            w = np.ascontiguousarray(self.weight(i))
            keep.append(w)
            s.W[i] = _ptr(w)
            if l["bias"]:
                b = np.ascontiguousarray(self.bias(i))
                keep.append(b)
                s.b[i] = _ptr(b)
            if grads is not None:
                gw = self.weight(i, grads)
                assert gw.flags["C_CONTIGUOUS"]
                s.dW[i] = _ptr(gw)
                if l["bias"]:
                    s.db[i] = _ptr(self.bias(i, grads))
        s.round_mode = int(round_mode)
        s.res_factor = int(res_factor)
        return s, keep

    def forward(self, X, round_mode=0, store=False):
        X = _f32(X)
        N = X.shape[0]
        s, keep = self._struct(round_mode, 1)
        out = np.zeros((N, self.n_out), dtype=np.float32)
        enc_out = np.zeros((N, self.layers[0]["cin"]), dtype=np.float32) if store else None
        pre = [np.zeros((N, l["cout"]), dtype=np.float32) for l in self.layers] if store else None
        pre_ptrs = (_fp * len(self.layers))(*[_ptr(p) for p in pre]) if store else None
        lib().qo_network_forward(ctypes.byref(s), _ptr(X), N, X.shape[1], _ptr(out), self.n_out,
                                 _ptr(enc_out), pre_ptrs)
        if store:
            return out, enc_out, pre
        return out

    def backward(self, X, adj_out, flags, round_mode=0, res_factor=1, return_dpre=False):
        X, adj_out = _f32(X), _f32(adj_out)
        N = X.shape[0]
        _, enc_out, pre = self.forward(X, round_mode, store=True)
        grads = np.zeros(self.num_parameters, dtype=np.float32) if flags & GRAD_WEIGHTS else None
        tgrads = [np.zeros(e[1].n_params, dtype=np.float32)
                  if (e[0] in ("hashgrid", "line") and flags & GRAD_ENCODINGS) else None
                  for e in self.encodings]
        s, keep = self._struct(round_mode, res_factor, grads, tgrads)
        adj_x = np.zeros((N, self.n_in), dtype=np.float32) if flags & GRAD_INPUT else None
        dpre = [np.zeros_like(p) for p in pre] if return_dpre else None
        nl = len(self.layers)
        pre_ptrs = (_fp * nl)(*[_ptr(p) for p in pre])
        dpre_ptrs = (_fp * nl)(*[_ptr(p) for p in dpre]) if return_dpre else None
        lib().qo_network_backward(ctypes.byref(s), _ptr(X), N, X.shape[1], _ptr(adj_out),
                                  self.n_out, int(flags), _ptr(enc_out), pre_ptrs, _ptr(adj_x),
                                  dpre_ptrs)
        res = dict(adj_x=adj_x, grads=grads, table_grads=tgrads, pre=pre, enc_out=enc_out)
        if return_dpre:
            res["dpre"] = dpre
        return res


def compare(actual, expected, rel=1e-2, abs_=1e-3):
    """Fraction of entries with |a-e| > abs + rel*|e| and the largest violation ratio."""
    a = np.asarray(actual, dtype=np.float64)
    e = np.asarray(expected, dtype=np.float64)
    assert a.shape == e.shape, (a.shape, e.shape)
    if a.size == 0:
        return 0.0, 0.0
    err = np.abs(a - e)
    tol = abs_ + rel * np.abs(e)
    bad = ~(err <= tol)
    return float(bad.mean()), float(np.nanmax(err / tol))
