"""CPU restatement of the reference's pull-push inpainting (test infrastructure only).

The shipped library never imports this module; the tests do. Everything runs in the dtype
of the inputs (use float64 for the checks). Two forms of every level operation:

* ``*_loops``: pure-Python loops, one statement per statement of the reference's kernels
  (src_cpp/include/qmlp/kernels/pullpush.cuh:24-301) - for small images only;
* the vectorised numpy form used for larger images, checked against the loops in the tests.

The recursion over the image pyramid follows src_cpp/src/utils.cpp:37-110 (forward) and
:182-303 (adjoint). One deliberate divergence: the adjoint of the down-sampling adds the
contributions of ALL low-res pixels whose window holds a high-res pixel; the reference adds
without atomics (pullpush.cuh:155 "every high-res pixel is accessed only once"), which is
only true for even sizes - for odd sizes the windows overlap and its result depends on the
thread order.

What pins this module (tests/test_pullpush_oracle.py): the down-sampling with a uniform mask
against torch's adaptive average / max pooling, the up-sampling with full low-res masks
against torch's bilinear interpolation, closed forms of the whole pyramid (full mask =
identity, constant data stays constant, a single known pixel floods the image), and every
gradient against central finite differences in float64.
"""
import math

import numpy as np

# bilinear weights of the 4 low-res neighbours (pullpush.cuh:98-101)
_W = (0.75 * 0.75, 0.25 * 0.75, 0.25 * 0.75, 0.25 * 0.25)


def start_index(a, b, c):
    """pullpush.cuh:24-26 (evaluated in fp32 there; exact for every size below 2^24)."""
    return int(math.floor(np.float32(a * c) / np.float32(b)))


def end_index(a, b, c):
    """pullpush.cuh:28-30."""
    return int(math.ceil(np.float32((a + 1) * c) / np.float32(b)))


def _neighbours(i, j):
    """pullpush.cuh:85-86, 98-101: (ii, jj, w) of the 4 low-res neighbours of pixel (i, j)."""
    io = -1 if i % 2 == 0 else +1
    jo = -1 if j % 2 == 0 else +1
    return ((i // 2, j // 2, _W[0]), (i // 2 + io, j // 2, _W[1]),
            (i // 2, j // 2 + jo, _W[2]), (i // 2 + io, j // 2 + jo, _W[3]))


# ---------------------------------------------------------------------------------------
# loops: the direct restatement
# ---------------------------------------------------------------------------------------

def down_loops(mask, data):
    """FastInpaintingFractionalKernel_Down, pullpush.cuh:32-65."""
    B, C, H, W = data.shape
    oH, oW = H // 2, W // 2
    mask_low = np.zeros((B, oH, oW), mask.dtype)
    data_low = np.zeros((B, C, oH, oW), data.dtype)
    for b in range(B):
        for i in range(oH):
            for j in range(oW):
                n1 = mask.dtype.type(0)
                n2 = mask.dtype.type(0)
                d = np.zeros(C, data.dtype)
                for jj in range(start_index(j, oW, W), end_index(j, oW, W)):
                    for ii in range(start_index(i, oH, H), end_index(i, oH, H)):
                        n1 += mask[b, ii, jj]
                        n2 = max(n2, mask[b, ii, jj])
                        d += mask[b, ii, jj] * data[b, :, ii, jj]
                mask_low[b, i, j] = n2
                data_low[b, :, i, j] = d / n1 if n1 > 0 else 0
    return mask_low, data_low


def up_loops(mask, data, mask_low, data_low):
    """FastInpaintingFractionalKernel_Up, pullpush.cuh:67-114."""
    B, C, H, W = data.shape
    oH, oW = H // 2, W // 2
    mask_high = np.zeros_like(mask)
    data_high = np.zeros_like(data)
    for b in range(B):
        for i in range(H):
            for j in range(W):
                weight = mask.dtype.type(0)
                n = mask.dtype.type(0)
                d = np.zeros(C, data.dtype)
                for ii, jj, w in _neighbours(i, j):
                    if 0 <= ii < oH and 0 <= jj < oW:
                        weight += w
                        n += w * mask_low[b, ii, jj]
                        d += w * mask_low[b, ii, jj] * data_low[b, :, ii, jj]
                m = mask[b, i, j]
                mask_high[b, i, j] = m + ((1 - m) * (n / weight) if n > 0 else 0)
                data_high[b, :, i, j] = m * data[b, :, i, j] + (1 - m) * (d / n if n > 0 else 0)
    return mask_high, data_high


def adjoint_down_loops(mask, data, grad_mask_low, grad_data_low, grad_mask, grad_data):
    """AdjFastInpaintingFractionKernel_Down, pullpush.cuh:119-182; adds into grad_mask, grad_data."""
    B, C, H, W = data.shape
    oH, oW = H // 2, W // 2
    for b in range(B):
        for i in range(oH):
            for j in range(oW):
                rows = range(start_index(i, oH, H), end_index(i, oH, H))
                cols = range(start_index(j, oW, W), end_index(j, oW, W))
                n1 = mask.dtype.type(0)
                n2 = mask.dtype.type(0)
                d = np.zeros(C, data.dtype)
                for jj in cols:
                    for ii in rows:
                        n1 += mask[b, ii, jj]
                        n2 = max(n2, mask[b, ii, jj])
                        d += mask[b, ii, jj] * data[b, :, ii, jj]
                g = grad_data_low[b, :, i, j]
                adj_d = g / n1 if n1 > 0 else np.zeros(C, data.dtype)
                adj_n1 = -np.sum(g * d / (n1 * n1)) if n1 > 0 else 0
                adj_n2 = grad_mask_low[b, i, j]
                for jj in cols:
                    for ii in rows:
                        grad_data[b, :, ii, jj] += adj_d * mask[b, ii, jj]
                        adj_mask = np.sum(adj_d * data[b, :, ii, jj]) + adj_n1
                        if n2 == mask[b, ii, jj]:
                            adj_mask += adj_n2
                        grad_mask[b, ii, jj] += adj_mask


def adjoint_up_loops(mask, data, mask_low, data_low, grad_mask_high, grad_data_high,
                     grad_mask, grad_data, grad_mask_low, grad_data_low):
    """AdjFastInpaintingFractionalKernel_Up, pullpush.cuh:184-277; adds into the last four."""
    B, C, H, W = data.shape
    oH, oW = H // 2, W // 2
    for b in range(B):
        for i in range(H):
            for j in range(W):
                weight = mask.dtype.type(0)
                n = mask.dtype.type(0)
                d = np.zeros(C, data.dtype)
                inside = [(ii, jj, w) for ii, jj, w in _neighbours(i, j) if 0 <= ii < oH and 0 <= jj < oW]
                for ii, jj, w in inside:
                    weight += w
                    n += w * mask_low[b, ii, jj]
                    d += w * mask_low[b, ii, jj] * data_low[b, :, ii, jj]
                m = mask[b, i, j]
                g = grad_data_high[b, :, i, j]
                filled = d / n if n > 0 else np.zeros(C, data.dtype)
                adj_mask = np.sum(g * (data[b, :, i, j] - filled))
                grad_data[b, :, i, j] += g * m
                adj_n = -np.sum(g * (1 - m) * d / (n * n)) if n > 0 else 0
                adj_d = g * (1 - m) / n if n > 0 else np.zeros(C, data.dtype)
                gm = grad_mask_high[b, i, j]
                adj_mask += gm * (1 - n / weight)
                adj_n += gm * ((1 - m) / weight)
                grad_mask[b, i, j] += adj_mask
                for ii, jj, w in inside:
                    grad_data_low[b, :, ii, jj] += adj_d * w * mask_low[b, ii, jj]
                    grad_mask_low[b, ii, jj] += np.sum(adj_d * w * data_low[b, :, ii, jj]) + adj_n * w


# ---------------------------------------------------------------------------------------
# vectorised numpy forms of the same operations
# ---------------------------------------------------------------------------------------

def _windows(n_low, n_high):
    """Window start and length of every low-res index along one axis."""
    start = np.array([start_index(a, n_low, n_high) for a in range(n_low)], dtype=np.int64)
    end = np.array([end_index(a, n_low, n_high) for a in range(n_low)], dtype=np.int64)
    return start, end - start


def _window_taps(H, W):
    """All (rows, cols, valid) index arrays, one per offset inside the (at most 3x3) windows."""
    oH, oW = H // 2, W // 2
    si, li = _windows(oH, H)
    sj, lj = _windows(oW, W)
    taps = []
    for di in range(int(li.max(initial=0))):
        for dj in range(int(lj.max(initial=0))):
            valid = (di < li)[:, None] & (dj < lj)[None, :]
            rows = np.minimum(si + di, H - 1)[:, None] + np.zeros((1, oW), np.int64)
            cols = np.minimum(sj + dj, W - 1)[None, :] + np.zeros((oH, 1), np.int64)
            taps.append((rows, cols, valid))
    return taps


def down(mask, data):
    B, C, H, W = data.shape
    oH, oW = H // 2, W // 2
    n1 = np.zeros((B, oH, oW), mask.dtype)
    n2 = np.zeros((B, oH, oW), mask.dtype)
    d = np.zeros((B, C, oH, oW), data.dtype)
    for rows, cols, valid in _window_taps(H, W):
        m = np.where(valid, mask[:, rows, cols], 0)
        n1 += m
        n2 = np.maximum(n2, m)
        d += m[:, None] * data[:, :, rows, cols]
    safe = np.where(n1 > 0, n1, 1)
    return n2, np.where(n1[:, None] > 0, d / safe[:, None], 0).astype(data.dtype)


def _neighbour_taps(H, W):
    oH, oW = H // 2, W // 2
    i = np.arange(H)[:, None] + np.zeros((1, W), np.int64)
    j = np.arange(W)[None, :] + np.zeros((H, 1), np.int64)
    io = np.where(i % 2 == 0, -1, 1)
    jo = np.where(j % 2 == 0, -1, 1)
    taps = []
    for (ii, jj), w in zip(((i // 2, j // 2), (i // 2 + io, j // 2), (i // 2, j // 2 + jo), (i // 2 + io, j // 2 + jo)), _W):
        inside = (ii >= 0) & (jj >= 0) & (ii < oH) & (jj < oW)
        taps.append((np.clip(ii, 0, max(oH - 1, 0)), np.clip(jj, 0, max(oW - 1, 0)), inside, w))
    return taps


def _up_sums(mask_low, data_low, H, W):
    B, C = data_low.shape[:2]
    weight = np.zeros((H, W), mask_low.dtype)
    n = np.zeros((B, H, W), mask_low.dtype)
    d = np.zeros((B, C, H, W), data_low.dtype)
    for ii, jj, inside, w in _neighbour_taps(H, W):
        ml = np.where(inside, mask_low[:, ii, jj], 0)
        weight += np.where(inside, w, 0).astype(mask_low.dtype)
        n += w * ml
        d += (w * ml)[:, None] * data_low[:, :, ii, jj]
    return weight, n, d


def up(mask, data, mask_low, data_low):
    H, W = mask.shape[1:]
    weight, n, d = _up_sums(mask_low, data_low, H, W)
    pos = n > 0
    safe = np.where(pos, n, 1)
    mask_high = mask + np.where(pos, (1 - mask) * (n / weight), 0)
    data_high = mask[:, None] * data + (1 - mask)[:, None] * np.where(pos[:, None], d / safe[:, None], 0)
    return mask_high.astype(mask.dtype), data_high.astype(data.dtype)


def adjoint_down(mask, data, grad_mask_low, grad_data_low, grad_mask, grad_data):
    B, C, H, W = data.shape
    taps = _window_taps(H, W)
    oH, oW = H // 2, W // 2
    n1 = np.zeros((B, oH, oW), mask.dtype)
    n2 = np.zeros((B, oH, oW), mask.dtype)
    d = np.zeros((B, C, oH, oW), data.dtype)
    for rows, cols, valid in taps:
        m = np.where(valid, mask[:, rows, cols], 0)
        n1 += m
        n2 = np.maximum(n2, m)
        d += m[:, None] * data[:, :, rows, cols]
    pos = n1 > 0
    safe = np.where(pos, n1, 1)
    adj_d = np.where(pos[:, None], grad_data_low / safe[:, None], 0)
    adj_n1 = -np.where(pos, np.sum(grad_data_low * d, axis=1) / (safe * safe), 0)
    bidx = np.arange(B)[:, None, None]
    for rows, cols, valid in taps:
        m = mask[:, rows, cols]
        adj_mask = np.sum(adj_d * data[:, :, rows, cols], axis=1) + adj_n1 + np.where(n2 == m, grad_mask_low, 0)
        np.add.at(grad_mask, (bidx, rows[None], cols[None]), np.where(valid, adj_mask, 0))
        np.add.at(grad_data, (bidx[:, None], np.arange(C)[None, :, None, None], rows[None, None], cols[None, None]),
                  np.where(valid, adj_d * m[:, None], 0))


def adjoint_up(mask, data, mask_low, data_low, grad_mask_high, grad_data_high,
               grad_mask, grad_data, grad_mask_low, grad_data_low):
    B, C, H, W = data.shape
    weight, n, d = _up_sums(mask_low, data_low, H, W)
    pos = n > 0
    safe = np.where(pos, n, 1)
    filled = np.where(pos[:, None], d / safe[:, None], 0)
    one_m = 1 - mask
    adj_mask = np.sum(grad_data_high * (data - filled), axis=1)
    grad_data += grad_data_high * mask[:, None]
    adj_n = -np.where(pos, np.sum(grad_data_high * d, axis=1) * one_m / (safe * safe), 0)
    adj_d = np.where(pos[:, None], grad_data_high * (one_m / safe)[:, None], 0)
    adj_mask += grad_mask_high * (1 - n / weight)
    adj_n += grad_mask_high * (one_m / weight)
    grad_mask += adj_mask
    bidx = np.arange(B)[:, None, None]
    for ii, jj, inside, w in _neighbour_taps(H, W):
        ml = mask_low[:, ii, jj]
        dl = data_low[:, :, ii, jj]
        np.add.at(grad_data_low, (bidx[:, None], np.arange(C)[None, :, None, None], ii[None, None], jj[None, None]),
                  np.where(inside, adj_d * w * ml[:, None], 0))
        np.add.at(grad_mask_low, (bidx, ii[None], jj[None]),
                  np.where(inside, np.sum(adj_d * w * dl, axis=1) + adj_n * w, 0))


# ---------------------------------------------------------------------------------------
# the pyramid
# ---------------------------------------------------------------------------------------

_LOOPS = {"down": down_loops, "up": up_loops, "adjoint_down": adjoint_down_loops, "adjoint_up": adjoint_up_loops}
_NUMPY = {"down": down, "up": up, "adjoint_down": adjoint_down, "adjoint_up": adjoint_up}


def _forward(mask, data, ops, saved):
    """fractionalPullpush_recursion, utils.cpp:37-110; returns (mask_out, data_out)."""
    H, W = mask.shape[1:]
    if H <= 1 or W <= 1:
        return mask.copy(), data.copy()
    mask_low_pre, data_low_pre = ops["down"](mask, data)
    mask_low_post, data_low_post = _forward(mask_low_pre, data_low_pre, ops, saved)
    saved.append((mask_low_pre, data_low_pre, mask_low_post, data_low_post))
    return ops["up"](mask, data, mask_low_post, data_low_post)


def _adjoint(mask, data, grad_mask_out, grad_data_out, grad_mask, grad_data, ops, saved):
    """adjointFractionalPullpush_recursion, utils.cpp:182-303."""
    H, W = mask.shape[1:]
    if H <= 1 or W <= 1:
        grad_mask += grad_mask_out
        grad_data += grad_data_out
        return
    mask_low_pre, data_low_pre, mask_low_post, data_low_post = saved.pop()
    g_mask_low_post = np.zeros_like(mask_low_pre)
    g_data_low_post = np.zeros_like(data_low_pre)
    ops["adjoint_up"](mask, data, mask_low_post, data_low_post, grad_mask_out, grad_data_out,
                      grad_mask, grad_data, g_mask_low_post, g_data_low_post)
    g_mask_low_pre = np.zeros_like(mask_low_pre)
    g_data_low_pre = np.zeros_like(data_low_pre)
    _adjoint(mask_low_pre, data_low_pre, g_mask_low_post, g_data_low_post, g_mask_low_pre, g_data_low_pre, ops, saved)
    ops["adjoint_down"](mask, data, g_mask_low_pre, g_data_low_pre, grad_mask, grad_data)


def _check(mask, data):
    assert mask.ndim == 3 and data.ndim == 4 and mask.dtype == data.dtype
    assert mask.shape == (data.shape[0],) + data.shape[2:]
    assert data.shape[1] < 16          # utils.cpp:135


def pullpush(mask, data, loops=False):
    """Utils::fractionalPullpush, utils.cpp:112-143: the inpainted data (B, C, H, W)."""
    _check(mask, data)
    return _forward(mask, data, _LOOPS if loops else _NUMPY, [])[1]


def pullpush_adjoint(mask, data, adj_output, loops=False):
    """Utils::adjointFractionalPullpush, utils.cpp:305-358: (adj_mask, adj_data)."""
    _check(mask, data)
    ops = _LOOPS if loops else _NUMPY
    saved = []
    _forward(mask, data, ops, saved)
    grad_mask = np.zeros_like(mask)
    grad_data = np.zeros_like(data)
    _adjoint(mask, data, np.zeros_like(mask), adj_output, grad_mask, grad_data, ops, saved)
    return grad_mask, grad_data
