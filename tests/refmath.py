"""Brute-force definitions and comparison helpers shared by the tests.

Everything here is written straight from the textbook definition with explicit
Python loops (tiny inputs only) so that it shares no code and no loop structure
with oracle/flref.c.
"""
import numpy as np


def rel_l2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    den = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / den) if den > 0 else float(np.linalg.norm(a - b))


def conv_out(H, K, s, p, d):
    return 1 + (H + 2 * p - (1 + (K - 1) * d)) // s


def brute_conv_fwd(x, w, b, stride, pad, dil, groups):
    x = x.astype(np.float64); w = w.astype(np.float64)
    N, C, H, W = x.shape
    K, Cg, KH, KW = w.shape
    sy, sx = stride; py, px = pad; dy_, dx_ = dil
    OH, OW = conv_out(H, KH, sy, py, dy_), conv_out(W, KW, sx, px, dx_)
    Kg = K // groups
    y = np.zeros((N, K, OH, OW))
    for n in range(N):
        for k in range(K):
            g = k // Kg
            for oh in range(OH):
                for ow in range(OW):
                    s = float(b[k]) if b is not None else 0.0
                    for c in range(Cg):
                        for kh in range(KH):
                            ih = oh * sy - py + kh * dy_
                            if ih < 0 or ih >= H:
                                continue
                            for kw in range(KW):
                                iw = ow * sx - px + kw * dx_
                                if iw < 0 or iw >= W:
                                    continue
                                s += x[n, g * Cg + c, ih, iw] * w[k, c, kh, kw]
                    y[n, k, oh, ow] = s
    return y


def brute_conv_bwd(x, w, dy, stride, pad, dil, groups):
    """(dx, dw, db) by accumulating every product of the forward definition."""
    x = x.astype(np.float64); w = w.astype(np.float64); dy = dy.astype(np.float64)
    N, C, H, W = x.shape
    K, Cg, KH, KW = w.shape
    sy, sx = stride; py, px = pad; dy_, dx_ = dil
    OH, OW = dy.shape[2:]
    Kg = K // groups
    gx = np.zeros_like(x); gw = np.zeros_like(w)
    for n in range(N):
        for k in range(K):
            g = k // Kg
            for oh in range(OH):
                for ow in range(OW):
                    go = dy[n, k, oh, ow]
                    for c in range(Cg):
                        for kh in range(KH):
                            ih = oh * sy - py + kh * dy_
                            if ih < 0 or ih >= H:
                                continue
                            for kw in range(KW):
                                iw = ow * sx - px + kw * dx_
                                if iw < 0 or iw >= W:
                                    continue
                                gx[n, g * Cg + c, ih, iw] += go * w[k, c, kh, kw]
                                gw[k, c, kh, kw] += go * x[n, g * Cg + c, ih, iw]
    return gx, gw, dy.sum(axis=(0, 2, 3))


def brute_pool_fwd(x, window, stride, pad, mode):
    """Returns (y, argmax) in float32 arithmetic; first maximum in (kh, kw) scan
    under strict '>' with padded positions skipped."""
    N, C, H, W = x.shape
    wy, wx = window; sy, sx = stride; py, px = pad
    OH = 1 + (H + 2 * py - wy) // sy
    OW = 1 + (W + 2 * px - wx) // sx
    y = np.zeros((N, C, OH, OW), np.float32)
    am = np.zeros((N, C, OH, OW), np.uint8)
    for n in range(N):
        for c in range(C):
            for oh in range(OH):
                for ow in range(OW):
                    vals = []
                    for kh in range(wy):
                        for kw in range(wx):
                            ih, iw = oh * sy - py + kh, ow * sx - px + kw
                            if 0 <= ih < H and 0 <= iw < W:
                                vals.append((kh * wx + kw, np.float32(x[n, c, ih, iw])))
                    if mode == 0:
                        best_i, best_v = vals[0]
                        for i, v in vals[1:]:
                            if v > best_v:
                                best_i, best_v = i, v
                        y[n, c, oh, ow] = best_v
                        am[n, c, oh, ow] = best_i
                    else:
                        s = np.float32(0)
                        for _, v in vals:
                            s = np.float32(s + v)
                        div = wy * wx if mode == 1 else len(vals)
                        y[n, c, oh, ow] = np.float32(s / np.float32(div))
    return y, am


def brute_pool_bwd(dy, am, x_shape, window, stride, pad, mode):
    N, C, H, W = x_shape
    wy, wx = window; sy, sx = stride; py, px = pad
    OH, OW = dy.shape[2:]
    dx = np.zeros(x_shape, np.float32)
    for n in range(N):
        for c in range(C):
            for oh in range(OH):
                for ow in range(OW):
                    g = np.float32(dy[n, c, oh, ow])
                    if mode == 0:
                        i = int(am[n, c, oh, ow])
                        ih, iw = oh * sy - py + i // wx, ow * sx - px + i % wx
                        dx[n, c, ih, iw] = np.float32(dx[n, c, ih, iw] + g)
                        continue
                    pos = [(oh * sy - py + kh, ow * sx - px + kw)
                           for kh in range(wy) for kw in range(wx)]
                    pos = [(a, b) for a, b in pos if 0 <= a < H and 0 <= b < W]
                    div = wy * wx if mode == 1 else len(pos)
                    q = np.float32(g / np.float32(div))
                    for a, b in pos:
                        dx[n, c, a, b] = np.float32(dx[n, c, a, b] + q)
    return dx
