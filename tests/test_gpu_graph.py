"""The library launches kernels only (no allocation, no memset, no synchronisation), so a
sequence of its calls can be captured into a HIP graph on the caller's stream.  The test
captures one training-style sequence (conv forward, batch norm, ReLU, max pool and the
backward passes), replays it several times with new inputs and the program's own eager
work and synchronisations in between, and checks every replay against the eager result."""
import numpy as np
import pytest
import torch

import flashlight_amd as fa
from flashlight_amd import ops

pytestmark = pytest.mark.gpu


def _sequence(x, w, b, g, beta, rm, rv, dy):
    kw = dict(sx=1, sy=1, px=1, py=1, dx=1, dy=1, groups=1)
    y = fa.conv2d(x, w, b, **kw)
    n, sm, si = fa.batchnorm(y, g, beta, rm, rv, [2], True, 0.1, 1e-5)
    r = ops.relu(n)
    p, am = fa.pool2d(r, 2, 2, 2, 2, 0, 0, mode=0, train=True)
    dr = fa.pool2d_backward(dy, tuple(r.shape), am, 2, 2, 2, 2, 0, 0, mode=0)
    dn = ops.relu_backward(dr, n)
    dyc, dg, dbeta = fa.batchnorm_backward(dn, y, g, sm, si, [2])
    dx = fa.conv2d_backward_data(dyc, tuple(x.shape), w, **kw)
    dw, db = fa.conv2d_backward_filter_bias(dyc, x, tuple(w.shape), True, **kw)
    return p, dx, dw, db, dg, dbeta


def test_capture_and_replay_matches_eager():
    dev = torch.device("cuda:0")
    gen = torch.Generator(device="cuda").manual_seed(5)
    N, C, H, W, K = 4, 32, 16, 16, 64
    rnd = lambda *s: torch.randn(*s, device=dev, generator=gen)
    x, w, b = rnd(N, C, H, W), rnd(K, C, 3, 3) / 17, rnd(K)
    g, beta, dy = 1 + 0.1 * rnd(K), rnd(K), rnd(N, K, H // 2, W // 2)
    rm, rv = torch.zeros(K, device=dev), torch.ones(K, device=dev)
    # warm-up on a side stream, as torch's graph capture asks
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            _sequence(x, w, b, g, beta, rm.clone(), rv.clone(), dy)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    rm_g, rv_g = rm.clone(), rv.clone()
    with torch.cuda.graph(graph):
        outs = _sequence(x, w, b, g, beta, rm_g, rv_g, dy)
    for it in range(3):
        # new inputs in the captured buffers, eager work of this program and a
        # synchronisation between the replays
        x.copy_(rnd(N, C, H, W))
        dy.copy_(rnd(N, K, H // 2, W // 2))
        rm_e, rv_e = rm_g.clone(), rv_g.clone()
        want = [t.clone() for t in _sequence(x, w, b, g, beta, rm_e, rv_e, dy)]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(outs, want):
            assert torch.equal(got, ref), it
        assert torch.equal(rm_g, rm_e) and torch.equal(rv_g, rv_e)


def test_rnn_capture_and_replay_matches_eager():
    dev = torch.device("cuda:0")
    gen = torch.Generator(device="cuda").manual_seed(9)
    I, H, L, T, B = 24, 32, 2, 6, 5
    n = ops.rnn_param_count(I, H, L, ops.RNN_LSTM, True)
    x = torch.randn(T, B, I, device=dev, generator=gen)
    w = torch.randn(n, device=dev, generator=gen) / H ** 0.5
    dy = torch.randn(T, B, 2 * H, device=dev, generator=gen)

    def seq():
        y, hy, cy, reserve = ops.rnn(x, None, None, w, H, L, ops.RNN_LSTM, True)
        dx, dhx, dcx, dw = ops.rnn_backward(x, w, reserve, H, L, ops.RNN_LSTM, True, dy)
        return y, hy, cy, dx, dw

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        seq()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = seq()
    for it in range(3):
        x.copy_(torch.randn(T, B, I, device=dev, generator=gen))
        want = [t.clone() for t in seq()]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(outs, want):
            assert torch.equal(got, ref), it
