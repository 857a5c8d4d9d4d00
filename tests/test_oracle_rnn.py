"""Pins the rnn / rnnBackward restatement of oracle/flref.c against PyTorch-CPU's
nn.RNN / nn.LSTM / nn.GRU in float64 (forward and autograd), with the flat weight vector
unpacked in cuDNN's order, and against the parameter counts the reference's own test
uses (flashlight/fl/test/autograd/AutogradRnnTest.cpp:37-49)."""
import numpy as np
import pytest
import torch

from oracle import flref
from refmath import rel_l2

GATES = {flref.RNN_RELU: 1, flref.RNN_TANH: 1, flref.RNN_LSTM: 4, flref.RNN_GRU: 3}


def torch_module(mode, I, H, L, bidir, w):
    """nn module in float64 whose parameters are views of the flat cuDNN-ordered vector."""
    D = 2 if bidir else 1
    G = GATES[mode]
    if mode == flref.RNN_LSTM:
        m = torch.nn.LSTM(I, H, L, bidirectional=bidir)
    elif mode == flref.RNN_GRU:
        m = torch.nn.GRU(I, H, L, bidirectional=bidir)
    else:
        m = torch.nn.RNN(I, H, L, bidirectional=bidir, nonlinearity="relu" if mode == flref.RNN_RELU else "tanh")
    m = m.double()
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    off = 0
    views = {}
    for l in range(L):
        inl = I if l == 0 else D * H
        for dr in range(D):
            sfx = "_l%d%s" % (l, "_reverse" if dr else "")
            views["weight_ih" + sfx] = wt[off:off + G * H * inl].reshape(G * H, inl)
            off += G * H * inl
            views["weight_hh" + sfx] = wt[off:off + G * H * H].reshape(G * H, H)
            off += G * H * H
    for l in range(L):
        for dr in range(D):
            sfx = "_l%d%s" % (l, "_reverse" if dr else "")
            views["bias_ih" + sfx] = wt[off:off + G * H]
            off += G * H
            views["bias_hh" + sfx] = wt[off:off + G * H]
            off += G * H
    assert off == wt.numel()
    return m, wt, views


def one_layer_module(mode, I, H, bidir):
    if mode == flref.RNN_LSTM:
        return torch.nn.LSTM(I, H, 1, bidirectional=bidir).double()
    if mode == flref.RNN_GRU:
        return torch.nn.GRU(I, H, 1, bidirectional=bidir).double()
    return torch.nn.RNN(I, H, 1, bidirectional=bidir, nonlinearity="relu" if mode == flref.RNN_RELU else "tanh").double()


@pytest.mark.parametrize("mode,nparams", [(flref.RNN_TANH, 56), (flref.RNN_LSTM, 224), (flref.RNN_GRU, 168)])
def test_param_count_of_the_reference_test(mode, nparams):
    # AutogradRnnTest.cpp: 2 layers, hidden 2, input 2, bidirectional
    assert flref.rnn_param_count(flref.rnn_desc(2, 2, 2, True, mode, 3, 2)) == nparams


@pytest.mark.parametrize("mode", [flref.RNN_RELU, flref.RNN_TANH, flref.RNN_LSTM, flref.RNN_GRU])
@pytest.mark.parametrize("I,H,L,bidir,T,B,states", [
    (2, 2, 2, True, 3, 2, False),       # the reference test's sizes
    (5, 7, 1, False, 6, 3, True),
    (4, 3, 3, True, 5, 2, True),
    (6, 4, 2, False, 1, 4, False),      # a single step
])
def test_rnn_against_torch_float64(mode, I, H, L, bidir, T, B, states):
    rng = np.random.default_rng(100 * mode + I + H + L + T)
    D = 2 if bidir else 1
    d = flref.rnn_desc(I, H, L, bidir, mode, T, B)
    w = (rng.standard_normal(flref.rnn_param_count(d)) * 0.4).astype(np.float32)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    hx = rng.standard_normal((L * D, B, H)).astype(np.float32) if states else None
    cx = rng.standard_normal((L * D, B, H)).astype(np.float32) if states and mode == flref.RNN_LSTM else None
    dy = rng.standard_normal((T, B, D * H)).astype(np.float32)
    dhy = rng.standard_normal((L * D, B, H)).astype(np.float32)
    dcy = rng.standard_normal((L * D, B, H)).astype(np.float32) if mode == flref.RNN_LSTM else None

    m, wt, views = torch_module(mode, I, H, L, bidir, w)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    h0 = torch.tensor(hx if hx is not None else np.zeros((L * D, B, H)), dtype=torch.float64, requires_grad=True)
    c0 = torch.tensor(cx if cx is not None else np.zeros((L * D, B, H)), dtype=torch.float64, requires_grad=True)
    state = (h0, c0) if mode == flref.RNN_LSTM else h0
    out, last = torch.func.functional_call(m, views, (xt, state))
    hn, cn = last if mode == flref.RNN_LSTM else (last, None)
    loss = (out * torch.tensor(dy, dtype=torch.float64)).sum() + (hn * torch.tensor(dhy, dtype=torch.float64)).sum()
    if cn is not None:
        loss = loss + (cn * torch.tensor(dcy, dtype=torch.float64)).sum()
    loss.backward()

    y, hy, cy = flref.rnn_fwd(d, x, w, hx, cx)
    assert rel_l2(y, out.detach().numpy()) < 1e-6
    assert rel_l2(hy, hn.detach().numpy()) < 1e-6
    if cn is not None:
        assert rel_l2(cy, cn.detach().numpy()) < 1e-6
    dx, dhx, dcx, dw = flref.rnn_bwd(d, x, w, hx, cx, dy, dhy, dcy)
    assert rel_l2(dx, xt.grad.numpy()) < 1e-5
    assert rel_l2(dhx, h0.grad.numpy()) < 1e-5
    if mode == flref.RNN_LSTM:
        assert rel_l2(dcx, c0.grad.numpy()) < 1e-5
    assert rel_l2(dw, wt.grad.numpy()) < 1e-5


def test_missing_gradients_count_as_zero():
    # the closure passes empty tensors for outputs nobody differentiated (Functions.cpp:1677-1699)
    rng = np.random.default_rng(5)
    d = flref.rnn_desc(3, 4, 2, True, flref.RNN_LSTM, 4, 2)
    w = (rng.standard_normal(flref.rnn_param_count(d)) * 0.4).astype(np.float32)
    x = rng.standard_normal((4, 2, 3)).astype(np.float32)
    dy = rng.standard_normal((4, 2, 8)).astype(np.float32)
    z = np.zeros((4, 2, 4), np.float32)
    a = flref.rnn_bwd(d, x, w, None, None, dy, None, None)
    b = flref.rnn_bwd(d, x, w, z, z, dy, z, z)
    for u, v in zip(a, b):
        assert np.array_equal(u, v)


@pytest.mark.parametrize("mode", [flref.RNN_RELU, flref.RNN_TANH, flref.RNN_LSTM, flref.RNN_GRU])
@pytest.mark.parametrize("I,H,L,bidir,T,B,p", [
    (3, 4, 2, True, 4, 3, 0.5),
    (5, 6, 3, False, 5, 2, 0.25),
])
def test_rnn_dropout_between_layers_against_torch(mode, I, H, L, bidir, T, B, p):
    """Dropout (cuDNN: on the output sequence of every layer but the last, scaled by 1 / (1 - p),
    states untouched; backend/cudnn/RNN.cpp:83-90) against a stack of one-layer torch modules with
    the same keep masks between them, forward and autograd in float64."""
    rng = np.random.default_rng(300 + 10 * mode + L)
    D = 2 if bidir else 1
    seed = 0x1234567890ABCDEF
    d = flref.rnn_desc(I, H, L, bidir, mode, T, B, dropout=p, seed=seed)
    w = (rng.standard_normal(flref.rnn_param_count(d)) * 0.4).astype(np.float32)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    hx = rng.standard_normal((L * D, B, H)).astype(np.float32)
    cx = rng.standard_normal((L * D, B, H)).astype(np.float32) if mode == flref.RNN_LSTM else None
    dy = rng.standard_normal((T, B, D * H)).astype(np.float32)
    dhy = rng.standard_normal((L * D, B, H)).astype(np.float32)
    dcy = rng.standard_normal((L * D, B, H)).astype(np.float32) if mode == flref.RNN_LSTM else None

    _, wt, views = torch_module(mode, I, H, L, bidir, w)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    h0 = torch.tensor(hx, dtype=torch.float64, requires_grad=True)
    c0 = torch.tensor(cx if cx is not None else np.zeros_like(hx), dtype=torch.float64, requires_grad=True)
    cur, hs, cs = xt, [], []
    for l in range(L):
        inl = I if l == 0 else D * H
        one = one_layer_module(mode, inl, H, bidir)
        lv = {k.replace("_l%d" % l, "_l0"): v for k, v in views.items() if "_l%d" % l in k}
        hl, cl = h0[l * D:(l + 1) * D], c0[l * D:(l + 1) * D]
        out, last = torch.func.functional_call(one, lv, (cur, (hl, cl) if mode == flref.RNN_LSTM else hl))
        hn, cn = last if mode == flref.RNN_LSTM else (last, None)
        hs.append(hn)
        cs.append(cn)
        if l + 1 < L:
            keep = flref.dropout_keep(seed, l, out.numel(), p).reshape(out.shape)
            out = out * torch.tensor(keep, dtype=torch.float64) / (1.0 - p)
        cur = out
    hn = torch.cat(hs)
    loss = (cur * torch.tensor(dy, dtype=torch.float64)).sum() + (hn * torch.tensor(dhy, dtype=torch.float64)).sum()
    if mode == flref.RNN_LSTM:
        loss = loss + (torch.cat(cs) * torch.tensor(dcy, dtype=torch.float64)).sum()
    loss.backward()

    y, hy, cy = flref.rnn_fwd(d, x, w, hx, cx)
    assert rel_l2(y, cur.detach().numpy()) < 1e-6
    assert rel_l2(hy, hn.detach().numpy()) < 1e-6
    dx, dhx, dcx, dw = flref.rnn_bwd(d, x, w, hx, cx, dy, dhy, dcy)
    assert rel_l2(dx, xt.grad.numpy()) < 1e-5
    assert rel_l2(dhx, h0.grad.numpy()) < 1e-5
    if mode == flref.RNN_LSTM:
        assert rel_l2(dcx, c0.grad.numpy()) < 1e-5
    assert rel_l2(dw, wt.grad.numpy()) < 1e-5
    # the mask really drops and really keeps, and dropout 0 is the plain stack
    keep0 = flref.dropout_keep(seed, 0, T * B * D * H, p)
    assert 0 < keep0.sum() < keep0.size
    y0, _, _ = flref.rnn_fwd(flref.rnn_desc(I, H, L, bidir, mode, T, B), x, w, hx, cx)
    assert rel_l2(y, y0) > 1e-3


def test_dropout_mask_statistics():
    # keep fraction and independence between layers / seeds of the counter-based mask
    n = 20000
    for p in (0.1, 0.5, 0.8):
        a = flref.dropout_keep(7, 0, n, p)
        b = flref.dropout_keep(7, 1, n, p)
        c = flref.dropout_keep(8, 0, n, p)
        for m in (a, b, c):
            assert abs(m.mean() - (1 - p)) < 4 * np.sqrt(p * (1 - p) / n)
        for u, v in ((a, b), (a, c)):
            both = (u & v).mean()
            assert abs(both - (1 - p) ** 2) < 0.02
        # neighbouring elements are not correlated
        assert abs(np.corrcoef(a[:-1], a[1:])[0, 1]) < 0.03
