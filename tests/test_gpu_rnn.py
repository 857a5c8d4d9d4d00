"""GPU parity of rnn / rnnBackward through the C ABI against oracle/flref.c (which is
pinned against PyTorch's RNN / LSTM / GRU in tests/test_oracle_rnn.py): all four modes,
stacked, bidirectional, with and without initial states and output gradients."""
import numpy as np
import pytest
import torch

from flashlight_amd import ops
from gpu_util import dev, host
from oracle import flref
from refmath import rel_l2

pytestmark = pytest.mark.gpu
MODES = [flref.RNN_RELU, flref.RNN_TANH, flref.RNN_LSTM, flref.RNN_GRU]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("I,H,L,bidir,T,B,states", [
    (2, 2, 2, True, 3, 2, False),          # AutogradRnnTest.cpp:24-31
    (5, 7, 1, False, 6, 3, True),
    (4, 3, 3, True, 5, 2, True),
    (6, 4, 2, False, 1, 4, False),         # one step
    (40, 64, 2, True, 20, 8, True),        # sizes that reach the matrix-core products
    (80, 96, 1, False, 33, 5, False),
    # hidden sizes that are multiples of 16 with at most 64 batch columns take the fused
    # step kernels: one, two and four batch tiles, fewer contraction chunks than waves,
    # a single batch column; 65 columns and the sizes above take the two-kernel steps
    (24, 16, 1, True, 4, 17, True),
    (10, 48, 2, True, 5, 33, True),
    (12, 128, 1, False, 7, 64, False),
    (9, 160, 2, True, 6, 1, True),
    (12, 32, 1, True, 4, 65, True),
    (5, 7, 2, False, 3, 1, True),          # stacked, layer activations of 21 floats (no 16-byte multiple)
    (3, 5, 3, True, 3, 1, False),
])
def test_rnn_forward_backward(mode, I, H, L, bidir, T, B, states):
    rng = np.random.default_rng(1000 * mode + I + H + L + T)
    D = 2 if bidir else 1
    d = flref.rnn_desc(I, H, L, bidir, mode, T, B)
    n = flref.rnn_param_count(d)
    assert ops.rnn_param_count(I, H, L, mode, bidir) == n
    w = (rng.standard_normal(n) / np.sqrt(H)).astype(np.float32)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    hx = rng.standard_normal((L * D, B, H)).astype(np.float32) if states else None
    cx = rng.standard_normal((L * D, B, H)).astype(np.float32) if states and mode == flref.RNN_LSTM else None
    dy = rng.standard_normal((T, B, D * H)).astype(np.float32)
    dhy = rng.standard_normal((L * D, B, H)).astype(np.float32)
    dcy = rng.standard_normal((L * D, B, H)).astype(np.float32) if mode == flref.RNN_LSTM else None
    ry, rhy, rcy = flref.rnn_fwd(d, x, w, hx, cx)
    rdx, rdhx, rdcx, rdw = flref.rnn_bwd(d, x, w, hx, cx, dy, dhy, dcy)

    o = lambda a: None if a is None else dev(a)
    y, hy, cy, reserve = ops.rnn(dev(x), o(hx), o(cx), dev(w), H, L, mode, bidir)
    assert rel_l2(host(y), ry) <= 1e-4 and rel_l2(host(hy), rhy) <= 1e-4
    if mode == flref.RNN_LSTM:
        assert rel_l2(host(cy), rcy) <= 1e-4
    else:
        assert cy is None
    dx, dhx, dcx, dw = ops.rnn_backward(dev(x), dev(w), reserve, H, L, mode, bidir, dev(dy), dev(dhy), o(dcy))
    assert rel_l2(host(dx), rdx) <= 2e-4
    assert rel_l2(host(dhx), rdhx) <= 2e-4
    assert rel_l2(host(dw), rdw) <= 2e-4
    if mode == flref.RNN_LSTM:
        assert rel_l2(host(dcx), rdcx) <= 2e-4


def _random_configs(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        out.append((int(rng.integers(0, 4)), int(rng.integers(1, 70)),
                    int(rng.choice([16, 32, 48, 64, 80, 96, 128, 20, 7])), int(rng.integers(1, 4)),
                    bool(rng.integers(0, 2)), int(rng.integers(1, 9)),
                    int(rng.choice([1, 2, 5, 16, 17, 31, 32, 33, 48, 64, 65, 70])), bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("mode,I,H,L,bidir,T,B,states", _random_configs(30, 11))
def test_random_configurations(mode, I, H, L, bidir, T, B, states):
    """Seeded random sizes around the conditions of the fused step kernels (hidden sizes that
    are / are not multiples of 16, batches around the 16-column tiles and the limit of 64)."""
    test_rnn_forward_backward(mode, I, H, L, bidir, T, B, states)


@pytest.mark.parametrize("mode", [flref.RNN_LSTM, flref.RNN_GRU])
def test_missing_output_gradients_are_zero(mode):
    # only y was differentiated: the closure hands empty dhy / dcy (Functions.cpp:1677-1699)
    rng = np.random.default_rng(7)
    I, H, L, T, B = 6, 5, 2, 4, 3
    d = flref.rnn_desc(I, H, L, True, mode, T, B)
    w = (rng.standard_normal(flref.rnn_param_count(d)) * 0.4).astype(np.float32)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    dy = rng.standard_normal((T, B, 2 * H)).astype(np.float32)
    rdx, rdhx, rdcx, rdw = flref.rnn_bwd(d, x, w, None, None, dy, None, None)
    y, hy, cy, reserve = ops.rnn(dev(x), None, None, dev(w), H, L, mode, True)
    dx, dhx, dcx, dw = ops.rnn_backward(dev(x), dev(w), reserve, H, L, mode, True, dev(dy))
    assert rel_l2(host(dx), rdx) <= 2e-4 and rel_l2(host(dw), rdw) <= 2e-4 and rel_l2(host(dhx), rdhx) <= 2e-4
    # and only the final state differentiated
    dhy = rng.standard_normal((2 * L, B, H)).astype(np.float32)
    rdx, _, _, rdw = flref.rnn_bwd(d, x, w, None, None, None, dhy, None)
    dx, _, _, dw = ops.rnn_backward(dev(x), dev(w), reserve, H, L, mode, True, None, dev(dhy))
    assert rel_l2(host(dx), rdx) <= 2e-4 and rel_l2(host(dw), rdw) <= 2e-4


def test_rnn_errors():
    x = dev(np.zeros((3, 2, 4), np.float32))
    w = dev(np.zeros(ops.rnn_param_count(4, 5, 1, ops.RNN_TANH, False), np.float32))
    with pytest.raises(ValueError):
        ops.rnn(x, None, None, w[:-1], 5, 1, ops.RNN_TANH, False)          # parameter count
    with pytest.raises(ValueError):
        ops.rnn(x, dev(np.zeros((1, 2, 6), np.float32)), None, w, 5, 1, ops.RNN_TANH, False)   # state dims
    with pytest.raises(ValueError):
        ops.rnn(x, None, dev(np.zeros((1, 2, 5), np.float32)), w, 5, 1, ops.RNN_TANH, False)   # cell state without LSTM
    with pytest.raises(ValueError):
        ops.rnn(x, None, None, w, 5, 1, ops.RNN_TANH, False, dropout=1.5)   # not a probability
    y, hy, cy, reserve = ops.rnn(x, None, None, w, 5, 1, ops.RNN_TANH, False)
    with pytest.raises(ValueError):
        ops.rnn_backward(x, w, None, 5, 1, ops.RNN_TANH, False, y)           # no payload


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("I,H,L,bidir,T,B,p", [
    (4, 3, 3, True, 5, 2, 0.5),            # the two-kernel steps
    (10, 48, 2, True, 5, 33, 0.3),         # the fused step kernels
    (40, 64, 3, False, 12, 8, 0.2),
    (5, 7, 2, False, 3, 1, 0.7),
])
def test_rnn_dropout_between_layers(mode, I, H, L, bidir, T, B, p):
    """Dropout on the output sequence of every layer but the last (backend/cudnn/RNN.cpp:83-90):
    same mask (a function of the seed) and scale as the CPU checker, forward and backward;
    another seed gives another result, one layer ignores the setting."""
    rng = np.random.default_rng(2000 * mode + I + H + L + T)
    D = 2 if bidir else 1
    seed = 0xC0FFEE1234567
    d = flref.rnn_desc(I, H, L, bidir, mode, T, B, dropout=p, seed=seed)
    w = (rng.standard_normal(flref.rnn_param_count(d)) / np.sqrt(H)).astype(np.float32)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    hx = rng.standard_normal((L * D, B, H)).astype(np.float32)
    cx = rng.standard_normal((L * D, B, H)).astype(np.float32) if mode == flref.RNN_LSTM else None
    dy = rng.standard_normal((T, B, D * H)).astype(np.float32)
    dhy = rng.standard_normal((L * D, B, H)).astype(np.float32)
    dcy = rng.standard_normal((L * D, B, H)).astype(np.float32) if mode == flref.RNN_LSTM else None
    ry, rhy, rcy = flref.rnn_fwd(d, x, w, hx, cx)
    rdx, rdhx, rdcx, rdw = flref.rnn_bwd(d, x, w, hx, cx, dy, dhy, dcy)

    o = lambda a: None if a is None else dev(a)
    y, hy, cy, reserve = ops.rnn(dev(x), o(hx), o(cx), dev(w), H, L, mode, bidir, dropout=p, seed=seed)
    assert rel_l2(host(y), ry) <= 1e-4 and rel_l2(host(hy), rhy) <= 1e-4
    if mode == flref.RNN_LSTM:
        assert rel_l2(host(cy), rcy) <= 1e-4
    dx, dhx, dcx, dw = ops.rnn_backward(dev(x), dev(w), reserve, H, L, mode, bidir, dev(dy), dev(dhy), o(dcy),
                                        dropout=p, seed=seed)
    assert rel_l2(host(dx), rdx) <= 2e-4
    assert rel_l2(host(dhx), rdhx) <= 2e-4
    assert rel_l2(host(dw), rdw) <= 2e-4
    if mode == flref.RNN_LSTM:
        assert rel_l2(host(dcx), rdcx) <= 2e-4
    y2 = ops.rnn(dev(x), o(hx), o(cx), dev(w), H, L, mode, bidir, dropout=p, seed=seed + 1)[0]
    assert rel_l2(host(y2), ry) > 1e-3
    y3 = ops.rnn(dev(x), o(hx), o(cx), dev(w), H, L, mode, bidir, dropout=p, seed=seed)[0]
    assert torch.equal(y3, y)


def test_rnn_dropout_needs_more_than_one_layer_and_a_valid_probability():
    x = dev(np.zeros((3, 2, 4), np.float32))
    w = dev(np.zeros(ops.rnn_param_count(4, 5, 1, flref.RNN_GRU, False), np.float32))
    a = ops.rnn(x, None, None, w, 5, 1, flref.RNN_GRU, False)[0]
    b = ops.rnn(x, None, None, w, 5, 1, flref.RNN_GRU, False, dropout=0.9, seed=3)[0]
    assert torch.equal(a, b)
    with pytest.raises(ValueError):
        ops.rnn(x, None, None, w, 5, 1, flref.RNN_GRU, False, dropout=1.0)
