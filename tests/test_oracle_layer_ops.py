"""Pins of the CPU oracle for the short convolution and the (gated) RMS norm against library routines and closed forms."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import layer_ops as ol


def test_conv_matches_library_conv1d_and_impulse_response():
    rng = np.random.default_rng(0)
    B, T, D, W = 2, 37, 16, 4
    x, w, b = rng.normal(size=(B, T, D)), rng.normal(size=(D, W)), rng.normal(size=D)
    got = ol.causal_conv1d(x, w, b)
    lib = F.conv1d(torch.from_numpy(x).transpose(1, 2), torch.from_numpy(w)[:, None, :], torch.from_numpy(b),
                   padding=W - 1, groups=D)[..., :T].transpose(1, 2)
    assert np.abs(got - lib.numpy()).max() < 1e-12
    # an impulse at t0 comes out as the taps in reverse order: the last tap sits on the current token
    imp = np.zeros((1, 10, D))
    imp[0, 3] = 1.0
    y = ol.causal_conv1d(imp, w)
    for k in range(W):
        assert np.allclose(y[0, 3 + k], w[:, W - 1 - k])
    assert np.all(y[0, :3] == 0) and np.all(y[0, 3 + W:] == 0)
    # SiLU and residual: library silu, then a plain add
    res = rng.normal(size=(B, T, D))
    act = ol.causal_conv1d(x, w, b, residual=res, activation="silu")
    assert np.abs(act - (F.silu(lib).numpy() + res)).max() < 1e-12


def test_conv_varlen_equals_independent_sequences_and_final_state():
    rng = np.random.default_rng(1)
    D, W = 8, 4
    cu = np.array([0, 5, 5, 7, 30])                                  # includes an empty and a short sequence
    x, w = rng.normal(size=(1, 30, D)), rng.normal(size=(D, W))
    got = ol.causal_conv1d(x, w, activation="swish", cu_seqlens=cu)
    for s in range(len(cu) - 1):
        if cu[s + 1] > cu[s]:
            one = ol.causal_conv1d(x[:, cu[s]:cu[s + 1]], w, activation="swish")
            assert np.array_equal(got[:, cu[s]:cu[s + 1]], one)
    st = ol.conv_final_state(x, W, cu)
    assert st.shape == (4, D, W) and np.all(st[1] == 0)
    assert np.array_equal(st[0], x[0, 1:5].T) and np.array_equal(st[3], x[0, 26:30].T)
    assert np.all(st[2][:, :2] == 0) and np.array_equal(st[2][:, 2:], x[0, 5:7].T)
    dense = ol.conv_final_state(x, W)
    assert np.array_equal(dense[0], x[0, 26:30].T)


def test_rms_norm_matches_library_and_invariants():
    rng = np.random.default_rng(2)
    x, g, w, b = rng.normal(size=(5, 7, 64)), rng.normal(size=(5, 7, 64)), rng.normal(size=64), rng.normal(size=64)
    y, s = ol.rms_norm(x, weight=w, eps=1e-6)
    lib = F.rms_norm(torch.from_numpy(x), (64,), torch.from_numpy(w), eps=1e-6)
    assert np.abs(y - lib.numpy()).max() < 1e-12 and np.array_equal(s, x)
    # unit weight, eps -> 0: rows of unit mean square, invariant to the scale of the input
    y1, _ = ol.rms_norm(x, eps=0.0)
    assert np.allclose((y1 ** 2).mean(-1), 1.0) and np.allclose(ol.rms_norm(3.7 * x, eps=0.0)[0], y1)
    # gate: library silu / sigmoid on g; bias added before the gate; residual added before the norm
    res = rng.normal(size=x.shape)
    yg, sg = ol.rms_norm(x, g, w, b, residual=res, eps=1e-5, activation="swish")
    base = F.rms_norm(torch.from_numpy(x + res), (64,), torch.from_numpy(w), eps=1e-5).numpy() + b
    assert np.abs(yg - base * F.silu(torch.from_numpy(g)).numpy()).max() < 1e-12 and np.array_equal(sg, x + res)
    ys, _ = ol.rms_norm(x, g, w, b, residual=res, eps=1e-5, activation="sigmoid")
    assert np.abs(ys - base * torch.sigmoid(torch.from_numpy(g)).numpy()).max() < 1e-12
